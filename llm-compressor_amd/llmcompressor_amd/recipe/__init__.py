"""Recipe: ``<stage>_stage: <group>_modifiers: <ModifierClass>: {args}`` (reference: recipe/recipe.py:87-285)."""
from __future__ import annotations

import json
import os
import re
from typing import Any, Dict, List, Optional, Union

import yaml
from pydantic import BaseModel, ConfigDict, Field

__all__ = ["Recipe"]


def _load_json_or_yaml_string(content: str) -> dict:
    try:
        return json.loads(content)
    except json.JSONDecodeError:
        try:
            obj = yaml.safe_load(content)
        except yaml.YAMLError as err:
            raise ValueError(f"Could not parse recipe from string {content}") from err
        if not isinstance(obj, dict):
            raise ValueError(f"Could not parse recipe from string {content}")
        return obj


def _parse_recipe_from_md(file_path: str, yaml_str: str) -> str:
    front = re.compile(r"^-+\n(.*?)\n-+", re.DOTALL)
    m = front.search(yaml_str)
    if not m:
        raise RuntimeError(f"Could not extract YAML front matter from recipe card: {file_path}")
    return m.group(1)


def _filter_dict(obj: dict, target_stage: Optional[str]) -> dict:
    if target_stage is None:
        return obj
    return {k: v for k, v in obj.items() if not k.endswith("_stage") or k == target_stage}


class Recipe(BaseModel):
    model_config = ConfigDict(arbitrary_types_allowed=True)

    args: Dict[str, Any] = Field(default_factory=lambda: {})
    stage: str = "default"
    modifiers: List[Any] = Field(default_factory=list)

    @classmethod
    def from_modifiers(cls, modifiers, modifier_group_name: Optional[str] = None) -> "Recipe":
        from ..modifiers import Modifier

        def leaves(x):
            if isinstance(x, (list, tuple)):
                out = []
                for y in x:
                    out.extend(leaves(y))
                return out
            return [x]

        mods = leaves(modifiers)
        if any(not isinstance(m, Modifier) for m in mods):
            raise ValueError("modifiers must be a list of Modifier instances")
        return cls(stage=modifier_group_name or "default", modifiers=mods)

    @classmethod
    def create_instance(cls, path_or_modifiers, modifier_group_name: Optional[str] = None,
                        target_stage: Optional[str] = None) -> "Recipe":
        from ..modifiers import Modifier

        if isinstance(path_or_modifiers, Recipe):
            return path_or_modifiers
        if isinstance(path_or_modifiers, (Modifier, list)):
            return cls.from_modifiers(path_or_modifiers, modifier_group_name)
        if not os.path.isfile(path_or_modifiers):
            return cls.from_dict(_filter_dict(_load_json_or_yaml_string(path_or_modifiers), target_stage))
        with open(path_or_modifiers, "r") as f:
            content = f.read().strip()
        low = path_or_modifiers.lower()
        if low.endswith(".md"):
            content = _parse_recipe_from_md(path_or_modifiers, content)
        if low.endswith(".json"):
            obj = json.loads(content)
        elif low.endswith((".yaml", ".yml")):
            obj = yaml.safe_load(content)
        else:
            try:
                obj = _load_json_or_yaml_string(content)
            except ValueError:
                raise ValueError(f"Could not parse recipe from path {path_or_modifiers}")
        return cls.from_dict(_filter_dict(obj, target_stage))

    @classmethod
    def from_dict(cls, recipe_dict: dict) -> "Recipe":
        from ..modifiers import ModifierFactory

        args = recipe_dict.get("args", {})
        modifiers, stage = [], "default"
        for stage_key, stage_val in recipe_dict.items():
            if stage_key.endswith("_stage") and isinstance(stage_val, dict):
                stage = stage_key.replace("_stage", "")
                for group_key, group_val in stage_val.items():
                    if group_key.endswith("_modifiers") and isinstance(group_val, dict):
                        inferred = group_key.replace("_modifiers", "")
                        for mod_type, mod_args in group_val.items():
                            mod_args = dict(mod_args or {})
                            group = mod_args.pop("group", inferred)
                            modifiers.append(ModifierFactory.create(mod_type, group=group, allow_registered=True,
                                                                    allow_experimental=True, **mod_args))
        return cls(args=args, stage=stage, modifiers=modifiers)

    def dict(self, *args, **kwargs) -> dict:
        stage_dict: dict = {}
        for mod in self.modifiers:
            group = f"{mod.group or 'default'}_modifiers"
            d = mod.model_dump(mode="json", exclude_unset=True)
            d.pop("group", None)
            d.pop("index", None)
            stage_dict.setdefault(group, {})[mod.__class__.__name__] = d
        return {f"{self.stage}_stage": stage_dict}

    def yaml(self, file_path: Optional[str] = None, existing_recipe_path: Optional[str] = None) -> str:
        existing = {}
        if existing_recipe_path:
            with open(existing_recipe_path, "r") as f:
                existing = _load_json_or_yaml_string(f.read())
        merged = dict(existing)
        for k, v in self.dict().items():
            key = k
            n = 0
            while key in merged:  # keep both recipes: suffix the stage name
                n += 1
                key = k.replace("_stage", f"_{n}_stage")
            merged[key] = v
        text = yaml.dump(merged, allow_unicode=True, sort_keys=False, default_flow_style=None, width=88)
        if file_path is not None:
            with open(file_path, "w") as f:
                f.write(text)
        return text
