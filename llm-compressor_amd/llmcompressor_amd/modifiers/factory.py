"""Name -> Modifier class registry (reference: modifiers/factory.py:74-189)."""
from __future__ import annotations

from typing import Dict, Type

from .modifier import Modifier

__all__ = ["ModifierFactory"]


class ModifierFactory:
    _registered_registry: Dict[str, Type[Modifier]] = {}
    _main_registry: Dict[str, Type[Modifier]] = {}
    _loaded = False

    @staticmethod
    def refresh():
        from .gptq.base import GPTQModifier
        from .pruning.sparsegpt.base import SparseGPTModifier
        from .quantization.quantization.base import QuantizationModifier

        ModifierFactory._main_registry = {c.__name__: c for c in (GPTQModifier, QuantizationModifier,
                                                                  SparseGPTModifier)}
        ModifierFactory._loaded = True

    @staticmethod
    def create(type_: str, allow_registered: bool = True, allow_experimental: bool = True, **kwargs) -> Modifier:
        if not ModifierFactory._loaded:
            ModifierFactory.refresh()
        if allow_registered and type_ in ModifierFactory._registered_registry:
            return ModifierFactory._registered_registry[type_](**kwargs)
        if type_ in ModifierFactory._main_registry:
            return ModifierFactory._main_registry[type_](**kwargs)
        raise ValueError(f"No modifier of type '{type_}' found.")

    @staticmethod
    def register(type_: str, modifier_class: Type[Modifier]):
        if not issubclass(modifier_class, Modifier):
            raise ValueError("The provided class does not subclass the Modifier base class.")
        if not isinstance(type_, str):
            raise ValueError("The provided registry type {type_} must be a string")
        ModifierFactory._registered_registry[type_] = modifier_class
