"""``model.save_pretrained(dir, save_compressed=True, quantization_format=None)`` after ``oneshot``.

The reference replaces a model's bound ``save_pretrained`` before calibration
(transformers/compression/compressed_tensors_utils.py:86-190, called from entrypoints/utils.py:96) so that the
call every example ends with writes the compressed-tensors checkpoint: packed weights, ``quantization_config`` in
``config.json``, ``recipe.yaml``.  Here the packed tensors come from the HIP quantise / pack kernel
(``compress_model_state_dict``) and are handed to the model's own writer as ``state_dict``, which keeps its
sharding, tied-weight handling, generation config and custom-code files; the model's modules are left as they are
(the reference compresses them in place and leaves them compressed).
"""
from __future__ import annotations

import json
import os
import weakref
from functools import wraps

import torch

from ...compressors import CompressionFormat, compress_model_state_dict, quantization_config_dict

__all__ = ["modify_save_pretrained"]


def _write_quantization_config(save_directory: str, qcfg: dict):
    path = os.path.join(save_directory, "config.json")
    config = {}
    if os.path.exists(path):
        with open(path, "r") as f:
            config = json.load(f)
    config["quantization_config"] = qcfg
    with open(path, "w") as f:
        json.dump(config, f, indent=2, sort_keys=True)
        f.write("\n")


def _write_recipe(save_directory: str, model_path):
    """``recipe.yaml`` of this session, appended to the one the model was loaded with (if it sits in a
    directory), as the reference's ``update_and_save_recipe`` does."""
    from ...core import active_session

    recipe = active_session().lifecycle.recipe
    if recipe is None or not getattr(recipe, "modifiers", None):
        return
    target = os.path.join(save_directory, "recipe.yaml")
    existing = None
    for candidate in (target, os.path.join(str(model_path), "recipe.yaml") if model_path else None):
        if candidate and os.path.isfile(candidate):
            existing = candidate
            break
    recipe.yaml(file_path=target, existing_recipe_path=existing)


def modify_save_pretrained(model: torch.nn.Module):
    """Wrap ``model.save_pretrained`` once; a model without that method is left alone."""
    bound = getattr(model, "save_pretrained", None)
    if bound is None or getattr(bound, "_overridden", False) or not hasattr(bound, "__func__"):
        return
    model_ref = weakref.ref(model)
    original = bound.__func__
    del bound

    @wraps(original)
    def save_pretrained_wrapper(save_directory, quantization_format=None, save_compressed: bool = True, **kwargs):
        model = model_ref()
        fmt = None if quantization_format is None else str(
            getattr(quantization_format, "value", quantization_format)).replace("_", "-")
        if fmt == CompressionFormat.dense:
            save_compressed, fmt = False, None
        kwargs.setdefault("max_shard_size", "20GB")
        # checked before anything is written: an override that cannot hold a scheme's codes raises here
        qcfg = quantization_config_dict(model, save_compressed, fmt)
        if "state_dict" not in kwargs:
            if qcfg is not None and save_compressed:
                kwargs["state_dict"] = compress_model_state_dict(model, fmt)
            else:
                kwargs["state_dict"] = {k: v for k, v in model.state_dict().items() if "_observer" not in k}
        original(model, save_directory, **kwargs)
        if qcfg is not None:
            _write_quantization_config(str(save_directory), qcfg)
        _write_recipe(str(save_directory), getattr(model, "name_or_path", None))

    save_pretrained_wrapper._overridden = True
    model.save_pretrained = save_pretrained_wrapper
