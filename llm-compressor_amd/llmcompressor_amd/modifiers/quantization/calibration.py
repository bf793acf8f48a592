"""Observer attachment and qparam updates (reference: modifiers/quantization/calibration.py:36-231).

The public names and their behaviour are the reference's; the observers they attach run the HIP min-max / MSE
kernels (``llmcompressor_amd.observers``).
"""
from __future__ import annotations

import logging
from typing import Any, Iterable, Iterator

import torch
from torch.nn import Module

from ...observers import Observer
from ...quantization import (
    DynamicType,
    QuantizationArgs,
    QuantizationStatus,
    forward_quantize,
    getattr_chain,
    update_offload_parameter,
)

logger = logging.getLogger("llmcompressor_amd")

__all__ = [
    "initialize_observer",
    "observe",
    "update_qparams",
    "calibrate_input_hook",
    "calibrate_output_hook",
    "freeze_module_quantization",
    "apply_calibration_status",
    "reset_quantization_status",
    "calibrate_query_hook",
    "calibrate_key_hook",
    "calibrate_value_hook",
]

# which part of a scheme describes an observed value; q / k / v of an attention module share the input arguments
_SCHEME_FIELD = {"weight": "weights", "output": "output_activations", "input": "input_activations",
                 "q": "input_activations", "k": "input_activations", "v": "input_activations"}
# weight observers never need history: a weight is observed once, so the running variants only cost memory
_MEMORYLESS = {"static_minmax": "memoryless_minmax", "minmax": "memoryless_minmax", "mse": "memoryless_mse"}
_OBSERVED = tuple(_SCHEME_FIELD)

_warned = set()


def _warn_once(msg):
    if msg not in _warned:
        _warned.add(msg)
        logger.warning(msg)


def _modules_of(target) -> Iterator[Module]:
    """One module, or every module of an iterable (an ``nn.ModuleList`` counts as one module)."""
    if isinstance(target, Module):
        yield target
    else:
        yield from target


def initialize_observer(module: Module, base_name: str):
    """Attach ``<base_name>_observer`` as the scheme asks; nothing for fully dynamic arguments."""
    args: QuantizationArgs = getattr_chain(module, f"quantization_scheme.{_SCHEME_FIELD[base_name]}", None)
    name = args.observer
    if base_name == "weight" and name in _MEMORYLESS:
        name = _MEMORYLESS[name]
        _warn_once(f"Overriding weight observer for lower memory usage ({args.observer} -> {name})")
    if args.dynamic is True:
        return
    observer = Observer.load_from_registry(name, base_name=base_name, args=args)
    module.register_module(f"{base_name}_observer", observer)
    observer.attach(module)


def observe(module: Module | Iterable[Module], base_name: str):
    """Show ``module.<base_name>`` (normally the weight) to its observer, for one module or many."""
    for m in _modules_of(module):
        observer = getattr(m, f"{base_name}_observer", None)
        if observer is not None:
            observer(getattr(m, base_name))


def update_qparams(module: Module | Iterable[Module], base_name: str | Iterable[str], only_update_onload: bool = False):
    """Turn the observers' statistics into ``<base_name>_scale`` / ``_zero_point`` / ``_global_scale``."""
    names = (base_name,) if isinstance(base_name, str) else tuple(base_name)
    for m in list(_modules_of(module)):
        for name in names:
            _update_one(m, name, only_update_onload)


def _update_one(module: Module, base_name: str, only_update_onload: bool):
    observer = getattr(module, f"{base_name}_observer", None)
    if observer is None:
        return
    if not observer.has_statistics:
        logger.warning(
            f"Attempted to calibrate a module {base_name} without statistics. This is often indicative of a bad "
            "calibration setup, such as not using `moe_calibrate_all_experts` or selecting the wrong calibration "
            "pipeline.")
        return
    # dynamic and local arguments keep only the global scale: their scales come from each call's values
    keep_only_global = getattr(observer.args, "dynamic", False) in (True, DynamicType.LOCAL)
    for key, value in observer.get_qparams().items():
        target = f"{base_name}_{key}"
        if value is None or (keep_only_global and key != "global_scale") or not hasattr(module, target):
            continue
        if only_update_onload:
            getattr(module, target).data = value
        else:
            update_offload_parameter(module, target, value)


def calibrate_input_hook(module: Module, args: Any):
    module.input_observer(args[0] if isinstance(args, tuple) else args)


def calibrate_output_hook(module: Module, _args: Any, output: torch.Tensor):
    module.output_observer(output)
    return forward_quantize(module=module, value=output, base_name="output",
                            args=module.quantization_scheme.output_activations)


def calibrate_query_hook(module: Module, query_states: torch.Tensor):
    module.q_observer(query_states)


def calibrate_key_hook(module: Module, key_states: torch.Tensor):
    module.k_observer(key_states)


def calibrate_value_hook(module: Module, value_states: torch.Tensor):
    module.v_observer(value_states)


def apply_calibration_status(module: Module):
    if getattr(module, "quantization_scheme", None):
        module.quantization_status = QuantizationStatus.CALIBRATION


def freeze_module_quantization(module: Module):
    """Drop the observers and mark the module frozen (idempotent)."""
    if not getattr(module, "quantization_scheme", None) or module.quantization_status == QuantizationStatus.FROZEN:
        return
    for base_name in _OBSERVED:
        attr = f"{base_name}_observer"
        observer = getattr(module, attr, None)
        if observer is not None:
            observer.detach(module)
            delattr(module, attr)
    module.quantization_status = QuantizationStatus.FROZEN


def reset_quantization_status(model: Module):
    for module in model.modules():
        if hasattr(module, "quantization_status"):
            delattr(module, "quantization_status")
