"""Observer attachment and qparam updates (reference: modifiers/quantization/calibration.py:36-231)."""
from __future__ import annotations

import logging
from collections.abc import Iterable
from itertools import product
from typing import Any

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

_warned = set()


def _warn_once(msg):
    if msg not in _warned:
        _warned.add(msg)
        logger.warning(msg)


def initialize_observer(module: Module, base_name: str):
    """Attach ``<base_name>_observer``; weights always get the memoryless variants."""
    if base_name == "weight":
        arg_name = "weights"
    elif base_name == "output":
        arg_name = "output_activations"
    else:  # input, q, k, v
        arg_name = "input_activations"
    args: QuantizationArgs = getattr_chain(module, f"quantization_scheme.{arg_name}", None)
    observer = args.observer
    if base_name == "weight" and args.observer in ("static_minmax", "minmax"):
        observer = "memoryless_minmax"
        _warn_once(f"Overriding weight observer for lower memory usage ({args.observer} -> {observer})")
    if base_name == "weight" and args.observer in ("mse",):
        observer = "memoryless_mse"
        _warn_once(f"Overriding weight observer for lower memory usage ({args.observer} -> {observer})")
    if args is not None and args.dynamic is not True:
        observer = Observer.load_from_registry(observer, base_name=base_name, args=args)
        module.register_module(f"{base_name}_observer", observer)
        observer.attach(module)


def observe(module: Module | Iterable[Module], base_name: str):
    if isinstance(module, Iterable) and not isinstance(module, Module):
        for m in module:
            observe(m, base_name)
        return
    observer = getattr(module, f"{base_name}_observer", None)
    if observer is None:
        return
    observer(getattr(module, base_name))


def update_qparams(module: Module | Iterable[Module], base_name: str | Iterable[str], only_update_onload: bool = False):
    if (isinstance(module, Iterable) and not isinstance(module, Module)) or not isinstance(base_name, str):
        modules = [module] if isinstance(module, Module) else module
        base_names = [base_name] if isinstance(base_name, str) else base_name
        for m, b in product(list(modules), list(base_names)):
            update_qparams(m, b, only_update_onload=only_update_onload)
        return
    observer = getattr(module, f"{base_name}_observer", None)
    if observer is None:
        return
    if not observer.has_statistics:
        logger.warning(
            f"Attempted to calibrate a module {base_name} without statistics. This is often indicative of a bad "
            "calibration setup, such as not using `moe_calibrate_all_experts` or selecting the wrong calibration "
            "pipeline.")
        return
    args = observer.args
    is_dynamic = getattr(args, "dynamic", False) in (True, DynamicType.LOCAL)
    qparams = observer.get_qparams()
    for param_name, param_val in qparams.items():
        if param_val is None:
            continue
        if is_dynamic and param_name in ("scale", "zero_point"):
            continue
        full = f"{base_name}_{param_name}"
        if hasattr(module, full):
            if not only_update_onload:
                update_offload_parameter(module, full, param_val)
            else:
                getattr(module, full).data = param_val


def calibrate_input_hook(module: Module, args: Any):
    args = args[0] if isinstance(args, tuple) else args
    module.input_observer(args)


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
    if not getattr(module, "quantization_scheme", None):
        return
    module.quantization_status = QuantizationStatus.CALIBRATION


def freeze_module_quantization(module: Module):
    if not getattr(module, "quantization_scheme", None):
        return
    if module.quantization_status == QuantizationStatus.FROZEN:
        return
    for name in ("input", "weight", "output", "q", "k", "v"):
        obs_name = f"{name}_observer"
        if hasattr(module, obs_name):
            getattr(module, obs_name).detach(module)
            delattr(module, obs_name)
    module.quantization_status = QuantizationStatus.FROZEN


def reset_quantization_status(model: Module):
    for module in model.modules():
        if hasattr(module, "quantization_status"):
            delattr(module, "quantization_status")
