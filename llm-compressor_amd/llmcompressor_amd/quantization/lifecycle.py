"""Module-level quantization lifecycle and the tensor-level numerics entry points.

Mirrors what the reference imports from compressed-tensors: ``apply_quantization_config``,
``initialize_module_for_quantization``, ``match_named_modules``, ``is_module_quantized``,
``enable_quantization`` / ``disable_quantization``, ``update_offload_parameter``,
``calculate_qparams``, ``generate_gparam``, ``fake_quantize`` / ``quantize`` and
``forward_quantize`` (call sites: ``modifiers/quantization/quantization/mixin.py:222-272``,
``modifiers/quantization/calibration.py:36-196``, ``observers/base.py:78-123``,
``modifiers/gptq/gptq_quantize.py:184-225``).  Every numeric function here is a thin
dispatcher onto the HIP kernels (``llmcompressor_amd.ops``); none has a torch fallback.
"""
from __future__ import annotations

import math
import re
from typing import Iterable, Iterator, Optional, Tuple

import torch
from torch.nn import Module, Parameter

from .. import ops
from ..torch_ops import llmc
from .quant_args import (
    ActivationOrdering,
    DynamicType,
    QuantizationArgs,
    QuantizationConfig,
    QuantizationScheme,
    QuantizationStatus,
    QuantizationStrategy,
    QuantizationType,
)

__all__ = [
    "match_named_modules",
    "apply_quantization_config",
    "initialize_module_for_quantization",
    "initialize_qparams",
    "is_module_quantized",
    "enable_quantization",
    "disable_quantization",
    "update_offload_parameter",
    "calculate_qparams",
    "generate_gparam",
    "fake_quantize",
    "quantize",
    "forward_quantize",
    "kernel_format",
    "scale_indexing",
    "effective_scale",
    "getattr_chain",
]

_SENTINEL = object()
BIG = 1 << 40


def getattr_chain(obj, chain: str, default=_SENTINEL):
    cur = obj
    for name in chain.split("."):
        if not hasattr(cur, name):
            if default is _SENTINEL:
                raise AttributeError(f"{chain} not found on {obj}")
            return default
        cur = getattr(cur, name)
    return cur


def _match_one(name: str, module: Module, target: str) -> bool:
    if target.startswith("re:"):
        return re.match(target[3:], name) is not None
    if name == target or name.endswith("." + target):
        return True
    return any(cls.__name__ == target for cls in type(module).__mro__)


def match_named_modules(model: Module, targets: Iterable[str], ignore: Iterable[str] = ()) -> Iterator[Tuple[str, Module]]:
    """(name, module) for modules whose class name, full name, name suffix or ``re:`` pattern is targeted."""
    targets, ignore = list(targets or []), list(ignore or [])
    for name, module in model.named_modules():
        if not any(_match_one(name, module, t) for t in targets):
            continue
        if any(_match_one(name, module, i) for i in ignore):
            continue
        yield name, module


def is_module_quantized(module: Module) -> bool:
    scheme = getattr(module, "quantization_scheme", None)
    if scheme is None:
        return False
    return any(a is not None for a in (scheme.weights, scheme.input_activations, scheme.output_activations))


def enable_quantization(module: Module):
    module.quantization_enabled = True


def disable_quantization(module: Module):
    module.quantization_enabled = False


def update_offload_parameter(module: Module, name: str, data: torch.Tensor):
    """Copy ``data`` into the module's parameter (creating it when the checkpoint layout adds one)."""
    param = getattr(module, name, None)
    if isinstance(param, (Parameter, torch.Tensor)) and param.shape == data.shape:
        with torch.no_grad():
            if param.dtype == data.dtype:
                param.data.copy_(data)
            else:
                param.data = data.to(param.dtype) if _castable(data, param.dtype) else data
    else:
        module.register_parameter(name, Parameter(data, requires_grad=False))


def _castable(data, dtype):
    return True


# --------------------------------------------------------------------------- kernel dispatch helpers


def kernel_format(args: QuantizationArgs) -> Tuple[int, int]:
    if args.type == QuantizationType.INT:
        return ops.FMT_INT, args.num_bits
    if args.num_bits == 8:
        return ops.FMT_FP8, 8
    if args.num_bits == 4:
        return ops.FMT_FP4, 4
    raise ValueError(f"unsupported float width {args.num_bits}")


def scale_mode(args: QuantizationArgs, with_global: bool) -> int:
    if args.is_mx:
        return ops.SCALE_MXFP4
    if args.strategy == QuantizationStrategy.TENSOR_GROUP and args.scale_dtype is not None and with_global:
        return ops.SCALE_NVFP4
    return ops.SCALE_PLAIN


def scale_indexing(args: QuantizationArgs, rows: int, cols: int) -> Tuple[int, int, int]:
    """(row_div, scale_row_stride, col_div) of llmc_quantize for an [rows, cols] value."""
    s = args.strategy
    if s == QuantizationStrategy.TENSOR:
        return BIG, 0, BIG
    if s in (QuantizationStrategy.CHANNEL, QuantizationStrategy.TOKEN):
        return 1, 1, BIG
    if s in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
        return 1, math.ceil(cols / args.group_size), args.group_size
    if s == QuantizationStrategy.BLOCK:
        bh, bw = args.block_structure
        return bh, math.ceil(cols / bw), bw
    raise ValueError(f"unsupported strategy {s}")


def effective_scale(scale: torch.Tensor, args: QuantizationArgs, like: torch.dtype) -> torch.Tensor:
    """The scale the kernels divide by: E8M0 codes -> 2^(e-127); e4m3 storage -> fp32."""
    if scale.dtype == torch.uint8:
        return torch.pow(2.0, scale.to(torch.float32) - 127.0).to(like if like != torch.float32 else torch.bfloat16)
    if scale.dtype == torch.float8_e4m3fn:
        return scale.to(torch.float32)
    return scale


def calculate_qparams(min_vals, max_vals, quantization_args: QuantizationArgs, global_scale=None):
    """-> (scale, zero_point).  NVFP4: scale holds e4m3-grid values in fp32; MXFP4: E8M0 codes (uint8)."""
    fmt, bits = kernel_format(quantization_args)
    mode = scale_mode(quantization_args, global_scale is not None)
    if mode == ops.SCALE_MXFP4 and min_vals.dtype != torch.bfloat16:
        # the shared exponent is read off the bf16 bit pattern of the group maximum; for statistics of another
        # dtype the rule is undefined (compressed-tensors asserts bf16 there), so nothing is guessed
        raise TypeError(f"MXFP4 scales are defined on bfloat16 statistics; got {min_vals.dtype}. Cast the weights "
                        "to bfloat16 or choose another scheme.")
    scale, zp, codes = llmc.qparams(
        min_vals, max_vals, fmt, bits, bool(quantization_args.symmetric), mode,
        global_scale if mode == ops.SCALE_NVFP4 else None, mode == ops.SCALE_MXFP4)
    if mode == ops.SCALE_MXFP4:
        scale = codes
    if scale.ndim == 0:
        scale, zp = scale.reshape(1), zp.reshape(1)
    zp_dtype = quantization_args.zp_dtype or torch.int8
    if zp_dtype != torch.int8:
        zp = zp.to(zp_dtype) if quantization_args.symmetric else zp
    return scale, zp


def generate_gparam(stats) -> torch.Tensor:
    """stats: list of (min_vals, max_vals) over a fused group -> fp32 [1] global scale."""
    return llmc.global_scale([mn for mn, _ in stats], [mx for _, mx in stats])


def _as_2d(x: torch.Tensor):
    if x.ndim == 1:
        return x.unsqueeze(0), x.shape
    if x.ndim == 2:
        return x, x.shape
    return x.reshape(-1, x.shape[-1]), x.shape


def _run_quantize(x, scale, zero_point, args: QuantizationArgs, out_mode, g_idx=None, global_scale=None):
    fmt, bits = kernel_format(args)
    x2, shape = _as_2d(x.contiguous() if not x.is_contiguous() else x)
    rows, cols = x2.shape
    row_div, srow, col_div = scale_indexing(args, rows, cols)
    if args.strategy == QuantizationStrategy.TENSOR and scale.numel() != 1:
        raise ValueError("tensor strategy expects a single scale")
    es = effective_scale(scale, args, x.dtype)
    zp = None
    if zero_point is not None and not args.symmetric:
        zp = zero_point.to(torch.int8)
    out = llmc.quant_pack(x2, es, zp, fmt, bits, row_div, srow, col_div, out_mode, g_idx, global_scale)
    if out_mode == ops.OUT_PACKED:
        return out
    return out.reshape(shape)


def fake_quantize(x, scale, zero_point, args: QuantizationArgs, g_idx=None, global_scale=None):
    """quantise then dequantise (same rounding points as the eager op chain of the reference)."""
    return _run_quantize(x, scale, zero_point, args, ops.OUT_FAKEQUANT, g_idx, global_scale)


def quantize(x, scale, zero_point, args: QuantizationArgs, dtype=None, g_idx=None, global_scale=None):
    """codes: int8 for integer formats, float8_e4m3fn for fp8, e2m1 nibble index (uint8) for fp4."""
    return _run_quantize(x, scale, zero_point, args, ops.OUT_CODES, g_idx, global_scale)


def forward_quantize(module: Module, value: torch.Tensor, base_name: str, args: QuantizationArgs):
    """fake-quantise an activation / weight with the module's (or dynamic) qparams."""
    if value.numel() == 0:
        return value
    if args.dynamic is True and args.strategy == QuantizationStrategy.TOKEN:
        fmt, bits = kernel_format(args)
        x2, shape = _as_2d(value)
        x2 = x2.contiguous()
        if args.symmetric and bits == 8:  # the fused kernel: row absmax, scale and fake-quant in one pass
            out, _ = llmc.fp8_dynamic_per_token(x2, fmt, bits)
            return out.reshape(shape)
        # other widths and asymmetric ranges: row min/max, qparams and fake-quant as separate kernels
        mn, mx = llmc.minmax_observe(x2, x2.shape[1])
        scale, zp = calculate_qparams(mn, mx, args)
        return fake_quantize(x2, scale, zp, args).reshape(shape)
    scale = getattr(module, f"{base_name}_scale", None)
    zp = getattr(module, f"{base_name}_zero_point", None)
    gs = getattr(module, f"{base_name}_global_scale", None)
    if args.dynamic in (True, DynamicType.LOCAL):
        # scales of this call's values (compressed-tensors ``compute_dynamic_scales_and_zp``): one per run of
        # group_size trailing elements, or one for the whole tensor; ``local`` keeps the calibrated global scale
        x2, shape = _as_2d(value if value.is_contiguous() else value.contiguous())
        rows, cols = x2.shape
        if args.strategy in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
            if cols % args.group_size != 0:
                raise ValueError(f"dynamic group quantization: last dimension {cols} is not a multiple of the "
                                 f"group size {args.group_size}")
            mn, mx = llmc.minmax_observe(x2, args.group_size)
        elif args.strategy == QuantizationStrategy.TENSOR:
            # one group holding every element: the split reduction of the row kernels fills the chip
            mn, mx = llmc.minmax_observe(x2.reshape(1, -1), rows * cols)
            mn, mx = mn.reshape(1), mx.reshape(1)
        else:
            raise ValueError(f"dynamic quantization does not support {args.strategy}")
        scale, zp = calculate_qparams(mn, mx, args, global_scale=gs)
        return fake_quantize(x2, scale, zp, args, global_scale=gs).reshape(shape)
    g_idx = getattr(module, f"{base_name}_g_idx", None)
    if g_idx is not None and bool((g_idx < 0).any()):
        g_idx = None
    return fake_quantize(value, scale, zp, args, g_idx=g_idx, global_scale=gs)


# --------------------------------------------------------------------------- module initialisation


def _qparam_shape(args: QuantizationArgs, observed_shape) -> Tuple[int, ...]:
    s = args.strategy
    if s == QuantizationStrategy.TENSOR:
        return (1,)
    if s == QuantizationStrategy.TOKEN:
        return (1, 1)
    if s == QuantizationStrategy.CHANNEL:
        return (observed_shape[-2], 1)
    if s in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
        ng = math.ceil(observed_shape[-1] / args.group_size)
        return (*observed_shape[:-1], ng) if len(observed_shape) > 1 else (ng,)
    if s == QuantizationStrategy.BLOCK:
        bh, bw = args.block_structure
        return (math.ceil(observed_shape[-2] / bh), math.ceil(observed_shape[-1] / bw))
    if s == QuantizationStrategy.ATTN_HEAD:
        return (observed_shape[-2], 1, 1) if len(observed_shape) >= 2 else (1,)
    raise ValueError(f"unsupported strategy {s}")


def initialize_qparams(module: Module, base_name: str, args: QuantizationArgs, observed_shape,
                       observed_dtype: torch.dtype, force_zero_point: bool = True):
    """Register ``<base>_scale`` / ``_zero_point`` (/ ``_global_scale`` / ``_g_idx``) parameters."""
    if args.dynamic is True:
        return
    device = next(module.parameters(), torch.empty(0)).device
    if base_name == "weight":
        shape = _qparam_shape(args, observed_shape)
    else:
        # activations: only the trailing dims determine the parameter shape
        if args.strategy in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
            shape = (math.ceil(observed_shape[-1] / args.group_size),)
        elif args.strategy == QuantizationStrategy.ATTN_HEAD:
            shape = (observed_shape[-2], 1, 1)
        else:
            shape = (1,)
    if args.strategy == QuantizationStrategy.TENSOR_GROUP:
        module.register_parameter(f"{base_name}_global_scale",
                                  Parameter(torch.empty(1, dtype=torch.float32, device=device), requires_grad=False))
    if args.dynamic is False:
        scale_dtype = args.scale_dtype if args.scale_dtype is not None else observed_dtype
        if scale_dtype not in (torch.float16, torch.bfloat16, torch.float32, torch.float64,
                               torch.float8_e4m3fn, torch.uint8):
            scale_dtype = torch.bfloat16
        module.register_parameter(f"{base_name}_scale",
                                  Parameter(torch.empty(shape, dtype=scale_dtype, device=device), requires_grad=False))
        if force_zero_point or not args.symmetric:
            zp_dtype = args.zp_dtype or torch.int8
            module.register_parameter(
                f"{base_name}_zero_point",
                Parameter(torch.zeros(shape, dtype=zp_dtype, device=device), requires_grad=False))
    if base_name == "weight" and args.actorder is not None and args.actorder == ActivationOrdering.GROUP:
        module.register_parameter(
            "weight_g_idx",
            Parameter(torch.full((observed_shape[-1],), -1, dtype=torch.int32, device=device), requires_grad=False))


def _wrapped_forward(module: Module):
    original = module.forward.__func__ if hasattr(module.forward, "__func__") else None

    def forward(self, *args, **kwargs):
        scheme: Optional[QuantizationScheme] = getattr(self, "quantization_scheme", None)
        enabled = getattr(self, "quantization_enabled", True)
        status = getattr(self, "quantization_status", None)
        if scheme is None or not enabled or status == QuantizationStatus.COMPRESSED:
            return original(self, *args, **kwargs)
        inp = args[0]
        if scheme.input_activations is not None and (
            scheme.input_activations.dynamic in (True, DynamicType.LOCAL) or hasattr(self, "input_scale")
        ) and status in (QuantizationStatus.CALIBRATION, QuantizationStatus.FROZEN):
            inp = forward_quantize(self, inp, "input", scheme.input_activations)
        if scheme.weights is not None and status in (QuantizationStatus.CALIBRATION, QuantizationStatus.FROZEN):
            saved = self.weight.data
            self.weight.data = forward_quantize(self, saved, "weight", scheme.weights)
            try:
                out = original(self, inp, *args[1:], **kwargs)
            finally:
                self.weight.data = saved
        else:
            out = original(self, inp, *args[1:], **kwargs)
        if scheme.output_activations is not None and (
            scheme.output_activations.dynamic in (True, DynamicType.LOCAL) or hasattr(self, "output_scale")
        ) and status in (
            QuantizationStatus.CALIBRATION, QuantizationStatus.FROZEN
        ):
            out = forward_quantize(self, out, "output", scheme.output_activations)
        return out

    return forward if original is not None else None


def initialize_module_for_quantization(module: Module, scheme: Optional[QuantizationScheme] = None,
                                       force_zero_point: bool = True):
    scheme = scheme or getattr(module, "quantization_scheme", None)
    if scheme is None:
        return
    module.quantization_scheme = scheme
    weight = getattr(module, "weight", None)
    if scheme.input_activations is not None and weight is not None:
        initialize_qparams(module, "input", scheme.input_activations, (1, weight.shape[-1]), weight.dtype,
                           force_zero_point)
    if scheme.weights is not None and weight is not None:
        initialize_qparams(module, "weight", scheme.weights, tuple(weight.shape), weight.dtype, force_zero_point)
    if scheme.output_activations is not None and weight is not None:
        initialize_qparams(module, "output", scheme.output_activations, (1, weight.shape[0]), weight.dtype,
                           force_zero_point)
    module.quantization_status = QuantizationStatus.INITIALIZED
    module.quantization_enabled = True
    if not getattr(module, "_llmc_forward_wrapped", False):
        fwd = _wrapped_forward(module)
        if fwd is not None:
            module.forward = fwd.__get__(module, type(module))
            module._llmc_forward_wrapped = True


def apply_quantization_config(model: Module, config: QuantizationConfig):
    """Attach each config group's scheme to the modules it targets (later groups do not override)."""
    ignore = config.ignore or []
    for scheme in config.config_groups.values():
        if not isinstance(scheme, QuantizationScheme):
            continue
        for _, module in match_named_modules(model, scheme.targets, ignore):
            if getattr(module, "quantization_scheme", None) is not None:
                continue
            initialize_module_for_quantization(module, scheme)
    model.quantization_config = config
