"""Oracle: number-format arithmetic (qparams, rounding, fake-quant).

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Restates compressed-tensors' ``quantization/utils/helpers.py``
(``calculate_qparams``, ``generate_gparam``, ``calculate_range``,
``compute_dynamic_scales_and_zp``), ``quantization/utils/mxfp4_utils.py`` and
``quantization/lifecycle/forward.py`` (``fake_quantize`` / ``quantize`` /
``dequantize``) as called from the reference at
``src/llmcompressor/observers/base.py:96,114-119``,
``src/llmcompressor/observers/mse_quant.py:268-280`` and
``src/llmcompressor/modifiers/gptq/gptq_quantize.py:184-225``.

All arithmetic is eager torch on CPU so every intermediate is rounded to the
tensor dtype after each op, exactly like the reference's eager op chain.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, replace
from typing import Optional

import torch

FP8_MAX = 448.0
FP4_MAX = 6.0
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


@dataclass
class QArgs:
    """Plain stand-in for compressed-tensors ``QuantizationArgs`` (field names kept)."""

    num_bits: int = 8
    type: str = "int"  # "int" | "float"
    symmetric: bool = True
    group_size: Optional[int] = None
    strategy: Optional[str] = None  # tensor|channel|group|tensor_group|block|token
    block_structure: Optional[list] = None
    dynamic: object = False  # False | True | "local"
    actorder: Optional[str] = None  # None | "weight" | "group"
    scale_dtype: Optional[torch.dtype] = None
    zp_dtype: Optional[torch.dtype] = None
    observer: Optional[str] = "minmax"
    observer_kwargs: dict = field(default_factory=dict)

    def __post_init__(self):
        if self.strategy is None:
            if self.group_size is None:
                self.strategy = "tensor"
            elif self.group_size > 0:
                self.strategy = "group"
            elif self.group_size == -1:
                self.strategy = "channel"
        if self.zp_dtype is None:
            if self.type == "int":
                self.zp_dtype = torch.int8 if self.num_bits <= 8 else torch.int32
            elif self.num_bits == 8:
                self.zp_dtype = torch.float8_e4m3fn
            else:
                self.zp_dtype = torch.float8_e4m3fn

    def copy(self, **kw) -> "QArgs":
        return replace(self, **kw)

    @property
    def is_fp4(self) -> bool:
        return self.type == "float" and self.num_bits == 4

    @property
    def is_mx(self) -> bool:
        # MXFP4: e2m1 elements, 32-wide groups, power-of-two scales stored as uint8
        return self.is_fp4 and self.scale_dtype == torch.uint8


def calculate_range(args: QArgs):
    """(q_min, q_max) as Python floats; CT ``calculate_range``."""
    if args.type == "int":
        half = 2 ** (args.num_bits - 1)
        return float(-half), float(half - 1)
    if args.num_bits == 8:
        return -FP8_MAX, FP8_MAX
    if args.num_bits == 4:
        return -FP4_MAX, FP4_MAX
    raise ValueError("unsupported float width")


def _dtype_eps(dtype: torch.dtype) -> float:
    if dtype == torch.float8_e4m3fn:
        return 0.125
    if dtype.is_floating_point:
        return torch.finfo(dtype).eps
    return 1.0


def round_to_dtype(t: torch.Tensor, dtype: torch.dtype, cast_back: bool = True):
    """clamp to ``dtype``'s range, round (RNE) into it, optionally cast back."""
    orig = t.dtype
    if dtype.is_floating_point:
        fi = torch.finfo(dtype)
        r = torch.clamp(t, fi.min, fi.max).to(dtype)
    else:
        ii = torch.iinfo(dtype)
        r = torch.round(torch.clamp(t, ii.min, ii.max)).to(dtype)
    return r.to(orig) if cast_back else r


def mxfp4_scale_exponent(absmax: torch.Tensor) -> torch.Tensor:
    """E8M0 biased exponent for an MXFP4 group (parity unpinned).

    Follows compressed-tensors ``generate_mxfp4_scales``: the bf16 bit pattern
    of the group's absmax gets a rounding bump of half of the e2m1 mantissa
    step, the mantissa is masked off (power of two), then
    ``127 + floor(log2(.)) - 2`` (2 = emax of e2m1).
    """
    x = absmax.to(torch.bfloat16).view(torch.int16).to(torch.int32) & 0xFFFF
    bump = 1 << (7 - 1 - 1)
    mask = ((1 << 9) - 1) << 7
    p2 = ((x + bump) & mask).to(torch.int16).view(torch.bfloat16)
    return 127 + torch.floor(torch.log2(p2.to(torch.float32))) - 2


def mxfp4_scale_from_exponent(e: torch.Tensor, dtype=torch.bfloat16):
    return (2.0 ** (e.to(torch.int32) - 127).to(torch.float32)).to(dtype)


def calculate_qparams(min_vals, max_vals, args: QArgs, global_scale=None):
    """Scale and zero-point from observed min/max (CT ``calculate_qparams``)."""
    min_vals = torch.min(min_vals, torch.zeros_like(min_vals))
    max_vals = torch.max(max_vals, torch.zeros_like(max_vals))
    qmin, qmax = calculate_range(args)
    bit_range = qmax - qmin

    if args.symmetric:
        absmax = torch.max(torch.abs(min_vals), torch.abs(max_vals))
        if args.is_mx:
            e = torch.clamp(mxfp4_scale_exponent(absmax), 0, 255)
            scales = mxfp4_scale_from_exponent(e, min_vals.dtype)
        else:
            scales = absmax / (float(bit_range) / 2)
        zero_points = torch.zeros(scales.shape, dtype=min_vals.dtype)
    else:
        if args.is_fp4:
            raise NotImplementedError("asymmetric FP4 is not supported")
        scales = (max_vals - min_vals) / float(bit_range)
        zero_points = qmin - (min_vals / scales)
        zero_points = torch.clamp(zero_points, qmin, qmax)

    if global_scale is not None:
        scales = global_scale * scales

    eps_dtype = scales.dtype
    if args.scale_dtype is not None and not args.is_mx:
        scales = round_to_dtype(scales, args.scale_dtype)
        eps_dtype = args.scale_dtype

    eps = _dtype_eps(eps_dtype)
    scales = torch.where(scales == 0, torch.tensor(eps, dtype=scales.dtype), scales)

    zero_points = round_to_dtype(zero_points, args.zp_dtype, cast_back=False)
    if scales.ndim == 0:
        scales = scales.reshape(1)
        zero_points = zero_points.reshape(1)
    return scales, zero_points


def generate_gparam(min_val, max_val, dtype=torch.float32):
    """NVFP4 global scale ``448 * 6 / absmax`` as compressed-tensors writes it: a Python float divided by a
    tensor, which torch evaluates as ``absmax.reciprocal() * 2688.0`` (``Tensor.__rtruediv__``) -- for bf16
    statistics the reciprocal is rounded to bf16 before the product (2688/40 -> 67.5, a single division would
    give 67.0).  The reference's golden vectors (2688/23 -> 117.0, 2688/11 -> 244.0) hold either way."""
    mn = torch.min(min_val, torch.zeros_like(min_val))
    mx = torch.max(max_val, torch.zeros_like(max_val))
    absmax = torch.max(torch.abs(mn), torch.abs(mx))
    gs = FP8_MAX * FP4_MAX / absmax
    return gs.to(dtype).reshape([1])


def cast_to_fp4(x: torch.Tensor) -> torch.Tensor:
    """Round |x| <= 6 to the e2m1 grid, ties to even mantissa, sign kept."""
    sign = torch.sign(x)
    a = torch.abs(x)
    out = torch.full_like(a, 6.0)
    out = torch.where(a <= 5.0, torch.full_like(a, 4.0), out)
    out = torch.where(a < 3.5, torch.full_like(a, 3.0), out)
    out = torch.where(a <= 2.5, torch.full_like(a, 2.0), out)
    out = torch.where(a < 1.75, torch.full_like(a, 1.5), out)
    out = torch.where(a <= 1.25, torch.full_like(a, 1.0), out)
    out = torch.where(a < 0.75, torch.full_like(a, 0.5), out)
    out = torch.where(a <= 0.25, torch.zeros_like(a), out)
    return out * sign


def round_to_qtype(t: torch.Tensor, args: QArgs, qmin: float, qmax: float):
    """clamp + round into the element format (CT ``round_to_quantized_type_args``)."""
    c = torch.clamp(t, qmin, qmax)
    if args.type == "int":
        return torch.round(c)
    if args.num_bits == 8:
        return c.to(torch.float8_e4m3fn).to(t.dtype)
    return cast_to_fp4(c)


def _quantize(x, scale, zp, args: QArgs, qmin, qmax, dtype=None, global_scale=None):
    if global_scale is not None:
        scale = scale.to(global_scale.dtype) / global_scale
    scaled = x / scale
    if zp is not None:
        scaled = scaled + zp.to(x.dtype)
    q = round_to_qtype(scaled, args, qmin, qmax)
    if dtype is not None:
        q = q.to(dtype)
    return q


def _dequantize(q, scale, zp=None, dtype=None, global_scale=None):
    if global_scale is not None:
        scale = scale.to(global_scale.dtype) / global_scale
    dq = q.to(scale.dtype)
    if zp is not None:
        dq = dq - zp.to(scale.dtype)
    dq = dq * scale
    if dtype is not None:
        dq = dq.to(dtype)
    return dq


def _process(x, scale, zp, args: QArgs, do_q, do_dq, dtype=None, global_scale=None, g_idx=None):
    qmin, qmax = calculate_range(args)
    strat = args.strategy
    if strat == "block":
        bh, bw = args.block_structure
        rows, cols = x.shape[-2], x.shape[-1]
        pr, pc = (-rows) % bh, (-cols) % bw
        xp = torch.nn.functional.pad(x, (0, pc, 0, pr)) if (pr or pc) else x
        R, C = xp.shape[-2], xp.shape[-1]
        xb = xp.reshape(R // bh, bh, C // bw, bw).transpose(1, 2)
        sb = scale.unsqueeze(-1).unsqueeze(-1)
        zb = zp.unsqueeze(-1).unsqueeze(-1) if zp is not None else None
        out = xb
        if do_q:
            out = _quantize(out, sb, zb, args, qmin, qmax, dtype, global_scale)
        if do_dq:
            out = _dequantize(out, sb, zb, global_scale=global_scale)
        out = out.transpose(1, 2).reshape(R, C)[:rows, :cols]
        return out
    if strat in ("group", "tensor_group"):
        out_dtype = dtype if dtype is not None else x.dtype
        gsz = args.group_size
        while scale.ndim < 2:
            scale = scale.unsqueeze(1)
            zp = zp.unsqueeze(1) if zp is not None else None
        cols = x.shape[-1]
        if cols >= gsz and cols % gsz != 0:
            raise ValueError("columns must be divisible by group_size")
        column_order = g_idx is None or bool((g_idx == -1).any())
        if not column_order:
            perm = torch.argsort(g_idx)
            x = x.index_select(-1, perm)
        xg = x.unflatten(-1, (math.ceil(cols / gsz), gsz))
        out = xg
        zz = zp.unsqueeze(-1) if zp is not None else None
        if do_q:
            out = _quantize(out, scale.unsqueeze(-1), zz, args, qmin, qmax, dtype, global_scale)
        if do_dq:
            out = _dequantize(out, scale.unsqueeze(-1), zz, global_scale=global_scale)
        out = out.flatten(start_dim=-2).to(out_dtype)
        if not column_order:
            out = out.index_select(-1, torch.argsort(perm))
        return out
    # tensor / channel / token / attn_head
    out = x
    if do_q:
        out = _quantize(out, scale, zp, args, qmin, qmax, dtype, global_scale)
    if do_dq:
        out = _dequantize(out, scale, zp, global_scale=global_scale)
    return out


def fake_quantize(x, scale, zero_point, args: QArgs, g_idx=None, global_scale=None):
    """quantise then dequantise (CT ``fake_quantize``)."""
    return _process(x, scale, zero_point, args, True, True, None, global_scale, g_idx)


def quantize(x, scale, zero_point, args: QArgs, dtype=None, g_idx=None, global_scale=None):
    return _process(x, scale, zero_point, args, True, False, dtype, global_scale, g_idx)


def dequantize(q, scale, zero_point, args: QArgs, dtype=None, g_idx=None, global_scale=None):
    out = _process(q, scale, zero_point, args, False, True, None, global_scale, g_idx)
    return out.to(dtype) if dtype is not None else out


def compute_dynamic_scales_and_zp(value, args: QArgs, global_scale=None):
    """Per-call qparams for ``dynamic`` activations (CT ``compute_dynamic_scales_and_zp``)."""
    keep = True
    if args.strategy == "token":
        reduce_dims = tuple(i for i in range(value.ndim) if i not in (0, 1))
    elif args.strategy == "tensor":
        reduce_dims = None
    elif args.strategy in ("group", "tensor_group"):
        reduce_dims = -1
        keep = False
        value = value.unflatten(-1, (math.ceil(value.shape[-1] / args.group_size), args.group_size))
    else:
        raise ValueError(f"dynamic quantization does not support {args.strategy}")
    if not reduce_dims:
        mn, mx = torch.aminmax(value)
    else:
        mn = torch.amin(value, dim=reduce_dims, keepdim=keep)
        mx = torch.amax(value, dim=reduce_dims, keepdim=keep)
    return calculate_qparams(mn, mx, args, global_scale=global_scale)


def forward_quantize_dynamic(value, args: QArgs, global_scale=None):
    """fake-quantise an activation with per-call scales (CT ``forward_quantize``, dynamic branch)."""
    scale, zp = compute_dynamic_scales_and_zp(value, args, global_scale)
    return fake_quantize(value, scale, zp, args, global_scale=global_scale), scale
