"""Oracle: compressed-tensors storage formats (no reference-held bytes exist; the layouts are pinned by
independent decoders in ``tests/test_oracle_formats.py``, see ``oracle/__init__.py``).

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Restates the compressors reached from
``src/llmcompressor/transformers/compression/compressed_tensors_utils.py:134-138``
and ``src/llmcompressor/entrypoints/model_free/process.py:125,205,226``:
``pack-quantized`` (int4/int8 in int32 words), ``int-quantized`` (int8),
``float-quantized`` (fp8 e4m3), ``nvfp4-pack-quantized`` and
``mxfp4-pack-quantized`` (two e2m1 nibbles per byte).  Tensor names and the
``pack_factor = 32 // num_bits`` rule are corroborated by the installed
``transformers/integrations/compressed_tensors.py:109-134``.
"""
from __future__ import annotations

import math

import torch

from .qformat import E2M1_VALUES, QArgs, mxfp4_scale_exponent, quantize


def pack_to_int32(value: torch.Tensor, num_bits: int) -> torch.Tensor:
    """int8 codes [R,K] -> int32 [R, ceil(K/pf)], element j of a word at bit j*num_bits."""
    offset = 1 << (num_bits - 1)
    v = (value.to(torch.int32) + offset).to(torch.uint8)
    pf = 32 // num_bits
    rows, cols = v.shape
    padded = math.ceil(cols / pf) * pf
    if padded != cols:
        v = torch.nn.functional.pad(v, (0, padded - cols))
    r = v.view(rows, padded // pf, pf).to(torch.int32)
    shifts = torch.arange(pf, dtype=torch.int32) * num_bits
    return (r << shifts).sum(dim=2, dtype=torch.int32)


def unpack_from_int32(packed: torch.Tensor, num_bits: int, shape) -> torch.Tensor:
    pf = 32 // num_bits
    mask = (1 << num_bits) - 1
    shifts = torch.arange(pf, dtype=torch.int32) * num_bits
    u = (packed.unsqueeze(-1) >> shifts) & mask
    u = u.reshape(packed.shape[0], -1)[:, : shape[1]]
    return (u - (1 << (num_bits - 1))).to(torch.int8)


def pack_fp4_to_uint8(x: torch.Tensor) -> torch.Tensor:
    """e2m1-valued tensor [R,K] -> uint8 [R,K/2]; even column in the low nibble; sign bit 3."""
    m, n = x.shape
    grid = torch.tensor(E2M1_VALUES, dtype=x.dtype)
    idx = torch.argmin(torch.abs(torch.abs(x).unsqueeze(-1) - grid), dim=-1)
    idx = idx + (torch.signbit(x).to(torch.long) << 3)
    idx = idx.reshape(-1, 2)
    return (idx[:, 0] | (idx[:, 1] << 4)).to(torch.uint8).reshape(m, n // 2)


def unpack_fp4_from_uint8(p: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    grid = torch.tensor(E2M1_VALUES + tuple(-v for v in E2M1_VALUES), dtype=dtype)
    lo = (p & 0xF).long()
    hi = (p >> 4).long()
    return torch.stack([grid[lo], grid[hi]], dim=-1).reshape(p.shape[0], -1)


def compress_weight(weight, scale, zero_point, args: QArgs, global_scale=None, g_idx=None):
    """weight + qparams -> dict of stored tensors for the scheme's format."""
    R, K = weight.shape
    out = {}
    if args.type == "int":
        q = quantize(weight, scale, zero_point, args, dtype=torch.int8, g_idx=g_idx)
        out["weight_packed"] = pack_to_int32(q, args.num_bits)
        out["weight_shape"] = torch.tensor([R, K], dtype=torch.int64)
        out["weight_scale"] = scale
        out["codes"] = q
        if not args.symmetric:
            out["weight_zero_point"] = zero_point
        return out
    if args.num_bits == 8:
        q = quantize(weight, scale, zero_point, args, dtype=torch.float8_e4m3fn)
        out["weight"] = q
        out["weight_scale"] = scale
        return out
    # fp4
    if args.is_mx:
        q = quantize(weight, scale, zero_point, args)
        out["weight_packed"] = pack_fp4_to_uint8(q)
        out["weight_scale"] = (torch.log2(scale.float()) + 127).to(torch.uint8)
        return out
    q = quantize(weight, scale, zero_point, args, global_scale=global_scale)
    out["weight_packed"] = pack_fp4_to_uint8(q)
    out["weight_scale"] = scale.to(torch.float8_e4m3fn)
    out["weight_global_scale"] = global_scale
    return out


def int8_store(weight, scale, zero_point, args: QArgs):
    """``int-quantized``: plain int8 codes."""
    return quantize(weight, scale, zero_point, args, dtype=torch.int8)


__all__ = [
    "pack_to_int32",
    "unpack_from_int32",
    "pack_fp4_to_uint8",
    "unpack_fp4_from_uint8",
    "compress_weight",
    "int8_store",
    "mxfp4_scale_exponent",
]
