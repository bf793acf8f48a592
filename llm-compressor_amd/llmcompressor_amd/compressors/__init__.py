"""compressed-tensors checkpoint layout: pack, save, reload.

Replaces ``ModelCompressor.compress_model`` / ``compress_module`` as called from the reference's
``save_pretrained`` wrapper (transformers/compression/compressed_tensors_utils.py:106-174) and from
``model_free_ptq`` (entrypoints/model_free/process.py:125,205,226).  Tensor names
(``weight_packed`` / ``weight_scale`` / ``weight_zero_point`` / ``weight_g_idx`` / ``weight_shape`` /
``weight_global_scale``) and format strings follow the layout transformers reads back
(integrations/compressed_tensors.py) and the reference's format-inference table
(tests/.../test_compress_tensor_utils.py:289-325).  Packing runs in the HIP quantise/pack kernel.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import math

import torch

from .. import ops
from ..torch_ops import llmc
from ..quantization import (
    QuantizationArgs,
    QuantizationConfig,
    QuantizationScheme,
    QuantizationStatus,
    QuantizationStrategy,
    QuantizationType,
    is_module_quantized,
)
from ..quantization.lifecycle import effective_scale, kernel_format, scale_indexing

__all__ = ["infer_format", "resolve_format", "compress_module", "decompress_weight", "compress_model_state_dict",
           "save_pretrained_compressed", "quantization_config_dict", "CompressionFormat"]


class CompressionFormat:
    dense = "dense"
    int_quantized = "int-quantized"
    float_quantized = "float-quantized"
    naive_quantized = "naive-quantized"
    pack_quantized = "pack-quantized"
    nvfp4_pack_quantized = "nvfp4-pack-quantized"
    mxfp4_pack_quantized = "mxfp4-pack-quantized"
    mixed_precision = "mixed-precision"


def infer_format(scheme: QuantizationScheme) -> str:
    w, a = scheme.weights, scheme.input_activations
    if w is None:
        return CompressionFormat.dense
    if w.type == QuantizationType.FLOAT and w.num_bits == 4:
        return CompressionFormat.mxfp4_pack_quantized if w.is_mx else CompressionFormat.nvfp4_pack_quantized
    weight_only = a is None
    if weight_only:
        if w.type == QuantizationType.INT and w.num_bits in (4, 8):
            return CompressionFormat.pack_quantized
        return CompressionFormat.naive_quantized
    # weights and activations quantised: 8-bit floats are stored as fp8, every integer width one code per byte
    # (compressed-tensors' branch order; the reference's own table, tests/.../test_compress_tensor_utils.py:289-325,
    # holds W8A8 rows only, so the W4A8 row is not pinned by a reference-held vector)
    if w.type == QuantizationType.FLOAT and w.num_bits == 8:
        return CompressionFormat.float_quantized
    if w.type == QuantizationType.INT:
        return CompressionFormat.int_quantized
    return CompressionFormat.naive_quantized


def resolve_format(scheme: QuantizationScheme, override=None) -> str:
    """The format a scheme's weights are written in: the inferred one, or the caller's ``quantization_format``
    (a string with hyphens or underscores, or an enum member with such a ``value``) when the codes of the scheme
    can be stored that way.  The reference's W4AFP8 example saves with ``quantization_format="pack-quantized"``
    (examples/quantization_w4a8_fp8/llama3_example.py:76-80, docs/guides/saving_a_model.md:54-79): int4 codes
    next to quantised activations are inferred as one code per byte and packed eight per word on request."""
    inferred = infer_format(scheme)
    if override is None:
        return inferred
    fmt = str(getattr(override, "value", override)).replace("_", "-")
    w = scheme.weights
    if w is None or fmt in (inferred, CompressionFormat.dense):
        return CompressionFormat.dense if w is None else fmt
    is_int = w.type == QuantizationType.INT
    fits = {
        CompressionFormat.pack_quantized: is_int and w.num_bits in (4, 8),
        CompressionFormat.int_quantized: is_int,
        CompressionFormat.naive_quantized: is_int or w.num_bits == 8,
        CompressionFormat.float_quantized: not is_int and w.num_bits == 8,
        CompressionFormat.nvfp4_pack_quantized: not is_int and w.num_bits == 4 and not w.is_mx,
        CompressionFormat.mxfp4_pack_quantized: not is_int and w.num_bits == 4 and w.is_mx,
    }
    if fmt not in fits:
        raise ValueError(f"unknown quantization_format {fmt!r}; known: {sorted(fits) + [CompressionFormat.dense]}")
    if not fits[fmt]:
        raise ValueError(f"quantization_format {fmt!r} cannot hold {w.num_bits}-bit {w.type.value} weights "
                         f"(inferred format: {inferred!r})")
    return fmt


def _run(weight, scale, zp, args: QuantizationArgs, mode, g_idx=None, global_scale=None):
    fmt, bits = kernel_format(args)
    R, K = weight.shape
    row_div, srow, col_div = scale_indexing(args, R, K)
    es = effective_scale(scale, args, weight.dtype)
    zpa = None if args.symmetric or zp is None else zp.to(torch.int8)
    if g_idx is not None and bool((g_idx < 0).any()):
        g_idx = None
    return llmc.quant_pack(weight.contiguous(), es, zpa, fmt, bits, row_div, srow, col_div, mode, g_idx, global_scale)


def compress_module(module: torch.nn.Module, fmt: Optional[str] = None) -> Dict[str, torch.Tensor]:
    """The tensors a quantised module contributes to the checkpoint (keys relative to the module)."""
    scheme: QuantizationScheme = module.quantization_scheme
    args = scheme.weights
    fmt = fmt or infer_format(scheme)
    weight = module.weight.data
    scale = module.weight_scale.data
    zp = getattr(module, "weight_zero_point", None)
    zp = None if zp is None else zp.data
    gs = getattr(module, "weight_global_scale", None)
    gs = None if gs is None else gs.data.to(torch.float32)
    g_idx = getattr(module, "weight_g_idx", None)
    g_idx = None if g_idx is None else g_idx.data
    out: Dict[str, torch.Tensor] = {}
    if fmt == CompressionFormat.pack_quantized:
        out["weight_packed"] = _run(weight, scale, zp, args, ops.OUT_PACKED, g_idx)
        out["weight_shape"] = torch.tensor(list(weight.shape), dtype=torch.int64, device=weight.device)
        out["weight_scale"] = scale
        if not args.symmetric and zp is not None and args.strategy not in (QuantizationStrategy.GROUP,
                                                                           QuantizationStrategy.CHANNEL):
            out["weight_zero_point"] = zp  # only group / channel zero points are packed
        elif not args.symmetric and zp is not None:
            # zero points are packed along the row dimension like the weights along the columns
            z = (zp.to(torch.int32) + (1 << (args.num_bits - 1))).to(torch.int32)
            pf = 32 // args.num_bits
            zt = z.t().contiguous()
            pad = (-zt.shape[1]) % pf
            if pad:
                zt = torch.nn.functional.pad(zt, (0, pad))
            shifts = torch.arange(pf, device=z.device, dtype=torch.int32) * args.num_bits
            out["weight_zero_point"] = (zt.view(zt.shape[0], -1, pf) << shifts).sum(dim=2, dtype=torch.int32).t().contiguous()
        if g_idx is not None and not bool((g_idx < 0).any()):
            out["weight_g_idx"] = g_idx.to(torch.int32)
    elif fmt in (CompressionFormat.int_quantized, CompressionFormat.float_quantized, CompressionFormat.naive_quantized):
        out["weight"] = _run(weight, scale, zp, args, ops.OUT_CODES, g_idx)
        out["weight_scale"] = scale
        if not args.symmetric and zp is not None:
            out["weight_zero_point"] = zp
    elif fmt == CompressionFormat.nvfp4_pack_quantized:
        out["weight_packed"] = _run(weight, scale, zp, args, ops.OUT_PACKED, None, gs)
        out["weight_scale"] = scale if scale.dtype == torch.float8_e4m3fn else scale.to(torch.float8_e4m3fn)
        out["weight_global_scale"] = gs
    elif fmt == CompressionFormat.mxfp4_pack_quantized:
        out["weight_packed"] = _run(weight, scale, zp, args, ops.OUT_PACKED)
        out["weight_scale"] = scale  # E8M0 codes (uint8)
    else:
        raise ValueError(f"unsupported compression format {fmt}")
    for name in ("input_scale", "input_zero_point", "input_global_scale", "output_scale", "output_zero_point"):
        t = getattr(module, name, None)
        if t is None:
            continue
        if name.endswith("zero_point"):  # zero points of symmetric arguments are all zero and are not stored
            act = scheme.input_activations if name.startswith("input") else scheme.output_activations
            if act is None or act.symmetric:
                continue
        out[name] = t.data
    if getattr(module, "bias", None) is not None:
        out["bias"] = module.bias.data
    return out


_E2M1 = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def _expand_qparam(param: torch.Tensor, args: QuantizationArgs, R: int, K: int, g_idx=None) -> torch.Tensor:
    """A scale / zero-point array broadcast to the weight's [R, K] layout for its strategy."""
    s = args.strategy
    if param.numel() == 1:
        return param.reshape(1, 1)
    if s in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
        param = param.reshape(R, -1)
        if g_idx is not None:
            return param[:, g_idx.long()]
        return param.repeat_interleave(args.group_size, dim=1)[:, :K]
    if s == QuantizationStrategy.BLOCK:
        bh, bw = args.block_structure
        return param.repeat_interleave(bh, dim=0)[:R].repeat_interleave(bw, dim=1)[:, :K]
    return param.reshape(R, 1)  # channel


def _unpack_int32(packed: torch.Tensor, num_bits: int, count: int) -> torch.Tensor:
    """Fields of `num_bits` bits from int32 words along the last dimension, lowest bits first, offset removed."""
    pf = 32 // num_bits
    shifts = torch.arange(pf, device=packed.device, dtype=torch.int32) * num_bits
    fields = (packed.unsqueeze(-1) >> shifts) & ((1 << num_bits) - 1)
    return fields.reshape(*packed.shape[:-1], -1)[..., :count] - (1 << (num_bits - 1))


def decompress_weight(tensors: Dict[str, torch.Tensor], args: QuantizationArgs, fmt: str, dtype=torch.bfloat16):
    """Inverse of compress_module for checks and reloads (plain tensor ops on the stored codes): every
    strategy, symmetric or with (packed) zero points."""
    if fmt in (CompressionFormat.pack_quantized, CompressionFormat.float_quantized, CompressionFormat.int_quantized,
               CompressionFormat.naive_quantized):
        if fmt == CompressionFormat.pack_quantized:
            R, K = [int(v) for v in tensors["weight_shape"].tolist()]
            codes = _unpack_int32(tensors["weight_packed"], args.num_bits, K).to(torch.float32)
        else:
            codes = tensors["weight"].to(torch.float32)
            R, K = codes.shape
        g_idx = tensors.get("weight_g_idx")
        zp = tensors.get("weight_zero_point")
        if zp is not None and not args.symmetric:
            if fmt == CompressionFormat.pack_quantized and zp.dtype == torch.int32:
                # packed along the rows: [ceil(rows / pack_factor), columns of the zero-point array]
                rows = 1 if args.strategy == QuantizationStrategy.TENSOR else (
                    math.ceil(R / args.block_structure[0]) if args.strategy == QuantizationStrategy.BLOCK else R)
                zp = _unpack_int32(zp.t().contiguous(), args.num_bits, rows).t()
            codes = codes - _expand_qparam(zp.to(torch.float32), args, R, K, g_idx)
        scale = _expand_qparam(tensors["weight_scale"].to(dtype), args, R, K, g_idx)
        return codes.to(dtype) * scale
    packed = tensors["weight_packed"]
    grid = torch.tensor(_E2M1 + tuple(-v for v in _E2M1), dtype=torch.float32, device=packed.device)
    vals = torch.stack([grid[(packed & 0xF).long()], grid[(packed >> 4).long()]], dim=-1).reshape(packed.shape[0], -1)
    if fmt == CompressionFormat.nvfp4_pack_quantized:
        s = tensors["weight_scale"].to(torch.float32) / tensors["weight_global_scale"].to(torch.float32)
    else:
        s = torch.pow(2.0, tensors["weight_scale"].to(torch.float32) - 127.0)
    return (vals.unflatten(-1, (-1, args.group_size)) * s.unsqueeze(-1)).flatten(-2).to(dtype)


def compress_model_state_dict(model: torch.nn.Module, quantization_format=None) -> Dict[str, torch.Tensor]:
    """Full state dict with every quantised module's weight replaced by its packed tensors."""
    quantised = {name: m for name, m in model.named_modules()
                 if is_module_quantized(m) and getattr(m.quantization_scheme, "weights", None) is not None
                 and hasattr(m, "weight_scale")}
    out: Dict[str, torch.Tensor] = {}
    skip = set()
    for name, m in quantised.items():
        prefix = f"{name}." if name else ""
        for k, v in compress_module(m, fmt=resolve_format(m.quantization_scheme, quantization_format)).items():
            out[prefix + k] = v
        for k, _ in list(m.named_parameters(recurse=False)) + list(m.named_buffers(recurse=False)):
            skip.add(prefix + k)
    for k, v in model.state_dict().items():
        if k in skip or k in out or "_observer" in k:
            continue
        out[k] = v
    return out


def quantization_config_dict(model: torch.nn.Module, save_compressed: bool = True,
                             quantization_format=None) -> Optional[dict]:
    config: Optional[QuantizationConfig] = getattr(model, "quantization_config", None)
    if config is None or not isinstance(config, QuantizationConfig):
        return None
    formats = set()
    groups = {}
    for name, scheme in config.config_groups.items():
        fmt = resolve_format(scheme, quantization_format) if save_compressed else CompressionFormat.dense
        formats.add(fmt)
        d = scheme.model_dump(mode="json")
        d["format"] = fmt
        groups[name] = d
    fmt = formats.pop() if len(formats) == 1 else CompressionFormat.mixed_precision
    ignore = list(config.ignore or [])
    # un-targeted Linear layers are listed explicitly, as the reference's QuantizationModifier does
    for name, m in model.named_modules():
        if isinstance(m, torch.nn.Linear) and not is_module_quantized(m) and name not in ignore:
            ignore.append(name)
    return {
        "quant_method": "compressed-tensors",
        "version": config.version,
        "format": fmt,
        "quantization_status": (QuantizationStatus.COMPRESSED if save_compressed else QuantizationStatus.FROZEN).value,
        "global_compression_ratio": None,
        "config_groups": groups,
        "kv_cache_scheme": None if config.kv_cache_scheme is None else config.kv_cache_scheme.model_dump(mode="json"),
        "ignore": ignore,
        "transform_config": {},
    }


def save_pretrained_compressed(model: torch.nn.Module, save_directory: str, save_compressed: bool = True,
                               recipe=None, max_shard_size: int = 5 * 2**30):
    """Write ``model.safetensors`` (+ index when sharded), ``config.json`` with ``quantization_config``
    and ``recipe.yaml``."""
    from safetensors.torch import save_file

    os.makedirs(save_directory, exist_ok=True)
    sd = compress_model_state_dict(model) if save_compressed else {
        k: v for k, v in model.state_dict().items() if "_observer" not in k}
    sd = {k: v.detach().contiguous().cpu() for k, v in sd.items()}
    shards, cur, size = [], {}, 0
    for k, v in sd.items():
        nbytes = v.numel() * v.element_size()
        if cur and size + nbytes > max_shard_size:
            shards.append(cur)
            cur, size = {}, 0
        cur[k] = v
        size += nbytes
    shards.append(cur)
    if len(shards) == 1:
        save_file(shards[0], os.path.join(save_directory, "model.safetensors"), metadata={"format": "pt"})
    else:
        index = {"metadata": {}, "weight_map": {}}
        for i, shard in enumerate(shards):
            fname = f"model-{i + 1:05d}-of-{len(shards):05d}.safetensors"
            save_file(shard, os.path.join(save_directory, fname), metadata={"format": "pt"})
            for k in shard:
                index["weight_map"][k] = fname
        with open(os.path.join(save_directory, "model.safetensors.index.json"), "w") as f:
            json.dump(index, f, indent=2)
    cfg = getattr(model, "config", None)
    cfg_dict = cfg.to_dict() if hasattr(cfg, "to_dict") else {}
    qcfg = quantization_config_dict(model, save_compressed)
    if qcfg is not None:
        cfg_dict["quantization_config"] = qcfg
    with open(os.path.join(save_directory, "config.json"), "w") as f:
        json.dump(cfg_dict, f, indent=2, default=str)
    if recipe is not None and getattr(recipe, "modifiers", None):
        path = os.path.join(save_directory, "recipe.yaml")
        recipe.yaml(file_path=path, existing_recipe_path=path if os.path.exists(path) else None)
