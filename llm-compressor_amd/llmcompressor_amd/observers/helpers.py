"""Calibration flattening and fused-layer bookkeeping.

Same contract as the reference's ``observers/helpers.py``: ``flatten_for_calibration``
(:28-157) returns a view of shape ``(num_observations, *qparam_shape, group_size)``;
``fuse_weight_observers`` (:174-215) links q/k/v, gate/up, q_a/kv_a and w1/w3 weight
observers so TENSOR_GROUP schemes share one global scale.
"""
from __future__ import annotations

import math

import torch
from torch.nn import Module

from ..quantization import QuantizationArgs, QuantizationStrategy

__all__ = ["flatten_for_calibration", "fuse_weight_observers", "FUSED_LAYER_NAMES", "ACTIVATION_OBS", "lerp"]

ACTIVATION_OBS = ("input", "output", "q", "k", "v")

FUSED_LAYER_NAMES = [
    ("gate_proj", "up_proj"),
    ("q_proj", "k_proj", "v_proj"),
    ("q_a_proj", "kv_a_proj_with_mqa"),
    ("w1", "w3"),
]


def _pad_for_block(value, block_structure):
    bh, bw = block_structure
    rows, cols = value.shape[-2], value.shape[-1]
    pr, pc = (-rows) % bh, (-cols) % bw
    if pr or pc:
        value = torch.nn.functional.pad(value, (0, pc, 0, pr))
    return value


def flatten_for_calibration(value: torch.Tensor, base_name: str, args: QuantizationArgs) -> torch.Tensor:
    s = args.strategy
    S = QuantizationStrategy
    if base_name == "weight":
        if s == S.TENSOR:
            return value.reshape((1, 1, -1))
        if s == S.TOKEN:
            raise ValueError("Token quantization cannot be applied to weights")
        if s == S.CHANNEL:
            return value.unsqueeze(-2).unsqueeze(0)
        if s in (S.GROUP, S.TENSOR_GROUP):
            return value.unflatten(-1, (-1, args.group_size)).unsqueeze(0)
        if s == S.BLOCK:
            bh, bw = args.block_structure
            value = _pad_for_block(value, args.block_structure)
            rows, cols = value.shape
            return value.reshape(rows // bh, bh, cols // bw, bw).transpose(1, 2).flatten(-2, -1).unsqueeze(0)
        if s == S.ATTN_HEAD:
            raise ValueError("Attention head quantization cannot be applied to weights")
        raise ValueError(f"Unknown strategy {s}")
    if base_name in ("input", "output"):
        if s == S.TENSOR:
            return value.reshape((-1, 1, value.size(-1)))
        if s == S.TOKEN:
            return value
        if s == S.CHANNEL:
            raise ValueError("Channel quantization cannot be applied to activations")
        if s in (S.GROUP, S.TENSOR_GROUP):
            return value.flatten(0, 1).unflatten(-1, (-1, args.group_size))
        if s == S.BLOCK:
            raise ValueError("Block quantization cannot be applied to activations")
        if s == S.ATTN_HEAD:
            raise ValueError("Attention head quantization cannot be applied to activations")
        raise ValueError(f"Unknown strategy {s}")
    if base_name in ("q", "k", "v"):
        if s == S.TENSOR:
            return value.transpose(1, 2).flatten(0, 1).flatten(-2, -1).unsqueeze(-2)
        if s == S.ATTN_HEAD:
            return value.transpose(1, 2).flatten(0, 1).unsqueeze(-2).unsqueeze(-2)
        names = {S.TOKEN: "Token", S.CHANNEL: "Channel", S.GROUP: "Group", S.TENSOR_GROUP: "Group", S.BLOCK: "Block"}
        if s in names:
            raise ValueError(f"{names[s]} quantization cannot be applied to attention")
        raise ValueError(f"Unknown strategy {s}")
    raise ValueError(f"Unknown quantization base name: {base_name}")


def fuse_weight_observers(model: Module):
    from .fusion import FusionHandler

    for submodule in model.modules():
        for group in FUSED_LAYER_NAMES:
            if not all(hasattr(submodule, name) for name in group):
                continue
            layers = [getattr(submodule, name) for name in group]
            only_obs, only_tg, pairs = True, True, []
            for layer in layers:
                if layer is None:
                    continue
                obs = getattr(layer, "weight_observer", None)
                if obs is None:
                    only_obs = False
                    continue
                if obs.args.strategy != QuantizationStrategy.TENSOR_GROUP:
                    only_tg = False
                    continue
                pairs.append((obs, layer))
            if not pairs:
                continue
            start = f"Some layers in fused group: {group} have"
            end = ", need all fused layers to have same quantization"
            assert only_obs, f"{start} no weight observer{end}"
            assert only_tg, f"{start} non-TENSOR_GROUP quantization{end}"
            FusionHandler.fuse(pairs)


def lerp(start: torch.Tensor, end: torch.Tensor, weight: float) -> torch.Tensor:
    """``start * (1 - weight) + end * weight`` with each of the three operations rounded to the tensors' dtype
    (reference: observers/helpers.py:218-220).  For 16-bit tensors every operation is spelled out as an fp32
    operation followed by a cast: the device compiler may otherwise fuse a product with its conversion to f16
    into one instruction with a single rounding, which differs from the eager result on near-ties."""
    if start.dtype in (torch.float16, torch.bfloat16):
        dt = start.dtype
        a = (start.float() * (1.0 - weight)).to(dt)
        b = (end.float() * weight).to(dt)
        return (a.float() + b.float()).to(dt)
    return (start * (1.0 - weight)) + (end * weight)


def num_groups(cols: int, group_size: int) -> int:
    return math.ceil(cols / group_size)
