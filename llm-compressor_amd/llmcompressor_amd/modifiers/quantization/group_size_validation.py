"""Reject weights whose columns do not divide by group_size (reference: group_size_validation.py:38-123)."""
from __future__ import annotations

import torch

from ...quantization import QuantizationStrategy, match_named_modules

__all__ = ["validate_group_size_divisibility", "get_layers_indivisible_by_group_size"]


def get_layers_indivisible_by_group_size(model: torch.nn.Module, targets, ignore):
    bad = []
    for name, module in match_named_modules(model, targets, ignore):
        args = getattr(getattr(module, "quantization_scheme", None), "weights", None)
        weight = getattr(module, "weight", None)
        if args is None or weight is None:
            continue
        if args.strategy not in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
            continue
        cols = weight.shape[-1]
        if cols >= args.group_size and cols % args.group_size != 0:
            bad.append((name, cols, args.group_size))
    return bad


def validate_group_size_divisibility(model: torch.nn.Module, targets, ignore) -> None:
    bad = get_layers_indivisible_by_group_size(model, targets, ignore)
    if not bad:
        return
    lines = "\n".join(f"  - {n} (columns={c}, group_size={g})" for n, c, g in bad)
    names = [n for n, _, _ in bad]
    raise ValueError(
        "The following layers have weight column counts not divisible by group_size. Group and tensor-group "
        "quantization require columns % group_size == 0; compressed-tensors will error when saving or running "
        f"forward. Add these layer names to the modifier's `ignore` list and re-run, or set "
        f"`bypass_divisibility_checks=True`.\n\n{lines}\n\nignore={names}")
