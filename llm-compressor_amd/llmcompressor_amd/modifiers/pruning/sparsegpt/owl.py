"""Helpers of the OWL sparsity profile (Outlier Weighed Layerwise sparsity, arXiv 2310.05175; the reference
infers it in modifiers/pruning/sparsegpt/sgpt_base.py:182-250).  Device-side reductions only."""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ...utils.hooks import HooksMixin

NUM_NORM_SAMPLES = 128  # the per-batch channel norms are averaged over this many samples


def channel_norms(owner: HooksMixin, model: torch.nn.Module, dataloader) -> Dict[str, torch.Tensor]:
    """name -> fp32 [in_features]: sum over the calibration batches of the batch's per-channel L2 norm / 128,
    for every Linear outside lm_head.  One sum-of-squares kernel per hook call, no fp32 copy of the input."""
    from ....torch_ops import llmc

    totals: Dict[str, torch.Tensor] = {}

    def pre_hook(name):
        def hook(_module, inputs):
            x = inputs[0] if isinstance(inputs, (tuple, list)) else inputs
            rows = x.detach().reshape(-1, x.shape[-1])
            sq = torch.zeros(rows.shape[1], dtype=torch.float32, device=rows.device)
            llmc.sumsq_accum_(sq, rows)  # device tensors only: the dispatcher refuses anything else
            norm = sq.sqrt_().div_(NUM_NORM_SAMPLES)
            if name in totals:
                totals[name] += norm
            else:
                totals[name] = norm
        return hook

    handles = {owner.register_hook(mod, pre_hook(name), "forward_pre")
               for name, mod in model.named_modules()
               if isinstance(mod, torch.nn.Linear) and "lm_head" not in name}
    device = next(model.parameters()).device
    try:
        with HooksMixin.disable_hooks(keep=handles), torch.no_grad():
            for batch in dataloader or ():
                if isinstance(batch, dict):
                    model(**{k: (v.to(device) if torch.is_tensor(v) else v) for k, v in batch.items()})
                else:
                    model(batch.to(device) if torch.is_tensor(batch) else batch)
    finally:
        owner.remove_hooks(handles)
    return totals


def outlier_percentage(members: List[Tuple[torch.Tensor, torch.Tensor]], multiple: float) -> float:
    """Percentage of the scores |W_ij| * a_j of all (weight, channel norm) pairs of one layer that exceed
    `multiple` times the mean score of the layer."""
    total, count = 0.0, 0
    for w, a in members:
        total += float((w.detach().abs().float() * a.to(w.device)[None, :]).sum(dtype=torch.float64))
        count += w.numel()
    if count == 0:
        return 0.0
    threshold = multiple * total / count
    above = sum(int(((w.detach().abs().float() * a.to(w.device)[None, :]) > threshold).sum()) for w, a in members)
    return 100.0 * above / count
