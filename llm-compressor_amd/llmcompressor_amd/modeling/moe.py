"""Per-expert Linear view of a fused MoE block for calibration (reference: modeling/moe/linear_experts.py:137-268,
modeling/moe/context.py:3-18).

Each expert is an ``ExpertMLP`` of plain ``nn.Linear`` layers so GPTQ / observers see ordinary Linears.
Every expert is called on every forward, also with zero routed tokens (an expert that never receives a
token keeps a zero Hessian, so GPTQ zeroes its weight exactly as the reference does).  Inside
``moe_calibration_context()`` every expert sees all tokens; outputs are still combined with the routing
weights of the tokens actually routed to it.
"""
from __future__ import annotations

import contextlib

import torch
from torch import nn

__all__ = ["ExpertMLP", "LinearExperts2D", "moe_calibration_context", "get_non_linearized_moes", "linearize_moe"]

_CALIBRATE_ALL_EXPERTS = False


@contextlib.contextmanager
def moe_calibration_context(calibrate_all_experts: bool = True):
    global _CALIBRATE_ALL_EXPERTS
    prev = _CALIBRATE_ALL_EXPERTS
    _CALIBRATE_ALL_EXPERTS = calibrate_all_experts
    try:
        yield
    finally:
        _CALIBRATE_ALL_EXPERTS = prev


class ExpertMLP(nn.Module):
    def __init__(self, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None, act_fn=None,
                 bias: bool = False):
        super().__init__()
        self.gate_proj = nn.Linear(hidden, intermediate, bias=bias, dtype=dtype, device=device)
        self.up_proj = nn.Linear(hidden, intermediate, bias=bias, dtype=dtype, device=device)
        self.down_proj = nn.Linear(intermediate, hidden, bias=bias, dtype=dtype, device=device)
        self.act_fn = act_fn if act_fn is not None else nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class LinearExperts2D(nn.ModuleList):
    """Experts as a list of ExpertMLP; ``from_fused`` splits [E, 2I, H] gate_up and [E, H, I] down tensors."""

    def __init__(self, num_experts: int, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None,
                 act_fn=None, bias: bool = False):
        super().__init__([ExpertMLP(hidden, intermediate, dtype, device, act_fn, bias) for _ in range(num_experts)])
        self.num_experts = num_experts

    @classmethod
    def from_fused(cls, gate_up_proj: torch.Tensor, down_proj: torch.Tensor, act_fn=None, gate_up_bias=None,
                   down_bias=None) -> "LinearExperts2D":
        E, two_i, H = gate_up_proj.shape
        inter = two_i // 2
        self = cls(E, H, inter, gate_up_proj.dtype, gate_up_proj.device, act_fn, bias=gate_up_bias is not None)
        with torch.no_grad():
            for e, expert in enumerate(self):
                expert.gate_proj.weight.copy_(gate_up_proj[e, :inter])
                expert.up_proj.weight.copy_(gate_up_proj[e, inter:])
                expert.down_proj.weight.copy_(down_proj[e])
                if gate_up_bias is not None:
                    expert.gate_proj.bias.copy_(gate_up_bias[e, :inter])
                    expert.up_proj.bias.copy_(gate_up_bias[e, inter:])
                    expert.down_proj.bias.copy_(down_bias[e])
        return self

    @classmethod
    def from_experts_module(cls, experts: nn.Module) -> "LinearExperts2D":
        """From a fused experts module in the standard transformers layout (reference:
        modeling/moe/linear_experts.py:186-208): ``gate_up_proj`` [E, 2I, H] and ``down_proj`` [E, H, I]
        parameters (``is_transposed``: [E, H, 2I] and [E, I, H]), optional ``*_bias`` parameters, ``act_fn``."""
        gate_up, down = experts.gate_up_proj.data, experts.down_proj.data
        if getattr(experts, "is_transposed", False):
            gate_up, down = gate_up.transpose(1, 2), down.transpose(1, 2)
        gub, db = getattr(experts, "gate_up_proj_bias", None), getattr(experts, "down_proj_bias", None)
        return cls.from_fused(gate_up, down, getattr(experts, "act_fn", None),
                              None if gub is None else gub.data, None if db is None else db.data)

    def forward(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor):
        """hidden_states [T,H]; top_k_index / top_k_weights [T,k].

        Same values as the reference's loop (``torch.where`` on a one-hot mask per expert, one ``index_add_`` per
        expert, modeling/moe/linear_experts.py:235-268) with the routing done once for all experts: the
        (slot, token) pairs are sorted by expert with a stable sort, which leaves each expert's pairs in the
        slot-major order ``torch.where`` yields; the routed rows are gathered once and every expert's Linears are
        called on a slice of that buffer (so their hooks fire as before, also for an expert with no token); the
        weighted outputs are added per token in ascending expert order, one rounding to the output dtype per
        addition, as the chain of ``index_add_`` calls does.  One host wait (the experts' token counts) per call
        instead of one per expert."""
        T, k = top_k_index.shape
        E = self.num_experts
        with torch.no_grad():
            flat = top_k_index.t().reshape(-1)  # pair p = slot * T + token
            order = torch.argsort(flat, stable=True)
            counts = torch.bincount(flat, minlength=E).tolist()
            slot_sorted = torch.div(order, T, rounding_mode="floor")
            tok_sorted = order - slot_sorted * T
            # position of each token's pairs in the sorted list, ascending = ascending expert
            place = torch.empty_like(order)
            place[order] = torch.arange(order.numel(), device=order.device)
            place = place.view(k, T).sort(dim=0).values
        routed = None if _CALIBRATE_ALL_EXPERTS else hidden_states[tok_sorted]
        outs, at = [], 0
        for e, expert in enumerate(self):
            n = counts[e]
            if _CALIBRATE_ALL_EXPERTS:
                outs.append(expert(hidden_states)[tok_sorted[at:at + n]])
            else:
                outs.append(expert(routed[at:at + n]))
            at += n
        weighted = (torch.cat(outs) * top_k_weights[tok_sorted, slot_sorted, None]).to(hidden_states.dtype)
        final = torch.zeros_like(hidden_states)
        for j in range(k):
            final = final + weighted[place[j]]
        return final


def get_non_linearized_moes(model: nn.Module):
    """(name, module) of every fused experts module: 3-D ``gate_up_proj`` and ``down_proj`` parameters whose
    shapes fit each other (reference: modeling/moe/linearize.py:128-147)."""
    found = []
    for name, module in model.named_modules():
        if isinstance(module, LinearExperts2D):
            continue
        gu, dn = getattr(module, "gate_up_proj", None), getattr(module, "down_proj", None)
        if not (isinstance(gu, torch.Tensor) and isinstance(dn, torch.Tensor) and gu.ndim == 3 and dn.ndim == 3
                and gu.shape[0] == dn.shape[0]):
            continue
        if getattr(module, "is_transposed", False):
            fits = gu.shape[2] == 2 * dn.shape[1] and gu.shape[1] == dn.shape[2]
        else:
            fits = gu.shape[1] == 2 * dn.shape[2] and gu.shape[2] == dn.shape[1]
        if fits:
            found.append((name, module))
    return found


def linearize_moe(model: nn.Module) -> nn.Module:
    """Replace every fused experts module by a ``LinearExperts2D`` of plain Linears, so that per-expert
    weights can be calibrated and quantised (reference: modeling/moe/linearize.py:97-125)."""
    for name, module in get_non_linearized_moes(model):
        model.set_submodule(name, LinearExperts2D.from_experts_module(module))
    return model
