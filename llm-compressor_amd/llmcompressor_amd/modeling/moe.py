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

__all__ = ["ExpertMLP", "LinearExperts2D", "moe_calibration_context"]

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
    def __init__(self, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.gate_proj = nn.Linear(hidden, intermediate, bias=False, dtype=dtype, device=device)
        self.up_proj = nn.Linear(hidden, intermediate, bias=False, dtype=dtype, device=device)
        self.down_proj = nn.Linear(intermediate, hidden, bias=False, dtype=dtype, device=device)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class LinearExperts2D(nn.ModuleList):
    """Experts as a list of ExpertMLP; ``from_fused`` splits [E, 2I, H] gate_up and [E, H, I] down tensors."""

    def __init__(self, num_experts: int, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None):
        super().__init__([ExpertMLP(hidden, intermediate, dtype, device) for _ in range(num_experts)])
        self.num_experts = num_experts

    @classmethod
    def from_fused(cls, gate_up_proj: torch.Tensor, down_proj: torch.Tensor) -> "LinearExperts2D":
        E, two_i, H = gate_up_proj.shape
        inter = two_i // 2
        self = cls(E, H, inter, gate_up_proj.dtype, gate_up_proj.device)
        with torch.no_grad():
            for e, expert in enumerate(self):
                expert.gate_proj.weight.copy_(gate_up_proj[e, :inter])
                expert.up_proj.weight.copy_(gate_up_proj[e, inter:])
                expert.down_proj.weight.copy_(down_proj[e])
        return self

    def forward(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor):
        """hidden_states [T,H]; top_k_index / top_k_weights [T,k]."""
        final = torch.zeros_like(hidden_states)
        onehot = torch.nn.functional.one_hot(top_k_index, num_classes=self.num_experts).permute(2, 1, 0)  # [E,k,T]
        for e, expert in enumerate(self):
            slot, token_idx = torch.where(onehot[e])
            if _CALIBRATE_ALL_EXPERTS:
                out = expert(hidden_states)[token_idx]
            else:
                out = expert(hidden_states[token_idx])
            if token_idx.numel() > 0:
                final.index_add_(0, token_idx, (out * top_k_weights[token_idx, slot, None]).to(final.dtype))
        return final
