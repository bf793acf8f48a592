"""Oracle: the per-expert loop of ``LinearExperts2D.forward``.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Restates ``src/llmcompressor/modeling/moe/linear_experts.py:235-268``: a one-hot mask ``[E, k, T]``, and per
expert ``torch.where`` on its ``[k, T]`` slice (pairs in slot-major order), the expert applied to the routed
rows (or to all rows, then indexed, when every expert is calibrated on all tokens), the routing weight of each
(token, slot) pair, and one ``index_add_`` into the output per expert, in expert order.

Parity status: pinned by the reference's own routing test (token counts per expert for hidden 16,
intermediate 32, 4 experts, top-2; ``tests/llmcompressor/modeling/test_linear_experts.py:12-106``) and by the
dense closed form ``sum_j w[t, j] * expert_{idx[t, j]}(x[t])`` in fp64.
"""
from __future__ import annotations

import torch


def experts_forward(experts, hidden_states, top_k_index, top_k_weights, calibrate_all_experts=False):
    """``experts``: a sequence of callables (one per expert).  Returns the combined output [T, H]."""
    num_experts = len(experts)
    final = torch.zeros_like(hidden_states)
    mask = torch.nn.functional.one_hot(top_k_index, num_experts).permute(2, 1, 0)
    for e in range(num_experts):
        slot, tokens = torch.where(mask[e])
        if calibrate_all_experts:
            out = experts[e](hidden_states)[tokens]
        else:
            out = experts[e](hidden_states[tokens])
        final.index_add_(0, tokens, (out * top_k_weights[tokens, slot, None]).to(final.dtype))
    return final
