"""Per-expert Linear view of a fused MoE block for calibration (reference: modeling/moe/linear_experts.py:137-268,
modeling/moe/context.py:3-18).

Each expert is an ``ExpertMLP`` of plain ``nn.Linear`` layers so GPTQ / observers see ordinary Linears.
Every expert is called on every forward, also with zero routed tokens (an expert that never receives a
token keeps a zero Hessian, so GPTQ zeroes its weight exactly as the reference does).  Inside
``moe_calibration_context()`` every expert sees all tokens; outputs are still combined with the routing
weights of the tokens actually routed to it.

When nothing observes the experts' Linears -- every hook on them was registered through ``HooksMixin`` and is
switched off (the propagation pass of a sequential pipeline), no quantised forward is active -- the
per-expert calls are replaced by two grouped launches over the routed-token buffer (``grouped_forward``).
"""
from __future__ import annotations

import contextlib
import inspect
import types

import torch
from torch import nn

__all__ = ["ExpertMLP", "LinearExperts2D", "Llama4LinearExperts", "moe_calibration_context",
           "get_calibrate_all_experts_flag",
           "get_non_linearized_moes", "linearize_moe"]

_CALIBRATE_ALL_EXPERTS = False
# replace the per-expert loop by grouped launches when no hook or quantised forward needs the single calls
GROUPED_FORWARD = True
# Off by default: take the grouped launches in observed passes too, when every hook that would fire on an
# expert Linear only reads the module's input (the Hessian hooks of GPTQ and SparseGPT say so about themselves).
# The hooks are then called with the same rows as in the loop, but what down_proj receives was computed by the
# grouped product, whose sums run in another order than the library GEMM's: equal to the last bf16 digit, not
# bit for bit.
GROUPED_CALIBRATION = False


def get_calibrate_all_experts_flag() -> bool:
    """Is every expert called on every token right now (reference: modeling/moe/context.py:6-7)?"""
    return _CALIBRATE_ALL_EXPERTS


@contextlib.contextmanager
def moe_calibration_context(calibrate_all_experts: bool = True, grouped: bool | None = None):
    """``calibrate_all_experts``: every expert is called on every token (reference: modeling/moe/context.py);
    ``grouped``: value of ``GROUPED_CALIBRATION`` inside the context (None = leave it as it is)."""
    global _CALIBRATE_ALL_EXPERTS, GROUPED_CALIBRATION
    prev = _CALIBRATE_ALL_EXPERTS, GROUPED_CALIBRATION
    _CALIBRATE_ALL_EXPERTS = calibrate_all_experts
    if grouped is not None:
        GROUPED_CALIBRATION = bool(grouped)
    try:
        yield
    finally:
        _CALIBRATE_ALL_EXPERTS, GROUPED_CALIBRATION = prev


class ExpertMLP(nn.Module):
    """One expert as plain Linears.  ``forward`` is ``down(apply_gate(cat[gate(x), up(x)]))`` as in the reference
    (modeling/moe/linear_experts.py:26-87): "gate" and "up" name the first and second half of the fused
    projection's output columns, and ``apply_gate`` is the fused module's own gating function (by default
    ``act_fn(first half) * second half``), so an interleaved layout or a clamped activation keeps its meaning."""

    def __init__(self, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None, act_fn=None,
                 bias: bool = False, apply_gate=None):
        super().__init__()
        self.gate_proj = nn.Linear(hidden, intermediate, bias=bias, dtype=dtype, device=device)
        self.up_proj = nn.Linear(hidden, intermediate, bias=bias, dtype=dtype, device=device)
        self.down_proj = nn.Linear(intermediate, hidden, bias=bias, dtype=dtype, device=device)
        self.act_fn = act_fn if act_fn is not None else nn.SiLU()
        self._gate_fn = apply_gate  # a plain callable (bound to the experts list), not a submodule

    def forward(self, x):
        if self._gate_fn is None:
            return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))
        return self.down_proj(self._gate_fn(torch.cat([self.gate_proj(x), self.up_proj(x)], dim=-1)))


def _hooks_inert(module: nn.Module, hook_is_inert) -> bool:
    """No hook of ``module`` would do anything if it were called now."""
    for hooks in (module._forward_hooks, module._forward_pre_hooks, module._backward_hooks,
                  module._backward_pre_hooks):
        if hooks and not all(hook_is_inert(h) for h in hooks.values()):
            return False
    return True


def _reads_input_only(hook) -> bool:
    return bool(getattr(hook, "_llmc_input_only", False)
                or getattr(getattr(hook, "__wrapped__", None), "_llmc_input_only", False))


def _input_hooks(module: nn.Module, hook_is_inert):
    """The forward hooks of ``module`` that would act now, if all of them only read the module's input and take
    the plain (module, args, output) call; None if some other hook would act."""
    d = module.__dict__
    for hooks in (d["_forward_pre_hooks"], d["_backward_hooks"], d["_backward_pre_hooks"]):
        if hooks and not all(hook_is_inert(h) for h in hooks.values()):
            return None
    if d.get("_forward_hooks_with_kwargs") or d.get("_forward_hooks_always_called"):
        return None
    live = [h for h in d["_forward_hooks"].values() if not hook_is_inert(h)]
    return live if all(_reads_input_only(h) for h in live) else None


class LinearExperts2D(nn.ModuleList):
    """Experts as a list of ExpertMLP; ``from_fused`` splits [E, 2I, H] gate_up and [E, H, I] down tensors."""

    def __init__(self, num_experts: int, hidden: int, intermediate: int, dtype=torch.bfloat16, device=None,
                 act_fn=None, bias: bool = False, apply_gate=None, gate_attributes=None):
        super().__init__()
        # what a fused module's own gating function reads from `self` (activation, clamp limits, ...)
        for key, value in (gate_attributes or {}).items():
            object.__setattr__(self, key, value)
        bound = types.MethodType(apply_gate, self) if apply_gate is not None else None
        self.extend([ExpertMLP(hidden, intermediate, dtype, device, act_fn, bias, bound) for _ in range(num_experts)])
        self.num_experts = num_experts

    @classmethod
    def from_fused(cls, gate_up_proj: torch.Tensor, down_proj: torch.Tensor, act_fn=None, gate_up_bias=None,
                   down_bias=None, apply_gate=None, gate_attributes=None) -> "LinearExperts2D":
        E, two_i, H = gate_up_proj.shape
        inter = two_i // 2
        self = cls(E, H, inter, gate_up_proj.dtype, gate_up_proj.device, act_fn, bias=gate_up_bias is not None,
                   apply_gate=apply_gate, gate_attributes=gate_attributes)
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
        parameters (``is_transposed``: [E, H, 2I] and [E, I, H]), optional ``*_bias`` parameters, ``act_fn``, and
        the class's own ``_apply_gate`` when it defines one."""
        gate_up, down = experts.gate_up_proj.data, experts.down_proj.data
        if getattr(experts, "is_transposed", False):
            gate_up, down = gate_up.transpose(1, 2), down.transpose(1, 2)
        gub, db = getattr(experts, "gate_up_proj_bias", None), getattr(experts, "down_proj_bias", None)
        apply_gate = getattr(type(experts), "_apply_gate", None)
        attributes = {k: v for k, v in vars(experts).items()
                      if not k.startswith("_") and isinstance(v, (int, float, bool)) and k != "training"}
        act_fn = getattr(experts, "act_fn", None)
        if act_fn is not None:
            attributes["act_fn"] = act_fn  # a plain attribute of the list, so that its length stays the expert count
        return cls.from_fused(gate_up, down, act_fn if isinstance(act_fn, nn.Module) else None,
                              None if gub is None else gub.data, None if db is None else db.data,
                              apply_gate=apply_gate, gate_attributes=attributes)

    # per instance switch for the grouped launches (see ``_grouped_plan``)
    grouped_forward = True

    def _grouped_plan(self, hidden_states: torch.Tensor, observed: bool = False):
        """(``observed``: hooks on the Linears that only read their input may be live; the plan then lists them
        under "hooks", per projection and expert, for the caller to call.)

        The experts' weights as two pointer tables, or None when the per-expert calls must stay: some hook on
        an expert or one of its Linears would fire (only hooks registered through ``HooksMixin`` can be told to be
        off), a Linear has a bias, a quantised forward is active, the experts are not plain ``ExpertMLP``s of
        bf16 Linears of one shape, gradients are recorded, or the shapes do not fit the kernel's tiles.  The
        grouped products add along k in another order than the library GEMM behind ``F.linear``: same values to
        the last bf16 digit, not the same bits, which is why observed passes keep the loop."""
        from ...modifiers.utils.hooks import hook_is_inert
        from ... import ops

        if (not hidden_states.is_cuda or hidden_states.dtype != torch.bfloat16 or torch.is_grad_enabled()
                or len(self) == 0 or nn.modules.module._global_forward_hooks
                or nn.modules.module._global_forward_pre_hooks):
            return None
        weights = ([], [], [])
        live_hooks = ([], [], [])
        first = self[0]
        act_type, gate_fn = type(first._modules["act_fn"]), first._gate_fn
        names = ("gate_proj", "up_proj", "down_proj")
        for expert in self._modules.values():
            d = expert.__dict__
            if type(expert) is not ExpertMLP or "forward" in d or d["_gate_fn"] is not gate_fn:
                return None
            if (d["_forward_hooks"] or d["_forward_pre_hooks"] or d["_backward_hooks"]
                    or d["_backward_pre_hooks"]) and not _hooks_inert(expert, hook_is_inert):
                return None
            mods = d["_modules"]
            if type(mods["act_fn"]) is not act_type:
                return None
            for slot in range(3):
                lin = mods[names[slot]]
                d = lin.__dict__
                if type(lin) is not nn.Linear or d["_parameters"]["bias"] is not None:
                    return None
                if (d["_forward_hooks"] or d["_forward_pre_hooks"] or d["_backward_hooks"]
                        or d["_backward_pre_hooks"]) and not _hooks_inert(lin, hook_is_inert):
                    found = _input_hooks(lin, hook_is_inert) if observed else None
                    if found is None:
                        return None
                    live_hooks[slot].append(found)
                elif observed:
                    live_hooks[slot].append(())
                if "forward" in d and not (
                        d.get("_llmc_forward_wrapped", False)
                        and (d.get("quantization_scheme") is None or not d.get("quantization_enabled", True))):
                    return None
                weights[slot].append(d["_parameters"]["weight"])
        if any(True for _ in first.act_fn.parameters()):
            return None
        key = tuple(w.data_ptr() for group in weights for w in group)
        cached = self.__dict__.get("_grouped_cache")
        if cached is not None and cached[0] == key and cached[1] == hidden_states.device:
            return dict(cached[2], hooks=live_hooks) if observed else cached[2]
        gate, up, down = weights
        inter, hidden = gate[0].shape
        for group, shape in ((gate, (inter, hidden)), (up, (inter, hidden)), (down, (hidden, inter))):
            for w in group:
                if (w.shape != shape or w.dtype != torch.bfloat16 or w.stride() != group[0].stride()
                        or w.stride(1) != 1 or w.stride(0) % 8 or w.device != hidden_states.device):
                    return None
        if not (ops.grouped_linear_supported(inter, hidden, torch.bfloat16)
                and ops.grouped_linear_supported(hidden, inter, torch.bfloat16)) or gate[0].stride() != up[0].stride():
            return None
        try:
            plan = dict(gate_up=ops.weight_pointer_table(gate + up, hidden_states.device), ld_gate_up=gate[0].stride(0),
                        down=ops.weight_pointer_table(down, hidden_states.device), ld_down=down[0].stride(0),
                        inter=inter, hidden=hidden)
        except ValueError:  # a weight that is not 16-byte aligned
            return None
        object.__setattr__(self, "_grouped_cache", (key, hidden_states.device, plan))
        return dict(plan, hooks=live_hooks) if observed else plan

    def _forward_grouped_observed(self, plan, hidden_states, expert_sorted, tok_sorted, counts) -> torch.Tensor:
        """The grouped launches with live input-reading hooks: every hook is called with the rows its Linear would
        have received in the loop (all rows of the block's input with ``calibrate_all_experts``, else the expert's
        routed rows; an expert without rows still gets its call), the output argument being None.  Returns the
        experts' outputs for the routed rows, sorted by expert.  With ``calibrate_all_experts`` gate and up of all
        experts are one library product on the stacked weights, and down_proj runs on the routed rows only."""
        from ... import ops

        E, inter, hidden = self.num_experts, plan["inter"], plan["hidden"]
        hooks_gate, hooks_up, hooks_down = plan["hooks"]
        names = ("gate_proj", "up_proj", "down_proj")
        lins = [[expert._modules[n] for expert in self._modules.values()] for n in names]
        tiles, ntiles = ops.grouped_linear_tiles(counts, hidden_states.device)
        first = self[0]

        def gate(gate_up):
            if first._gate_fn is not None:
                return first._gate_fn(gate_up).contiguous()
            return (first.act_fn(gate_up[:, :inter]) * gate_up[:, inter:]).contiguous()

        def call(found, lin, rows):
            for hook in found:
                hook(lin, (rows,), None)

        if _CALIBRATE_ALL_EXPERTS:
            T = hidden_states.shape[0]
            # every expert reads the same rows: one library product with the experts' gate / up weights stacked
            # into one [E * 2I, H] matrix (a copy per call, so that it is never stale) instead of E tiles' worth of
            # grouped launches
            stacked = torch.cat([lin.weight for pair in zip(lins[0], lins[1]) for lin in pair])
            gate_up = torch.nn.functional.linear(hidden_states, stacked).view(T * E, 2 * inter)
            del stacked
            for e in range(E):  # the host walks the hooks while the device multiplies
                call(hooks_gate[e], lins[0][e], hidden_states)
                call(hooks_up[e], lins[1][e], hidden_states)
            mid = gate(gate_up).view(T, E, inter).permute(1, 0, 2).contiguous().view(E * T, inter)
            del gate_up
            for e in range(E):
                if hooks_down[e]:
                    call(hooks_down[e], lins[2][e], mid[e * T:(e + 1) * T])
            routed_mid = mid[expert_sorted * T + tok_sorted]
        else:
            routed = hidden_states[tok_sorted]
            gate_up = ops.grouped_linear(routed, plan["gate_up"], E, 2, inter, plan["ld_gate_up"], tiles, ntiles)
            at = 0
            for e in range(E):
                rows = routed[at:at + counts[e]]
                call(hooks_gate[e], lins[0][e], rows)
                call(hooks_up[e], lins[1][e], rows)
                at += counts[e]
            routed_mid = gate(gate_up)
            del gate_up
            at = 0
            for e in range(E):
                if hooks_down[e]:
                    call(hooks_down[e], lins[2][e], routed_mid[at:at + counts[e]])
                at += counts[e]
        return ops.grouped_linear(routed_mid, plan["down"], E, 1, hidden, plan["ld_down"], tiles, ntiles)

    def _forward_grouped(self, plan, routed: torch.Tensor, counts) -> torch.Tensor:
        """``expert(rows)`` for every expert's rows of ``routed`` (sorted by expert) in two launches."""
        from ... import ops

        E, inter = self.num_experts, plan["inter"]
        tiles, ntiles = ops.grouped_linear_tiles(counts, routed.device)
        gate_up = ops.grouped_linear(routed, plan["gate_up"], E, 2, inter, plan["ld_gate_up"], tiles, ntiles)
        first = self[0]
        if first._gate_fn is not None:
            mid = first._gate_fn(gate_up)
        else:
            mid = first.act_fn(gate_up[:, :inter]) * gate_up[:, inter:]
        return ops.grouped_linear(mid.contiguous(), plan["down"], E, 1, plan["hidden"], plan["ld_down"], tiles, ntiles)

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
        plan = self._grouped_plan(hidden_states) if GROUPED_FORWARD and self.grouped_forward else None
        observed = None
        if plan is None and GROUPED_CALIBRATION and GROUPED_FORWARD and self.grouped_forward:
            observed = self._grouped_plan(hidden_states, observed=True)
        if plan is not None:
            expert_out = self._forward_grouped(plan, hidden_states[tok_sorted], counts)
        elif observed is not None:
            expert_out = self._forward_grouped_observed(observed, hidden_states, flat[order], tok_sorted, counts)
        else:
            routed = None if _CALIBRATE_ALL_EXPERTS else hidden_states[tok_sorted]
            outs, at = [], 0
            for e, expert in enumerate(self):
                n = counts[e]
                if _CALIBRATE_ALL_EXPERTS:
                    outs.append(expert(hidden_states)[tok_sorted[at:at + n]])
                else:
                    outs.append(expert(routed[at:at + n]))
                at += n
            expert_out = torch.cat(outs)
        weighted = (expert_out * top_k_weights[tok_sorted, slot_sorted, None]).to(hidden_states.dtype)
        final = torch.zeros_like(hidden_states)
        for j in range(k):
            final = final + weighted[place[j]]
        return final


class Llama4LinearExperts(LinearExperts2D):
    """Per-expert Linears for ``Llama4TextExperts`` (reference: modeling/moe/llama4.py:15-110).  That module is
    called with the tokens already laid out per expert, ``[E * T, H]`` (every expert sees every token; the router's
    scores were applied upstream), stores ``gate_up_proj`` as [E, H, 2I] and ``down_proj`` as [E, I, H], and
    returns ``[E * T, H]``."""

    @classmethod
    def from_experts_module(cls, experts: nn.Module) -> "Llama4LinearExperts":
        gate_up, down = experts.gate_up_proj.data.transpose(1, 2), experts.down_proj.data.transpose(1, 2)
        return cls.from_fused(gate_up, down, getattr(experts, "act_fn", None))

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        per_expert = hidden_states.view(self.num_experts, -1, hidden_states.shape[-1])
        outs = []
        for e, expert in enumerate(self):
            if _CALIBRATE_ALL_EXPERTS:
                outs.append(expert(hidden_states).view(self.num_experts, -1, hidden_states.shape[-1])[e])
            else:
                outs.append(expert(per_expert[e]))
        return torch.cat(outs, dim=0)


# fused modules whose call convention differs from (hidden_states, top_k_index, top_k_weights), by class name
_SPECIAL_EXPERTS = {"Llama4TextExperts": Llama4LinearExperts}


def _takes_routing_arguments(module: nn.Module) -> bool:
    """forward(hidden_states, top_k_index, top_k_weights): the call LinearExperts2D.forward answers."""
    try:
        params = [p for p in inspect.signature(module.forward).parameters.values()
                  if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
    except (TypeError, ValueError):
        return False
    if any(p.kind == p.VAR_POSITIONAL for p in inspect.signature(module.forward).parameters.values()):
        return True  # a dispatching wrapper (*args, **kwargs)
    return len(params) == 3


def get_non_linearized_moes(model: nn.Module):
    """(name, module) of every fused experts module: 3-D ``gate_up_proj`` and ``down_proj`` parameters whose
    shapes fit each other (reference: modeling/moe/linearize.py:128-147)."""
    found = []
    for name, module in model.named_modules():
        if isinstance(module, LinearExperts2D):
            continue
        if type(module).__name__ in _SPECIAL_EXPERTS:
            found.append((name, module))
            continue
        gu, dn = getattr(module, "gate_up_proj", None), getattr(module, "down_proj", None)
        if not (isinstance(gu, torch.Tensor) and isinstance(dn, torch.Tensor) and gu.ndim == 3 and dn.ndim == 3
                and gu.shape[0] == dn.shape[0]):
            continue
        if getattr(module, "is_transposed", False):
            fits = gu.shape[2] == 2 * dn.shape[1] and gu.shape[1] == dn.shape[2]
        else:
            fits = gu.shape[1] == 2 * dn.shape[2] and gu.shape[2] == dn.shape[1]
        if fits and _takes_routing_arguments(module):
            found.append((name, module))
    return found


def linearize_moe(model: nn.Module) -> nn.Module:
    """Replace every fused experts module by a ``LinearExperts2D`` of plain Linears, so that per-expert
    weights can be calibrated and quantised (reference: modeling/moe/linearize.py:97-125)."""
    for name, module in get_non_linearized_moes(model):
        cls = _SPECIAL_EXPERTS.get(type(module).__name__, LinearExperts2D)
        model.set_submodule(name, cls.from_experts_module(module))
    return model
