"""Observer base class and registry (reference: observers/base.py:29-206).

Statistics come from the HIP min-max / MSE kernels and qparams from the HIP qparams
kernel; the class keeps the reference's names and lifecycle: ``forward(observed)``,
``update_statistics_from_observed``, ``get_qparams() -> {scale, zero_point,
global_scale}``, ``get_global_scale``, ``delete_statistics``, ``Observer.register`` /
``Observer.load_from_registry``.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple, TypedDict

import torch

from .. import ops
from ..torch_ops import llmc
from ..quantization import QuantizationArgs, QuantizationStrategy, calculate_qparams, generate_gparam
from .fusion import FusionHandler
from .helpers import flatten_for_calibration

__all__ = ["Observer", "MinMaxTuple", "QParamsDict"]

MinMaxTuple = Tuple[torch.Tensor, torch.Tensor]


class QParamsDict(TypedDict, total=False):
    scale: torch.Tensor
    zero_point: torch.Tensor
    global_scale: Optional[torch.Tensor]


def _observed_layout(value: torch.Tensor, base_name: str, args: QuantizationArgs):
    """How the flattened view ``(n0, *qshape, G)`` of ``value`` maps onto the kernels.

    Returns ("groups", w2d, group) | ("blocks", w2d, (bh, bw)) | ("strided", x, (n0, n1, G, s0, s1)),
    plus the shape the statistics must take.
    """
    S = QuantizationStrategy
    s = args.strategy
    if base_name == "weight":
        w = value if value.is_contiguous() else value.contiguous()
        w2 = w.reshape(-1, w.shape[-1])
        if s == S.TENSOR:
            return ("groups", w2.reshape(1, -1), w2.numel()), (1,)
        if s == S.CHANNEL:
            return ("groups", w2, w2.shape[1]), (w2.shape[0], 1)
        if s in (S.GROUP, S.TENSOR_GROUP):
            if w2.shape[1] % args.group_size != 0:
                raise ValueError(f"weight columns {w2.shape[1]} are not divisible by group_size {args.group_size}")
            return ("groups", w2, args.group_size), (w2.shape[0], w2.shape[1] // args.group_size)
        if s == S.BLOCK:
            bh, bw = args.block_structure
            return ("blocks", w2, (bh, bw)), (-(-w2.shape[0] // bh), -(-w2.shape[1] // bw))
        flatten_for_calibration(value, base_name, args)  # raises the reference's error
    if base_name in ("input", "output"):
        x = value if value.is_contiguous() else value.contiguous()
        if x.ndim == 1:
            x = x.unsqueeze(0)
        if x.ndim == 2:
            x = x.unsqueeze(0)
        K = x.shape[-1]
        if s == S.TENSOR:
            return ("groups", x.reshape(1, -1), x.numel()), (1,)
        if s == S.TOKEN:
            x3 = x.reshape(x.shape[0], -1, K)
            return ("strided", x3, (x3.shape[0], x3.shape[1], K, x3.shape[1] * K, K)), (x3.shape[1],)
        if s in (S.GROUP, S.TENSOR_GROUP):
            g = args.group_size
            if K % g != 0:  # the reference's unflatten into (K // g, g) raises here as well
                raise ValueError(f"activation width {K} is not divisible by group_size {g}")
            n0 = x.numel() // K
            return ("strided", x, (n0, K // g, g, K, g)), (K // g,)
        flatten_for_calibration(value, base_name, args)
    if base_name in ("q", "k", "v"):
        x = value if value.is_contiguous() else value.contiguous()
        if s == S.TENSOR:
            return ("groups", x.reshape(1, -1), x.numel()), (1,)
        if s == S.ATTN_HEAD:
            B, H, T, D = x.shape
            return ("strided", x, (B, H, T * D, H * T * D, T * D)), (H, 1, 1)
        flatten_for_calibration(value, base_name, args)
    raise ValueError(f"Unknown quantization base name: {base_name}")


class Observer(torch.nn.Module):
    """Computes quantization parameters from observations of weights, activations or attention states."""

    _registry: Dict[str, type] = {}
    _act_sync_dict: Dict[str, object] = {}
    _stats_attrs: List[str] = ["min_vals", "max_vals"]

    # -- registry (compressed-tensors RegistryMixin contract)
    @classmethod
    def register(cls, name: str, alias=None):
        def deco(klass):
            names = [name] + ([alias] if isinstance(alias, str) else list(alias or []))
            for n in names:
                Observer._registry[n.lower().replace("-", "_")] = klass
            return klass

        return deco

    @classmethod
    def get_value_from_registry(cls, name: str):
        key = name.lower().replace("-", "_")
        if key not in Observer._registry:
            raise KeyError(f"Unable to find {name} registered under type Observer. "
                           f"Registered values: {sorted(Observer._registry)}")
        return Observer._registry[key]

    @classmethod
    def load_from_registry(cls, name: str, **constructor_kwargs):
        return cls.get_value_from_registry(name)(**constructor_kwargs)

    def __init__(self, base_name: str, args: QuantizationArgs, **observer_kwargs):
        super().__init__()
        self.base_name = base_name
        self.args = args
        self.args.observer_kwargs = self.args.observer_kwargs or {}
        self.args.observer_kwargs.update(observer_kwargs)
        self.fusion_handler = FusionHandler(self)

    @property
    def has_statistics(self) -> bool:
        return all(hasattr(self, a) for a in self._stats_attrs)

    @property
    def is_weight_obs(self) -> bool:
        return self.base_name == "weight"

    # -- statistics
    def _min_max_kernel(self, value: torch.Tensor) -> MinMaxTuple:
        """min/max over dims (0,-1) of the calibration view of ``value``; subclasses may search instead."""
        (kind, t, p), shape = _observed_layout(value, self.base_name, self.args)
        if kind == "groups":
            mn, mx = llmc.minmax_observe(t, p)
        elif kind == "blocks":
            mn, mx = llmc.minmax_observe_blocks(t, *p)
        else:
            mn, mx = llmc.minmax_observe_strided(t, *p)
        return mn.reshape(shape), mx.reshape(shape)

    def compute_min_max(self, value: torch.Tensor) -> MinMaxTuple:
        return self._min_max_kernel(value)

    def update_statistics(self, min_vals: torch.Tensor, max_vals: torch.Tensor) -> None:
        """Fold a fresh (min, max) into the running statistics (memoryless: replace)."""
        self.min_vals, self.max_vals = min_vals, max_vals

    def update_statistics_from_observed(self, observed: torch.Tensor) -> None:
        """Reference entry point: ``observed`` is already flattened to (num_observations, *qparam_shape, group)."""
        n0, G = observed.shape[0], observed.shape[-1]
        qshape = tuple(observed.shape[1:-1])
        flat = observed.reshape(n0, -1, G)
        flat = flat if flat.is_contiguous() else flat.contiguous()
        n1 = flat.shape[1]
        if n0 == 1:
            mn, mx = self._rows(flat.reshape(n1, G))
        else:
            mn, mx = self._strided(flat, n0, n1, G)
        self.update_statistics(mn.reshape(qshape), mx.reshape(qshape))

    def _rows(self, rows2d):
        mn, mx = llmc.minmax_observe(rows2d, rows2d.shape[1])
        return mn, mx

    def _strided(self, flat, n0, n1, G):
        return llmc.minmax_observe_strided(flat, n0, n1, G, n1 * G, G)

    def get_global_scale(self) -> Optional[torch.Tensor]:
        if self.args.strategy != QuantizationStrategy.TENSOR_GROUP:
            return None
        all_stats = self.fusion_handler.get_fused_statistics()
        return generate_gparam([(s["min_vals"], s["max_vals"]) for s in all_stats])

    @torch.no_grad()
    def get_qparams(self) -> QParamsDict:
        assert self.has_statistics, "No statistics available. Call observer(value) first."
        global_scale = self.get_global_scale()
        scale, zero_point = calculate_qparams(
            min_vals=self.min_vals, max_vals=self.max_vals, quantization_args=self.args, global_scale=global_scale
        )
        self.delete_statistics()
        return {"scale": scale, "zero_point": zero_point, "global_scale": global_scale}

    @torch.no_grad()
    def forward(self, observed: torch.Tensor) -> "Observer":
        if observed.numel() == 0:
            return self
        if self.is_weight_obs and self.has_statistics:
            return self
        mn, mx = self.compute_min_max(observed)
        self.update_statistics(mn, mx)
        self.fusion_handler.get_fused_statistics()
        return self

    def sync_activation_stats(self) -> list:
        """Single-GPU build: nothing to all-reduce (reference: observers/base.py:147-162)."""
        return []

    def delete_statistics(self, check_fused: bool = True) -> None:
        if check_fused:
            self.fusion_handler.maybe_delete_statistics()
        else:
            for attr in self._stats_attrs:
                if hasattr(self, attr):
                    delattr(self, attr)

    def get_statistics(self) -> dict[str, torch.Tensor]:
        assert self.has_statistics, "No statistics available. Call observer(value) first."
        return {attr: getattr(self, attr) for attr in self._stats_attrs}

    def attach(self, module: torch.nn.Module) -> None:
        pass

    def detach(self, module: torch.nn.Module) -> None:
        pass
