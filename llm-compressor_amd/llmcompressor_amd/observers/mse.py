"""MSE observers (reference: observers/mse.py:12-131, observers/mse_quant.py:19-141)."""
import torch

from .. import ops
from ..torch_ops import llmc
from ..quantization import QuantizationStrategy
from ..quantization.lifecycle import kernel_format
from .base import Observer, _observed_layout
from .helpers import lerp

__all__ = ["MemorylessMSEObserver", "MovingAverageMSEObserver", "NVFP4ExpandedMSEObserver"]


@Observer.register("memoryless_mse")
class MemorylessMSEObserver(Observer):
    """min/max minimising |fq(x) - x|^norm over a grid of shrink factors."""

    _defaults = dict(maxshrink=0.20, patience=5, grid=100.0, norm=2.4, chunk_size=5, expand=1.0)

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        kw = self.args.observer_kwargs
        d = self._defaults
        self.maxshrink = kw.get("maxshrink", d["maxshrink"])
        self.patience = kw.get("patience", d["patience"])
        self.grid = kw.get("grid", d["grid"])
        self.norm = kw.get("norm", d["norm"])
        self.chunk_size = kw.get("chunk_size", d["chunk_size"])
        self.expand = kw.get("expand", d["expand"])
        if self.chunk_size <= 0:
            raise ValueError(f"chunk_size must be positive, got {self.chunk_size}")
        if self.expand < 1.0:
            raise ValueError(f"expand value must be at least 1.0, got {self.expand}")

    def _search_kwargs(self):
        return dict(maxshrink=self.maxshrink, patience=self.patience, grid=self.grid, norm=self.norm,
                    expand=self.expand)

    def compute_min_max(self, value):
        (kind, t, p), shape = _observed_layout(value, self.base_name, self.args)
        fmt, bits = kernel_format(self.args)
        # the search runs with plain scales; only MXFP4 keeps its power-of-two scale rule
        mode = ops.SCALE_MXFP4 if self.args.is_mx else ops.SCALE_PLAIN
        kw = self._search_kwargs()
        if kind == "groups":
            mn, mx = llmc.mse_observe(t, p, fmt, bits, self.args.symmetric, mode, **kw)
        elif kind == "blocks":
            mn, mx = llmc.mse_observe_blocks(t, p[0], p[1], fmt, bits, self.args.symmetric, mode, **kw)
        else:
            mn, mx = llmc.mse_observe_strided(t, *p, fmt, bits, self.args.symmetric, mode, **kw)
        return mn.reshape(shape), mx.reshape(shape)

    def _rows(self, rows2d):
        fmt, bits = kernel_format(self.args)
        mode = ops.SCALE_MXFP4 if self.args.is_mx else ops.SCALE_PLAIN
        return llmc.mse_observe(rows2d, rows2d.shape[1], fmt, bits, self.args.symmetric, mode, **self._search_kwargs())

    def _strided(self, flat, n0, n1, G):
        fmt, bits = kernel_format(self.args)
        mode = ops.SCALE_MXFP4 if self.args.is_mx else ops.SCALE_PLAIN
        return llmc.mse_observe_strided(flat, n0, n1, G, n1 * G, G, fmt, bits, self.args.symmetric, mode,
                                        **self._search_kwargs())


@Observer.register("mse")
class MovingAverageMSEObserver(MemorylessMSEObserver):
    """MSE search with exponential moving average of the found ranges."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.avg_constant = self.args.observer_kwargs.get("averaging_constant", 0.01)

    def update_statistics(self, min_vals, max_vals):
        if hasattr(self, "min_vals") and self.avg_constant != 1.0:
            min_vals = lerp(self.min_vals, min_vals, self.avg_constant)
            max_vals = lerp(self.max_vals, max_vals, self.avg_constant)
        self.min_vals, self.max_vals = min_vals, max_vals


@Observer.register("nvfp4_expanded_mse")
class NVFP4ExpandedMSEObserver(MemorylessMSEObserver):
    """Searches from 1.8x down to ~0.8x of the observed range in 112 steps."""

    _defaults = dict(maxshrink=1 - 0.8 / 1.8, patience=1000, grid=200.0, norm=2.4, chunk_size=5, expand=1.8)
