"""Importance-weighted MSE observer (reference: observers/imatrix.py:24-328).

``imatrix_mse``: the shrink-factor search of the MSE observer with the error of every weight multiplied by
E[x^2] of its input channel, collected by a forward-pre hook.  CHANNEL, GROUP and TENSOR_GROUP weight
observers; anything else falls back to the uniform search (or raises with ``strict``)."""
from __future__ import annotations

import logging
import math
from typing import Optional

import torch

from .. import ops
from ..torch_ops import llmc
from ..quantization import QuantizationStrategy
from ..quantization.lifecycle import kernel_format
from .base import Observer, _observed_layout

logger = logging.getLogger("llmcompressor_amd")

__all__ = ["IMatrixMSEObserver"]

_GROUP_STRATEGIES = (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP)
IMATRIX_PRECISION = torch.float32
_warned = set()


def _warn_once(msg: str):
    if msg not in _warned:
        _warned.add(msg)
        logger.warning(msg)


@Observer.register("imatrix_mse")
class IMatrixMSEObserver(Observer):
    _stats_attrs = ["min_vals", "max_vals", "_imatrix_sum", "_imatrix_count"]

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        kw = self.args.observer_kwargs
        self.maxshrink = kw.get("maxshrink", 0.95)
        self.patience = kw.get("patience", 5)
        self.grid = kw.get("grid", 20)
        self.norm = kw.get("norm", 3.0)
        self.strict = kw.get("strict", False)
        self.expand = kw.get("expand", 1.0)
        self._imatrix_sum: Optional[torch.Tensor] = None
        self._imatrix_count = torch.tensor(0, dtype=torch.int64)
        self._imatrix_hook = None
        if self.grid <= 0:
            raise ValueError(f"grid must be > 0, got {self.grid}")
        if self.patience < 0:
            raise ValueError(f"patience must be >= 0, got {self.patience}")
        if not (0 <= self.maxshrink <= 1):
            raise ValueError(f"maxshrink must be in [0, 1], got {self.maxshrink}")
        if not isinstance(self.norm, (int, float)) or not math.isfinite(self.norm) or self.norm <= 0:
            raise ValueError(f"norm must be a finite positive number, got {self.norm}")

    # -- hook lifecycle: E[x^2] per input channel
    def attach(self, module: torch.nn.Module) -> None:
        if self._imatrix_hook is not None:
            self._imatrix_hook.remove()
            self._imatrix_hook = None
        if not hasattr(module, "in_features"):
            return
        param = next(module.parameters(), None)
        device = param.device if param is not None else None
        self._imatrix_sum = torch.zeros(module.in_features, dtype=IMATRIX_PRECISION, device=device)
        self._imatrix_count = torch.tensor(0, dtype=torch.int64, device=device)

        def _hook(_mod, args):
            from ..modifiers.utils.hooks import HooksMixin

            if HooksMixin._HOOKS_DISABLED and self._imatrix_hook not in HooksMixin._HOOKS_KEEP_ENABLED:
                return
            x = args[0] if isinstance(args, tuple) else args
            if isinstance(x, tuple):
                x = x[0]
            if x is None or not isinstance(x, torch.Tensor):
                return
            x = x.detach()
            n_tokens = math.prod(x.shape[:-1])
            self._imatrix_sum = self._imatrix_sum.to(x.device)
            self._imatrix_count = self._imatrix_count.to(x.device)
            llmc.sumsq_accum_(self._imatrix_sum, x.reshape(-1, x.shape[-1]))
            self._imatrix_count += n_tokens

        self._imatrix_hook = module.register_forward_pre_hook(_hook)

    def detach(self, module: torch.nn.Module) -> None:
        if self._imatrix_hook is not None:
            self._imatrix_hook.remove()
            self._imatrix_hook = None

    # -- statistics
    def compute_min_max(self, value):
        (kind, t, p), shape = _observed_layout(value, self.base_name, self.args)
        imp = self._validated_importance(value, kind, t, p)
        if imp is not None:
            imp = imp.to(device=t.device, dtype=torch.float32)
            imp = imp / (imp.mean() + torch.finfo(torch.float32).tiny)
        fmt, bits = kernel_format(self.args)
        mode = ops.SCALE_MXFP4 if self.args.is_mx else ops.SCALE_PLAIN
        kw = dict(maxshrink=self.maxshrink, patience=self.patience, grid=self.grid, norm=self.norm,
                  expand=self.expand)
        if kind == "groups":
            mn, mx = llmc.imatrix_observe(t, p, fmt, bits, self.args.symmetric, mode, importance=imp, **kw)
        elif kind == "blocks":  # no importance here: _validated_importance sent block-wise weights to the fall-back
            mn, mx = llmc.imatrix_observe_blocks(t, p[0], p[1], fmt, bits, self.args.symmetric, mode, **kw)
        else:
            mn, mx = llmc.imatrix_observe_strided(t, *p, fmt, bits, self.args.symmetric, mode, **kw)
        return mn.reshape(shape), mx.reshape(shape)

    def _fallback(self, exc_type, msg: str):
        if self.strict:
            raise exc_type(f"imatrix_mse: {msg}")
        _warn_once(f"imatrix_mse: {msg}. Falling back to uniform MSE.")
        return None

    def _validated_importance(self, value, kind, t, group) -> Optional[torch.Tensor]:
        """The importance vector if it can be used (imatrix.py:141-245), else None (uniform search)."""
        if self.base_name != "weight":
            return self._fallback(NotImplementedError, "only supported for weight observers")
        if self.args.strategy == QuantizationStrategy.TENSOR:
            return self._fallback(NotImplementedError, "TENSOR strategy not supported")
        if self._imatrix_sum is None or int(self._imatrix_count.item()) == 0:
            return self._fallback(ValueError, "no importance data available")
        imp = self._imatrix_sum / self._imatrix_count.float()
        if not bool(torch.isfinite(imp).all()):
            return self._fallback(ValueError, "contains non-finite values")
        if bool((imp < 0).any()):
            return self._fallback(ValueError, "contains negative values")
        if bool(torch.all(imp == 0)):
            return self._fallback(ValueError, "all zeros")
        if self.args.strategy == QuantizationStrategy.CHANNEL or self.args.strategy in _GROUP_STRATEGIES:
            expected = value.shape[-1]
        else:
            return self._fallback(NotImplementedError, f"unsupported strategy {self.args.strategy}")
        if imp.numel() != expected:
            return self._fallback(ValueError, f"size mismatch: expected {expected}, got {imp.numel()}")
        return imp
