"""Oracle: observers (min-max family, MSE grid search) and calibration flattening.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Follows ``src/llmcompressor/observers/helpers.py:28-157`` (flatten),
``observers/min_max.py:10-74``, ``observers/mse.py:12-131``,
``observers/mse_quant.py:19-141,255-285`` (eager search), ``observers/base.py:78-145``
(global scale, qparams) and ``observers/fusion.py:17-105`` (shared global scale).
"""
from __future__ import annotations

import math

import torch

from .qformat import QArgs, calculate_qparams, fake_quantize, generate_gparam


def _pad_for_block(value, block_structure):
    bh, bw = block_structure
    rows, cols = value.shape[-2], value.shape[-1]
    pr, pc = (-rows) % bh, (-cols) % bw
    if pr or pc:
        value = torch.nn.functional.pad(value, (0, pc, 0, pr))
    return value


def flatten_for_calibration(value, base_name: str, args: QArgs):
    """-> (num_observations, *qparam_shape, group_size); helpers.py:28-157."""
    s = args.strategy
    if base_name == "weight":
        if s == "tensor":
            return value.reshape((1, 1, -1))
        if s == "channel":
            return value.unsqueeze(-2).unsqueeze(0)
        if s in ("group", "tensor_group"):
            return value.unflatten(-1, (-1, args.group_size)).unsqueeze(0)
        if s == "block":
            bh, bw = args.block_structure
            value = _pad_for_block(value, args.block_structure)
            rows, cols = value.shape
            return (
                value.reshape(rows // bh, bh, cols // bw, bw)
                .transpose(1, 2)
                .flatten(-2, -1)
                .unsqueeze(0)
            )
        raise ValueError(f"{s} quantization cannot be applied to weights")
    if base_name in ("input", "output"):
        if s == "tensor":
            return value.reshape((-1, 1, value.size(-1)))
        if s == "token":
            return value
        if s in ("group", "tensor_group"):
            return value.flatten(0, 1).unflatten(-1, (-1, args.group_size))
        raise ValueError(f"{s} quantization cannot be applied to activations")
    if base_name in ("q", "k", "v"):
        if s == "tensor":
            return value.transpose(1, 2).flatten(0, 1).flatten(-2, -1).unsqueeze(-2)
        if s == "attn_head":
            return value.transpose(1, 2).flatten(0, 1).unsqueeze(-2).unsqueeze(-2)
        raise ValueError(f"{s} quantization cannot be applied to attention")
    raise ValueError(f"Unknown quantization base name: {base_name}")


def get_min_max(observed):
    """min_max.py:70-74"""
    return torch.amin(observed, dim=(0, -1)), torch.amax(observed, dim=(0, -1))


def lerp(start, end, weight):
    """helpers.py:218-220"""
    return (start * (1.0 - weight)) + (end * weight)


def calculate_error(observed, args: QArgs, token_args: QArgs, mn, mx, norm):
    """mse_quant.py:255-285"""
    scales, zps = calculate_qparams(mn, mx, args, global_scale=None)
    q = fake_quantize(observed, scales.unsqueeze(-1), zps.unsqueeze(-1), token_args).to(
        observed.dtype
    )
    return torch.sum((q - observed).abs().pow(norm), dim=(0, -1))


def grid_search_mse(observed, args: QArgs, maxshrink=0.20, patience=5, grid=100.0, norm=2.4, expand=1.0):
    """Eager shrink-factor search, mse_quant.py:19-141."""
    token_args = args.copy(strategy="token")
    if args.strategy == "tensor_group" and args.scale_dtype is not None:
        args = args.copy(scale_dtype=None)
        token_args = token_args.copy(scale_dtype=None)
    min_val = torch.amin(observed, dim=(0, -1)) * expand
    max_val = torch.amax(observed, dim=(0, -1)) * expand
    best_error = torch.full_like(min_val, torch.finfo(min_val.dtype).max)
    best_min = min_val.clone()
    best_max = max_val.clone()
    no_improve = 0
    for i in range(int(maxshrink * grid)):
        p = 1 - i / grid
        smin = min_val * p
        smax = max_val * p
        err = calculate_error(observed, args, token_args, smin, smax, norm)
        improved = err < best_error
        if torch.any(improved):
            best_error[improved] = err[improved]
            best_min[improved] = smin[improved]
            best_max[improved] = smax[improved]
            no_improve = 0
        else:
            no_improve += 1
            if no_improve >= patience:
                break
    return best_min, best_max


def prepare_importance(imatrix_sum, imatrix_count, observed, args: QArgs):
    """imatrix.py:126-139: E[x^2] per input channel, normalised to mean 1, laid out like ``observed``."""
    imp = imatrix_sum / float(imatrix_count)
    imp = imp.to(torch.float32)
    imp = imp / (imp.mean() + torch.finfo(torch.float32).tiny)
    rows = observed.shape[1]
    return flatten_for_calibration(imp.unsqueeze(0).expand(rows, -1), "weight", args)


def imatrix_grid_search(observed, args: QArgs, maxshrink=0.95, patience=5, grid=20, norm=3.0, expand=1.0,
                        importance_weights=None):
    """Importance-weighted shrink-factor search, imatrix.py:255-328: candidates i = 0..max(1, int(maxshrink*grid))
    inclusive, error |fq(x) - x|^norm formed, weighted and summed in fp32, global early stop only when
    patience > 0.  parity unpinned by reference vectors; pinned by the reference's own property (uniform
    importance == the plain search on fp32 inputs) and a brute-force fp64 argmin in tests/test_oracle_imatrix.py."""
    token_args = args.copy(strategy="token")
    if args.strategy == "tensor_group" and args.scale_dtype is not None:
        args = args.copy(scale_dtype=None)
        token_args = token_args.copy(scale_dtype=None)
    min_val = torch.amin(observed, dim=(0, -1)) * expand
    max_val = torch.amax(observed, dim=(0, -1)) * expand
    best_error = torch.full(min_val.shape, torch.finfo(torch.float32).max, dtype=torch.float32)
    best_min, best_max = min_val.clone(), max_val.clone()
    no_improve = 0
    observed_f = observed.float()
    for i in range(max(1, int(maxshrink * grid)) + 1):
        p = 1 - i / grid
        smin, smax = p * min_val, p * max_val
        scales, zps = calculate_qparams(smin, smax, args, global_scale=None)
        q = fake_quantize(observed, scales.unsqueeze(-1), zps.unsqueeze(-1), token_args).float()
        e = (q - observed_f).abs().pow(norm)
        if importance_weights is not None:
            e = e * importance_weights
        err = e.sum(dim=(0, -1))
        improved = err < best_error
        if torch.any(improved):
            best_error[improved] = err[improved]
            best_min[improved] = smin[improved]
            best_max[improved] = smax[improved]
            no_improve = 0
        else:
            no_improve += 1
            if patience > 0 and no_improve >= patience:
                break
    return best_min, best_max


class Observer:
    """Minimal observer with the reference's statistics / qparams / fusion contract."""

    registry = {}

    def __init__(self, name: str, base_name: str, args: QArgs, **kw):
        self.name = name
        self.base_name = base_name
        self.args = args
        self.kw = dict(args.observer_kwargs or {})
        self.kw.update(kw)
        self.min_vals = None
        self.max_vals = None
        self.fused = []  # other observers sharing the global scale
        self.weight_ref = None
        self._deletion_called = False

    @property
    def has_statistics(self):
        return self.min_vals is not None

    def __call__(self, observed):
        if observed.numel() == 0:
            return self
        if self.base_name == "weight" and self.has_statistics:
            return self
        obs = flatten_for_calibration(observed, self.base_name, self.args)
        self._update(obs)
        self._fused_statistics()
        return self

    def _update(self, obs):
        n, k = self.name, self.kw
        if n in ("memoryless_minmax", "static_minmax", "minmax"):
            mn, mx = get_min_max(obs)
        else:
            if n == "nvfp4_expanded_mse":
                d = dict(expand=1.8, maxshrink=1 - 0.8 / 1.8, grid=200.0, patience=1000)
            else:
                d = dict(expand=1.0, maxshrink=0.20, grid=100.0, patience=5)
            mn, mx = grid_search_mse(
                obs,
                self.args,
                maxshrink=k.get("maxshrink", d["maxshrink"]),
                patience=k.get("patience", d["patience"]),
                grid=k.get("grid", d["grid"]),
                norm=k.get("norm", 2.4),
                expand=k.get("expand", d["expand"]),
            )
        if n == "static_minmax" and self.has_statistics:
            mn = torch.min(mn, self.min_vals)
            mx = torch.max(mx, self.max_vals)
        if n in ("minmax", "mse") and self.has_statistics:
            c = k.get("averaging_constant", 0.01)
            if c != 1.0:
                mn = lerp(self.min_vals, mn, c)
                mx = lerp(self.max_vals, mx, c)
        self.min_vals, self.max_vals = mn, mx

    # fusion.py:60-79
    def _fused_statistics(self):
        group = [self] + self.fused
        for o in group:
            if not o.has_statistics:
                assert o.weight_ref is not None
                o(o.weight_ref)
        return [(o.min_vals, o.max_vals) for o in group]

    @staticmethod
    def fuse(observers_and_weights):
        pairs = list(observers_and_weights)
        for o, w in pairs:
            o.weight_ref = w
        for o, _ in pairs:
            o.fused = [p for p, _ in pairs if p is not o]

    # base.py:78-96
    def get_global_scale(self):
        if self.args.strategy != "tensor_group":
            return None
        stats = self._fused_statistics()
        absmax = stats[0][1].max()
        for mn, mx in stats:
            absmax = torch.max(absmax, -mn.min())
            absmax = torch.max(absmax, mx.max())
        return generate_gparam(-absmax.reshape(1), absmax.reshape(1))

    # base.py:98-123
    def get_qparams(self):
        assert self.has_statistics, "No statistics available. Call observer(value) first."
        gs = self.get_global_scale()
        scale, zp = calculate_qparams(self.min_vals, self.max_vals, self.args, global_scale=gs)
        self.delete_statistics()
        return {"scale": scale, "zero_point": zp, "global_scale": gs}

    # fusion.py:81-101
    def delete_statistics(self, check_fused=True):
        if not check_fused or not self.fused:
            self.min_vals = self.max_vals = None
            return
        self._deletion_called = True
        if all(o._deletion_called for o in self.fused):
            for o in [self] + self.fused:
                o._deletion_called = False
                o.min_vals = o.max_vals = None


def weight_observer_name(name: str) -> str:
    """weights always use the memoryless variants; calibration.py:65-78"""
    if name in ("static_minmax", "minmax"):
        return "memoryless_minmax"
    if name == "mse":
        return "memoryless_mse"
    return name


def num_groups(cols, group_size):
    return math.ceil(cols / group_size)
