"""``torch.ops.llmc.*``: the C ABI of ``libllmc_amd.so`` registered with the torch dispatcher.

Every op is a thin shim: the registered implementation (``ops.py``) extracts ``data_ptr``, sizes, strides and
the current HIP stream from its tensor arguments and calls one plain ``extern "C"`` function of the library.
The ops are registered for the CUDA (= HIP on ROCm) dispatch key only.  There is no CPU implementation on
purpose: a call with host tensors fails in the dispatcher ("could not run 'llmc::...' with arguments from the
'CPU' backend") instead of silently computing somewhere else.

Seams of the reference that the ops stand behind (src/llmcompressor/...):
``hessian_accum_`` -> accumulate_hessian (modifiers/gptq/gptq_quantize.py:28-64);
``gptq_prepare_hinv_`` / ``gptq_quantize`` -> quantize_weight (:144-164 / :167-250);
``minmax_observe*`` -> _get_min_max (observers/min_max.py:70-74); ``mse_observe*`` -> _grid_search_mse
(observers/mse_quant.py:19-141); ``qparams`` / ``global_scale`` -> Observer.get_qparams / get_global_scale
(observers/base.py:78-123); ``quant_pack`` -> fake_quantize / quantize / the compressors' pack step;
``fp8_dynamic_per_token`` -> forward_quantize with strategy "token" (modifiers/quantization/calibration.py:178-183).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import ops as _impl

NAMESPACE = "llmc"

_defs = torch.library.Library(NAMESPACE, "DEF")
_cuda = torch.library.Library(NAMESPACE, "IMPL", "CUDA")

OP_NAMES: List[str] = []


def _register(schema: str, fn) -> None:
    name = schema.split("(", 1)[0]
    _defs.define(schema)
    _cuda.impl(name, fn)
    OP_NAMES.append(name)


# ---- GPTQ Hessian --------------------------------------------------------------------------------------------

def _hessian_accum_(H, X, alpha=2.0, assume_symmetric=True):
    _impl.hessian_accumulate_(H, X, alpha=alpha, assume_symmetric=assume_symmetric)


def _hessian_accum_segments_(H, Xs, alpha=2.0, assume_symmetric=True):
    _impl.hessian_accumulate_segments_(H, list(Xs), alpha=alpha, assume_symmetric=assume_symmetric)


def _hessian_accum_grouped_(Hs, Xs, alpha=2.0, assume_symmetric=True):
    _impl.hessian_accumulate_grouped_(list(Hs), list(Xs), alpha=alpha, assume_symmetric=assume_symmetric)


_register("hessian_accum_(Tensor(a!) H, Tensor X, float alpha=2.0, bool assume_symmetric=True) -> ()", _hessian_accum_)
_register("hessian_accum_segments_(Tensor(a!) H, Tensor[] Xs, float alpha=2.0, bool assume_symmetric=True) -> ()",
          _hessian_accum_segments_)
_register("hessian_accum_grouped_(Tensor(a!)[] Hs, Tensor[] Xs, float alpha=2.0, bool assume_symmetric=True) -> ()",
          _hessian_accum_grouped_)


# ---- damped Cholesky chain and the column loop ------------------------------------------------------------------

def _gptq_prepare_hinv_(H, perm=None, divisor=1.0, percdamp=0.01, form=0):
    _, dead, info = _impl.gptq_hinv_(H, perm, divisor=divisor, percdamp=percdamp, form=form)
    return dead, info


def _gptq_prepare_hinv_grouped(Hs, perms=None, divisors=None, percdamp=0.01, form=0):
    return _impl.gptq_hinv_grouped(list(Hs), perms, None if divisors is None else list(divisors), percdamp, form=form)


def _gptq_quantize(W, Hinv, scale, zero_point, fmt, num_bits, row_div, scale_row_stride, g_idx=None, perm=None,
                   dead=None, global_scale=None, blocksize=128, form=0):
    return _impl.gptq_quantize(W, Hinv, scale, zero_point, fmt, num_bits, row_div, scale_row_stride, g_idx=g_idx,
                               perm=perm, dead=dead, global_scale=global_scale, blocksize=blocksize, form=form)


def _gptq_quantize_grouped(Ws, Hinv, scales, zero_points, fmt, num_bits, row_div, scale_row_stride, g_idxs=None,
                           perms=None, dead=None, global_scales=None, blocksize=128, form=0):
    outs, loss = _impl.gptq_quantize_grouped(
        list(Ws), Hinv, list(scales), None if zero_points is None else list(zero_points), fmt, num_bits, row_div,
        scale_row_stride, g_idxs=None if g_idxs is None else list(g_idxs), perms=perms, dead=dead,
        global_scales=None if global_scales is None else list(global_scales), blocksize=blocksize, form=form)
    return outs, loss


def _sparsegpt_sparsify(W, Hinv, sparsity, prune_n=0, prune_m=0, dead=None, blocksize=128,
                        preserve_sparsity_mask=False, form=0):
    return _impl.sparsegpt_sparsify(W, Hinv, sparsity, prune_n=prune_n, prune_m=prune_m, dead=dead,
                                    blocksize=blocksize, preserve_sparsity_mask=preserve_sparsity_mask, form=form)


_register("gptq_prepare_hinv_(Tensor(a!) H, Tensor? perm=None, float divisor=1.0, float percdamp=0.01, int form=0) "
          "-> (Tensor dead, Tensor info)", _gptq_prepare_hinv_)
_register("gptq_prepare_hinv_grouped(Tensor[] Hs, Tensor? perms=None, float[]? divisors=None, float percdamp=0.01, "
          "int form=0) "
          "-> (Tensor U, Tensor dead, Tensor info)", _gptq_prepare_hinv_grouped)
_register("gptq_quantize(Tensor W, Tensor Hinv, Tensor scale, Tensor? zero_point, int fmt, int num_bits, int row_div, "
          "int scale_row_stride, Tensor? g_idx=None, Tensor? perm=None, Tensor? dead=None, Tensor? global_scale=None, "
          "int blocksize=128, int form=0) -> (Tensor weight, Tensor loss)", _gptq_quantize)
_register("gptq_quantize_grouped(Tensor[] Ws, Tensor Hinv, Tensor[] scales, Tensor[]? zero_points, int fmt, "
          "int num_bits, int row_div, int scale_row_stride, Tensor[]? g_idxs=None, Tensor? perms=None, "
          "Tensor? dead=None, Tensor[]? global_scales=None, int blocksize=128, int form=0) "
          "-> (Tensor[] weights, Tensor loss)",
          _gptq_quantize_grouped)
_register("sparsegpt_sparsify(Tensor W, Tensor Hinv, float sparsity, int prune_n=0, int prune_m=0, Tensor? dead=None, "
          "int blocksize=128, bool preserve_sparsity_mask=False, int form=0) -> (Tensor weight, Tensor loss)",
          _sparsegpt_sparsify)


# ---- observers ---------------------------------------------------------------------------------------------------

def _minmax_observe(W, group):
    return _impl.minmax_groups(W, group)


def _minmax_observe_blocks(W, block_h, block_w):
    return _impl.minmax_blocks(W, block_h, block_w)


def _minmax_observe_strided(x, n0, n1, group, stride0, stride1):
    return _impl.minmax_strided(x, n0, n1, group, stride0, stride1)


def _mse_observe(W, group, fmt, num_bits, symmetric, scale_mode=0, maxshrink=0.20, patience=5, grid=100.0, norm=2.4,
                 expand=1.0):
    return _impl.mse_observe_groups(W, group, fmt, num_bits, symmetric, scale_mode, maxshrink=maxshrink,
                                    patience=patience, grid=grid, norm=norm, expand=expand)


def _mse_observe_blocks(W, block_h, block_w, fmt, num_bits, symmetric, scale_mode=0, maxshrink=0.20, patience=5,
                        grid=100.0, norm=2.4, expand=1.0):
    return _impl.mse_observe_blocks(W, block_h, block_w, fmt, num_bits, symmetric, scale_mode, maxshrink=maxshrink,
                                    patience=patience, grid=grid, norm=norm, expand=expand)


def _mse_observe_strided(x, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode=0, maxshrink=0.20,
                         patience=5, grid=100.0, norm=2.4, expand=1.0):
    return _impl.mse_observe_strided(x, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode,
                                     maxshrink=maxshrink, patience=patience, grid=grid, norm=norm, expand=expand)


def _sumsq_accum_(total, x):
    _impl.sumsq_accumulate_(total, x)


def _sumsq_accum_noalloc_(total, x):
    _impl.sumsq_accumulate_noalloc_(total, x)


def _imatrix_observe(W, group, fmt, num_bits, symmetric, scale_mode=0, importance=None, maxshrink=0.95, patience=5,
                     grid=20.0, norm=3.0, expand=1.0):
    return _impl.imatrix_observe_groups(W, group, fmt, num_bits, symmetric, scale_mode, importance=importance,
                                        maxshrink=maxshrink, patience=patience, grid=grid, norm=norm, expand=expand)


def _imatrix_observe_blocks(W, block_h, block_w, fmt, num_bits, symmetric, scale_mode=0, maxshrink=0.95, patience=5,
                            grid=20.0, norm=3.0, expand=1.0):
    return _impl.imatrix_observe_blocks(W, block_h, block_w, fmt, num_bits, symmetric, scale_mode,
                                        maxshrink=maxshrink, patience=patience, grid=grid, norm=norm, expand=expand)


def _imatrix_observe_strided(x, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode=0,
                             maxshrink=0.95, patience=5, grid=20.0, norm=3.0, expand=1.0):
    return _impl.imatrix_observe_strided(x, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode,
                                         maxshrink=maxshrink, patience=patience, grid=grid, norm=norm, expand=expand)


_SEARCH = ("int fmt, int num_bits, bool symmetric, int scale_mode=0, float maxshrink=0.20, int patience=5, "
           "float grid=100.0, float norm=2.4, float expand=1.0) -> (Tensor min, Tensor max)")
_ISEARCH = ("float maxshrink=0.95, int patience=5, float grid=20.0, float norm=3.0, float expand=1.0) "
            "-> (Tensor min, Tensor max)")
_register("minmax_observe(Tensor W, int group) -> (Tensor min, Tensor max)", _minmax_observe)
_register("minmax_observe_blocks(Tensor W, int block_h, int block_w) -> (Tensor min, Tensor max)", _minmax_observe_blocks)
_register("minmax_observe_strided(Tensor x, int n0, int n1, int group, int stride0, int stride1) "
          "-> (Tensor min, Tensor max)", _minmax_observe_strided)
_register("mse_observe(Tensor W, int group, " + _SEARCH, _mse_observe)
_register("mse_observe_blocks(Tensor W, int block_h, int block_w, " + _SEARCH, _mse_observe_blocks)
_register("mse_observe_strided(Tensor x, int n0, int n1, int group, int stride0, int stride1, " + _SEARCH,
          _mse_observe_strided)
_register("sumsq_accum_(Tensor(a!) total, Tensor x) -> ()", _sumsq_accum_)
_register("sumsq_accum_noalloc_(Tensor(a!) total, Tensor x) -> ()", _sumsq_accum_noalloc_)
_register("imatrix_observe(Tensor W, int group, int fmt, int num_bits, bool symmetric, int scale_mode=0, "
          "Tensor? importance=None, " + _ISEARCH, _imatrix_observe)
_register("imatrix_observe_blocks(Tensor W, int block_h, int block_w, int fmt, int num_bits, bool symmetric, "
          "int scale_mode=0, " + _ISEARCH, _imatrix_observe_blocks)
_register("imatrix_observe_strided(Tensor x, int n0, int n1, int group, int stride0, int stride1, int fmt, "
          "int num_bits, bool symmetric, int scale_mode=0, " + _ISEARCH, _imatrix_observe_strided)


# ---- qparams, quantise, pack ---------------------------------------------------------------------------------------

def _global_scale(mins, maxs):
    return _impl.global_scale_from_stats(list(zip(mins, maxs)))


def _qparams(min_vals, max_vals, fmt, num_bits, symmetric, scale_mode=0, global_scale=None, want_codes=False):
    return _impl.calculate_qparams(min_vals, max_vals, fmt, num_bits, symmetric, scale_mode, global_scale, want_codes)


def _quant_pack(x, scale, zero_point, fmt, num_bits, row_div, scale_row_stride, col_div, out_mode=0, g_idx=None,
                global_scale=None, out_dtype=None):
    return _impl.quantize(x, scale, zero_point, fmt, num_bits, row_div, scale_row_stride, col_div, out_mode=out_mode,
                          g_idx=g_idx, global_scale=global_scale, out_dtype=out_dtype)


def _fp8_dynamic_per_token(X, fmt=1, num_bits=8, out_mode=0):
    return _impl.dynamic_per_token_quantize(X, fmt, num_bits, out_mode)


_register("global_scale(Tensor[] mins, Tensor[] maxs) -> Tensor", _global_scale)
_register("qparams(Tensor min_vals, Tensor max_vals, int fmt, int num_bits, bool symmetric, int scale_mode=0, "
          "Tensor? global_scale=None, bool want_codes=False) -> (Tensor scale, Tensor zero_point, Tensor? scale_code)",
          _qparams)
_register("quant_pack(Tensor x, Tensor scale, Tensor? zero_point, int fmt, int num_bits, int row_div, "
          "int scale_row_stride, int col_div, int out_mode=0, Tensor? g_idx=None, Tensor? global_scale=None, "
          "ScalarType? out_dtype=None) -> Tensor", _quant_pack)
_register("fp8_dynamic_per_token(Tensor X, int fmt=1, int num_bits=8, int out_mode=0) -> (Tensor out, Tensor scale)",
          _fp8_dynamic_per_token)

llmc = getattr(torch.ops, NAMESPACE)
