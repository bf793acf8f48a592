"""GPTQ numerics behind the reference's function seams (modifiers/gptq/gptq_quantize.py).

``make_empty_hessian`` (:19-25), ``accumulate_hessian`` (:28-64) and ``quantize_weight``
(:67-264) keep their names, arguments, return values and error behaviour; the work is done
by the HIP kernels: ``llmc_hessian_accumulate`` (MFMA SYRK), ``llmc_gptq_hinv`` (damped
Cholesky chain, identity fallback on a non-positive pivot) and ``llmc_gptq_quantize``
(block column loop + MFMA trailing updates).
"""
from __future__ import annotations

import logging
import math

import torch

from ... import ops  # noqa: F401  (format constants)
from ...torch_ops import llmc
from ...quantization import ActivationOrdering, QuantizationArgs, QuantizationStrategy
from ...quantization.lifecycle import effective_scale, kernel_format

logger = logging.getLogger("llmcompressor_amd")

GPTQ_PRECISION = torch.float32

__all__ = ["make_empty_hessian", "accumulate_hessian", "quantize_weight", "quantize_weight_tensors",
           "quantize_weight_group", "begin_weight_group", "finish_weight_group", "group_key", "width_key"]


def make_empty_hessian(module: torch.nn.Module, device: torch.device | None = None) -> torch.Tensor:
    weight = module.weight
    num_columns = weight.shape[1]
    device = device if device is not None else weight.device
    return torch.zeros((num_columns, num_columns), device=device, dtype=GPTQ_PRECISION)


def accumulate_hessian(inp: torch.Tensor, module: torch.nn.Module, H: torch.Tensor | None,
                       num_samples: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """H += 2 X^T X in place; num_samples += batch entries (not tokens)."""
    inp = inp.to(device=H.device)
    if len(inp.shape) == 2:
        inp = inp.unsqueeze(0)
    elif len(inp.shape) > 3:
        inp = inp.reshape(inp.shape[0], -1, inp.shape[-1])
    num_added = inp.shape[0]
    if isinstance(module, torch.nn.Conv2d):
        unfold = torch.nn.Unfold(module.kernel_size, dilation=module.dilation, padding=module.padding,
                                 stride=module.stride)
        inp = unfold(inp).permute([1, 0, 2]).flatten(1).t()
    else:  # Linear / Conv1D: rows are tokens
        inp = inp.reshape((-1, inp.shape[-1]))
    num_samples += num_added
    if inp.shape[0] > 0:
        llmc.hessian_accum_(H, inp.contiguous(), 2.0, True)
    return H, num_samples


def _diag_order(Hs) -> torch.Tensor:
    """[n, K] column orders of the activation ordering: ``argsort(diag H, descending, stable)`` per Hessian (stable:
    equal diagonal entries keep their column order, so the order and with it the result is reproducible; torch
    leaves the order of ties unspecified otherwise).  One launch for Hessians the kernel takes, torch otherwise."""
    H0 = Hs[0]
    if (H0.is_cuda and H0.shape[0] <= ops.DIAG_ORDER_MAX_K
            and all(H.dtype == torch.float32 and H.stride(1) == 1 and H.stride(0) == H0.stride(0) for H in Hs)):
        return ops.diag_argsort_desc(Hs)
    return torch.argsort(torch.stack([torch.diagonal(H) for H in Hs]), dim=1, descending=True, stable=True)


def _scale_layout(strategy, quant_args: QuantizationArgs, num_rows: int, num_columns: int):
    """(row_div, scale_row_stride, base g_idx or None) of llmc_gptq_quantize."""
    S = QuantizationStrategy
    if strategy == S.TENSOR:
        return 1 << 40, 0, None
    if strategy == S.CHANNEL:
        return 1, 1, None
    if strategy in (S.GROUP, S.TENSOR_GROUP):
        return 1, math.ceil(num_columns / quant_args.group_size), quant_args.group_size
    if strategy == S.BLOCK:
        bh, bw = quant_args.block_structure
        return bh, math.ceil(num_columns / bw), bw
    raise ValueError(f"Quantization strategy is not supported for GPTQ: {strategy}")


def quantize_weight_tensors(weight: torch.Tensor, observer, quant_args: QuantizationArgs, hessian: torch.Tensor,
                            blocksize: int = 128, percdamp: float = 0.01, hessian_divisor: float = 1.0):
    """quantize_weight on bare tensors: ``weight`` [R,K], ``observer`` holding its statistics.

    ``hessian_divisor`` folds the caller's ``H / num_samples`` into the factorisation's first pass."""
    strategy = quant_args.strategy
    actorder = quant_args.actorder
    final_shape, final_dtype = weight.shape, weight.dtype
    W2 = weight.reshape(weight.shape[0], -1) if weight.ndim != 2 else weight
    if not W2.is_contiguous():
        W2 = W2.contiguous()
    num_rows, num_columns = W2.shape
    H = hessian

    if actorder == ActivationOrdering.GROUP and strategy not in (QuantizationStrategy.GROUP,
                                                                 QuantizationStrategy.TENSOR_GROUP):
        logger.warning("ActivationOrdering.GROUP requires a grouped quantization strategy; "
                       "falling back to actorder=None for this module.")
        actorder = None

    perm = None
    if actorder:
        # stable: equal diagonal entries keep their column order, so that the column order (and with it the
        # result) is reproducible; torch leaves the order of ties unspecified otherwise
        perm = _diag_order([H])[0]
    if actorder == ActivationOrdering.GROUP:
        # re-observe the permuted weight so that groups are runs of the permuted columns.  The reference observes
        # its fp32 work copy here (gptq_quantize.py:88,111-114), so these statistics and the scales the column
        # loop divides by are fp32, not rounded to the weight's dtype as on the other paths
        observer.delete_statistics(check_fused=False)
        observer(W2[:, perm].to(GPTQ_PRECISION).contiguous())

    row_div, srow, divisor = _scale_layout(strategy, quant_args, num_rows, num_columns)
    g_idx = None
    if divisor is not None:
        g_idx = torch.arange(num_columns, device=W2.device, dtype=torch.int) // divisor
        if actorder == ActivationOrdering.WEIGHT:
            g_idx = g_idx[perm]

    qparams = observer.get_qparams()
    scale, zero_point, global_scale = qparams["scale"], qparams["zero_point"], qparams["global_scale"]

    # dead columns, damping, Cholesky -> inverse -> upper factor; identity on failure
    # (where the width allows it the chain stops at the Cholesky factor of H outside 512-column diagonal blocks
    # and the column loop works from that: same result up to fp32 rounding, a third less arithmetic in the chain)
    form = ops.gptq_factor_form(num_columns, blocksize)
    dead, info = llmc.gptq_prepare_hinv_(H, perm, float(hessian_divisor), float(percdamp), form)
    U = H  # overwritten in place by the factor

    fmt, bits = kernel_format(quant_args)
    zp = None if quant_args.symmetric else zero_point.to(torch.int8)
    kscale = effective_scale(scale, quant_args, final_dtype)
    Wq, loss = llmc.gptq_quantize(W2, U, kscale, zp, fmt, bits, row_div, srow, g_idx=g_idx, perm=perm, dead=dead,
                                  global_scale=global_scale, blocksize=blocksize, form=form)
    if int(info.item()) != 0:
        logger.warning("Failed to invert hessian due to numerical instability. Consider increasing "
                       "GPTQModifier.dampening_frac, increasing the number of calibration samples, or shuffling "
                       "the calibration dataset. Falling back to round-to-nearest for this module.")
    W = Wq.reshape(final_shape)
    q_param_dict = {
        "weight": W,
        "weight_scale": scale if scale.dtype in (torch.uint8, torch.float8_e4m3fn) else scale.to(dtype=final_dtype),
        "weight_zero_point": zero_point.to(dtype=quant_args.zp_dtype),
    }
    if quant_args.scale_dtype == torch.float8_e4m3fn and scale.dtype == torch.float32:
        q_param_dict["weight_scale"] = scale  # e4m3-grid values; stored as float8 by the parameter
    if global_scale is not None:
        q_param_dict["weight_global_scale"] = global_scale.to(dtype=final_dtype)
    if actorder == ActivationOrdering.GROUP:
        invperm = torch.argsort(perm)
        q_param_dict["weight_g_idx"] = g_idx[invperm]
    return loss.item(), q_param_dict


def quantize_weight(module: torch.nn.Module, quant_args: QuantizationArgs, hessian: torch.Tensor,
                    blocksize: int = 128, percdamp: float = 0.01, hessian_divisor: float = 1.0) -> tuple[float, dict]:
    """Quantize a module weight according to the GPTQ algorithm.

    :param module: module with weight being quantized (must carry ``weight_observer`` with statistics)
    :param quant_args: quantization arguments used to find quantization parameters
    :param hessian: preaccumulated hessian for quantization (consumed)
    :param blocksize: chunk size of quantization updates
    :param percdamp: dampening factor on hessian diagonal
    :return: loss, dict of weight / weight_scale / weight_zero_point [/ weight_global_scale / weight_g_idx]
    """
    return quantize_weight_tensors(module.weight.data, module.weight_observer, quant_args, hessian, blocksize,
                                   percdamp, hessian_divisor)


def group_key(module: torch.nn.Module, quant_args: QuantizationArgs, hessian: torch.Tensor):
    """Modules with equal keys share one lock-step column loop in ``quantize_weight_group``; None = not eligible."""
    w = module.weight
    if not isinstance(module, torch.nn.Linear) or w.ndim != 2 or not w.is_cuda or not hessian.is_cuda:
        return None
    actorder = quant_args.actorder
    if actorder == ActivationOrdering.GROUP:  # re-observes the permuted weight per module
        return None
    return (tuple(w.shape), w.dtype, w.device, w.stride(0), hessian.stride(0),
            quant_args.model_dump_json() if hasattr(quant_args, "model_dump_json") else repr(quant_args))


def width_key(module: torch.nn.Module, quant_args: QuantizationArgs, hessian: torch.Tensor):
    """Modules with equal keys can share one lock-step Cholesky chain (``quantize_weight_group``): same number
    of columns, device and Hessian layout, and all or none ordered by activation; None = not eligible."""
    if group_key(module, quant_args, hessian) is None:
        return None
    return (module.weight.shape[1], module.weight.device, hessian.stride(0), bool(quant_args.actorder))


def quantize_weight_group(modules, hessians, hessian_divisors, blocksize: int = 128, percdamp: float = 0.01):
    """``quantize_weight`` for several Linears of one width at once (the experts of an MoE layer, or the
    projections of a decoder layer that read the hidden state): one lock-step Cholesky chain for all of them,
    and one lock-step column loop per set of equal shape and scheme, instead of a chain of small kernels per
    module.  Same results as calling ``quantize_weight`` on each.  Returns a list of
    (loss tensor, q_param_dict, info tensor) in the order of ``modules``."""
    return finish_weight_group(begin_weight_group(modules, hessians, hessian_divisors, percdamp, blocksize),
                               blocksize)


def begin_weight_group(modules, hessians, hessian_divisors, percdamp: float = 0.01, blocksize: int = 128):
    """First half of ``quantize_weight_group``: column orders and the lock-step Cholesky chain, which need the
    Hessians only.  The weight observers' statistics are not read before ``finish_weight_group``, so a caller may
    enqueue the chains of several sets, observe the weights while they run, and finish afterwards."""
    n = len(modules)
    keys = [group_key(m, m.quantization_scheme.weights, H) for m, H in zip(modules, hessians)]
    # members of one column-loop set next to each other, so that their factors are one slice of the batch
    order = sorted(range(n), key=lambda i: (keys.index(keys[i]), i))
    mods = [modules[i] for i in order]
    Hs = [hessians[i] for i in order]
    divs = [hessian_divisors[i] for i in order]
    keys = [keys[i] for i in order]
    # Members that were given the very same Hessian tensor (Linears fed one input: q/k/v, gate/up) with the same
    # divisor and the same ordering rule have the same column order and the same factor: the chain runs once per
    # distinct Hessian and the members take copies of its results.
    ordered = [bool(m.quantization_scheme.weights.actorder) for m in mods]
    first_of, source = {}, []
    for i, (H, d, o) in enumerate(zip(Hs, divs, ordered)):
        source.append(first_of.setdefault((id(H), float(d), o), i))
    distinct = sorted(set(source))
    shared = len(distinct) < n
    uH, udiv, uord = [Hs[i] for i in distinct], [divs[i] for i in distinct], [ordered[i] for i in distinct]
    # the column orders of all members in one sort (row-wise stable, so each row is what the per-module call sorts)
    all_perms = None
    if all(uord):
        all_perms = _diag_order(uH)
        perms = all_perms
    else:
        single = [_diag_order([H])[0] if o else None for o, H in zip(uord, uH)]
        perms = torch.stack(single) if single[0] is not None else None
    form = ops.gptq_factor_form(uH[0].shape[0], blocksize)
    U, dead, info = llmc.gptq_prepare_hinv_grouped(uH, perms, [float(d) for d in udiv], float(percdamp), form)
    if shared:
        slot = {i: j for j, i in enumerate(distinct)}
        # through pinned memory, so that the host does not wait for the chain it has just enqueued
        take = torch.tensor([slot[i] for i in source]).pin_memory().to(U.device, non_blocking=True)
        U, dead, info = U[take], dead[take], info[take]
        if perms is not None:
            perms = perms[take]
            all_perms = perms if all_perms is not None else None
    return dict(n=n, order=order, mods=mods, keys=keys, perms=perms, all_perms=all_perms, U=U, dead=dead, info=info,
                form=form, blocksize=blocksize)


def finish_weight_group(ctx, blocksize: int = 128):
    """Second half of ``quantize_weight_group``: quantisation parameters from the weight observers, the lock-step
    column loops on the factors of ``begin_weight_group``, and the results in the caller's order."""
    n, order, mods, keys = ctx["n"], ctx["order"], ctx["mods"], ctx["keys"]
    perms, all_perms, U, dead, info = ctx["perms"], ctx["all_perms"], ctx["U"], ctx["dead"], ctx["info"]
    form = ctx["form"]
    if ops.gptq_factor_form(U.shape[-1], blocksize) != ops.gptq_factor_form(U.shape[-1], ctx["blocksize"]):
        raise ValueError(f"finish_weight_group: block size {blocksize} does not fit the factors, which were prepared "
                         f"for block size {ctx['blocksize']}")
    prep = []
    base_g_idx = {}
    for j, m in enumerate(mods):
        quant_args = m.quantization_scheme.weights
        strategy, actorder = quant_args.strategy, quant_args.actorder
        W = m.weight.data if m.weight.data.is_contiguous() else m.weight.data.contiguous()
        num_rows, num_columns = W.shape
        perm = perms[j] if (perms is not None and actorder) else None
        row_div, srow, divisor = _scale_layout(strategy, quant_args, num_rows, num_columns)
        g_idx = None
        if divisor is not None:
            if (num_columns, divisor) not in base_g_idx:
                base_g_idx[(num_columns, divisor)] = torch.arange(num_columns, device=W.device,
                                                                  dtype=torch.int) // divisor
            g_idx = base_g_idx[(num_columns, divisor)]
            if actorder == ActivationOrdering.WEIGHT:
                if all_perms is not None:  # one gather for every member with this group width
                    if ("permuted", divisor) not in base_g_idx:
                        base_g_idx[("permuted", divisor)] = g_idx[all_perms]
                    g_idx = base_g_idx[("permuted", divisor)][j]
                else:
                    g_idx = g_idx[perm]
        qp = m.weight_observer.get_qparams()
        prep.append(dict(args=quant_args, W=W, perm=perm, g_idx=g_idx, qp=qp, row_div=row_div, srow=srow,
                         zp=None if quant_args.symmetric else qp["zero_point"].to(torch.int8),
                         kscale=effective_scale(qp["scale"], quant_args, W.dtype)))

    outs, losses = [None] * n, [None] * n
    at = 0
    while at < n:
        end = at + 1
        while end < n and keys[end] == keys[at]:
            end += 1
        part = prep[at:end]
        first = part[0]
        fmt, bits = kernel_format(first["args"])
        if end - at == 1:
            outs[at], losses[at] = llmc.gptq_quantize(
                first["W"], U[at], first["kscale"], first["zp"], fmt, bits, first["row_div"], first["srow"],
                g_idx=first["g_idx"], perm=first["perm"], dead=dead[at], global_scale=first["qp"]["global_scale"],
                blocksize=blocksize, form=form)
        else:
            has_gs = first["qp"]["global_scale"] is not None
            o, l = llmc.gptq_quantize_grouped(
                [p["W"] for p in part], U[at:end], [p["kscale"] for p in part],
                None if first["zp"] is None else [p["zp"] for p in part], fmt, bits, first["row_div"], first["srow"],
                g_idxs=None if first["g_idx"] is None else [p["g_idx"] for p in part],
                perms=None if perms is None else perms[at:end], dead=dead[at:end],
                global_scales=[p["qp"]["global_scale"] for p in part] if has_gs else None, blocksize=blocksize,
                form=form)
            for b in range(end - at):
                outs[at + b], losses[at + b] = o[b], l[b]
        at = end

    results = [None] * n
    for j, (m, p) in enumerate(zip(mods, prep)):
        quant_args, qp = p["args"], p["qp"]
        final_dtype = p["W"].dtype
        scale, zero_point, global_scale = qp["scale"], qp["zero_point"], qp["global_scale"]
        q = {
            "weight": outs[j].reshape(m.weight.shape),
            "weight_scale": scale if scale.dtype in (torch.uint8, torch.float8_e4m3fn) else scale.to(dtype=final_dtype),
            "weight_zero_point": zero_point.to(dtype=quant_args.zp_dtype),
        }
        if quant_args.scale_dtype == torch.float8_e4m3fn and scale.dtype == torch.float32:
            q["weight_scale"] = scale
        if global_scale is not None:
            q["weight_global_scale"] = global_scale.to(dtype=final_dtype)
        results[order[j]] = (losses[j].reshape(()), q, info[j])
    return results
