"""Oracle: GPTQ Hessian accumulation and ``quantize_weight``.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Follows ``src/llmcompressor/modifiers/gptq/gptq_quantize.py`` op for op:
``make_empty_hessian`` (:19-25), ``accumulate_hessian`` (:28-64, Linear branch),
``quantize_weight`` (:67-264) and ``_apply_activation_ordering`` (:267-278).
"""
from __future__ import annotations

import math

import torch

from .observers import Observer
from .qformat import QArgs, fake_quantize

GPTQ_PRECISION = torch.float32


def make_empty_hessian(num_columns: int):
    return torch.zeros((num_columns, num_columns), dtype=GPTQ_PRECISION)


def accumulate_hessian(inp, H, num_samples):
    """H += (sqrt2 X)^T (sqrt2 X); num_samples += batch dim (gptq_quantize.py:28-64)."""
    if inp.ndim == 2:
        inp = inp.unsqueeze(0)
    elif inp.ndim > 3:
        inp = inp.reshape(inp.shape[0], -1, inp.shape[-1])
    num_added = inp.shape[0]
    inp = inp.reshape((-1, inp.shape[-1])).t()
    num_samples += num_added
    inp = inp.to(dtype=GPTQ_PRECISION)
    inp = math.sqrt(2) * inp
    H += inp.matmul(inp.t())
    return H, num_samples


def apply_activation_ordering(W, H):
    perm = torch.argsort(torch.diag(H), descending=True)
    return W[:, perm], H[perm][:, perm], perm


def hessian_inverse_factor(H, percdamp):
    """dead-column mask is the caller's; returns (Hinv upper factor, ok)."""
    try:
        damp = percdamp * torch.mean(torch.diag(H))
        diag = torch.arange(H.shape[0])
        H[diag, diag] += damp
        H = torch.linalg.cholesky(H)
        H = torch.cholesky_inverse(H)
        H = torch.linalg.cholesky(H, upper=True)
        return H, True
    except torch._C._LinAlgError:
        return torch.eye(H.shape[0], dtype=H.dtype), False


def quantize_weight(weight, observer: Observer, quant_args: QArgs, hessian, blocksize=128, percdamp=0.01,
                    fused_update=False):
    """gptq_quantize.py:67-264.  ``weight`` [R,K] in its own dtype; ``hessian`` is consumed.

    Returns ``(loss, q_param_dict, info)`` where ``info['ok']`` is False when the
    identity (round-to-nearest) fallback was taken.

    ``fused_update=True`` is NOT the reference: it forms the in-block update ``w - err * U[i, j]`` with one
    rounding (an fma, which is what the device's block kernel issues) instead of rounding the outer product
    first (gptq_quantize.py:232-233).  It exists so that a test can bound the effect of that one-rounding
    difference on the codes.
    """
    strategy = quant_args.strategy
    actorder = quant_args.actorder
    final_shape = weight.shape
    final_dtype = weight.dtype
    W = weight.clone().to(dtype=GPTQ_PRECISION)
    H = hessian
    num_rows, num_columns = W.shape

    if actorder == "group" and strategy not in ("group", "tensor_group"):
        actorder = None
    if actorder:
        W, H, perm = apply_activation_ordering(W, H)
    if actorder == "group":
        observer.delete_statistics(check_fused=False)
        observer(W)
    g_idx = None
    if strategy in ("group", "tensor_group", "block"):
        divisor = quant_args.group_size if strategy != "block" else quant_args.block_structure[1]
        g_idx = torch.arange(num_columns, dtype=torch.int) // divisor
        if actorder == "weight":
            g_idx = g_idx[perm]

    qp = observer.get_qparams()
    scale, zero_point, global_scale = qp["scale"], qp["zero_point"], qp["global_scale"]

    losses = torch.zeros(num_rows)
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0

    Hinv, ok = hessian_inverse_factor(H, percdamp)

    chan_args = quant_args.copy(strategy="channel")
    for i1 in range(0, num_columns, blocksize):
        i2 = min(i1 + blocksize, num_columns)
        count = i2 - i1
        W1 = W[:, i1:i2].clone()
        Q1 = torch.zeros_like(W1)
        Err1 = torch.zeros_like(W1)
        losses1 = torch.zeros_like(W1)
        Hinv1 = Hinv[i1:i2, i1:i2]
        for i in range(count):
            w = W1[:, i]
            d = Hinv1[i, i]
            q = w.clone()
            if strategy == "tensor":
                q = fake_quantize(q, scale, zero_point, quant_args, global_scale=global_scale)
            elif strategy == "channel":
                q = fake_quantize(q, scale[:, 0], zero_point[:, 0], quant_args, global_scale=global_scale)
            elif strategy in ("group", "tensor_group"):
                gi = g_idx[i1 + i]
                q = fake_quantize(q, scale[:, gi], zero_point[:, gi], chan_args, global_scale=global_scale)
            elif strategy == "block":
                # the reference hands a [R,1] slice with scale [R/bh, 1] to the
                # BLOCK fake-quant; arithmetic per element is the CHANNEL one with
                # each row using its block-row's scale
                bc = int(g_idx[i1 + i])
                bh = quant_args.block_structure[0]
                srow = scale[:, bc].repeat_interleave(bh)[:num_rows]
                zrow = zero_point[:, bc].repeat_interleave(bh)[:num_rows]
                q = fake_quantize(q, srow, zrow, chan_args, global_scale=global_scale)
            else:
                raise ValueError(f"Quantization strategy is not supported for GPTQ: {strategy}")
            Q1[:, i] = q
            losses1[:, i] = (w - q) ** 2 / d**2
            err1 = (w - q) / d
            if fused_update:
                # exact product of two fp32 values in fp64, one rounding of the difference back to fp32
                W1[:, i:] = (W1[:, i:].double() - err1.double().unsqueeze(1) * Hinv1[i, i:].double().unsqueeze(0)).float()
            else:
                W1[:, i:] -= err1.unsqueeze(1).matmul(Hinv1[i, i:].unsqueeze(0))
            Err1[:, i] = err1
        W[:, i1:i2] = Q1
        losses += torch.sum(losses1, 1) / 2
        W[:, i2:] -= Err1.matmul(Hinv[i1:i2, i2:])

    if actorder:
        invperm = torch.argsort(perm)
        W = W[:, invperm]
    W = W.reshape(final_shape).to(final_dtype)
    loss = torch.sum(losses).item()
    out = {
        "weight": W,
        "weight_scale": scale.to(dtype=final_dtype),
        "weight_zero_point": zero_point.to(dtype=quant_args.zp_dtype),
    }
    if global_scale is not None:
        out["weight_global_scale"] = global_scale.to(dtype=final_dtype)
    if actorder == "group":
        out["weight_g_idx"] = g_idx[invperm]
    return loss, out, {"ok": ok, "Hinv": Hinv}


def textbook_gptq_fp64(W, H, quantize_col, percdamp=0.01):
    """Un-blocked GPTQ (Frantar et al. 2022, Alg. 1 without lazy batching) in fp64.

    Independent of the blocked restatement above: explicit inverse, explicit
    upper Cholesky factor, one column at a time.  ``quantize_col(j, w)`` returns
    the quantised column.  Used only to pin ``quantize_weight`` on tiny inputs.
    """
    W = W.double().clone()
    H = H.double().clone()
    K = W.shape[1]
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    H += torch.eye(K, dtype=torch.float64) * percdamp * torch.mean(torch.diag(H))
    Hinv = torch.linalg.inv(H)
    U = torch.linalg.cholesky(Hinv, upper=True)
    Q = torch.zeros_like(W)
    for j in range(K):
        q = quantize_col(j, W[:, j])
        Q[:, j] = q
        e = (W[:, j] - q) / U[j, j]
        W[:, j:] -= e.unsqueeze(1) * U[j, j:].unsqueeze(0)
    return Q
