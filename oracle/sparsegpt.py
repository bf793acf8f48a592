"""Oracle: SparseGPT Hessian accumulation and ``sparsify_weight``.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Restates ``src/llmcompressor/modifiers/pruning/sparsegpt/sgpt_sparsify.py``:
``accumulate_hessian`` (:19-56, Linear branch: the *running average*
``H <- H*n/(n+b) + (2/(n+b)) X^T X``) and ``sparsify_weight`` (:59-213): dead
columns, damped ``cholesky -> cholesky_inverse -> cholesky(upper)``, then per
block of columns either the unstructured mask (saliency ``w^2/d^2`` not above
the ``int(numel*sparsity)``-th smallest of the block, :141-156) or the N:M mask
chosen group by group inside the column loop (:165-176), the OBS update of the
rest of the block (:181-188) and the lazy update of the columns beyond it
(:193-198), with an existing sparsity pattern optionally preserved.

Parity status: no reference-held vector exists for this function (the
reference's SparseGPT tests need hub models).  Pinned by mathematics in
``tests/test_oracle_sparsegpt.py``: diagonal Hessian == magnitude/saliency
pruning with no compensation, exact zero counts (unstructured: ``k+1`` per
block without ties; N:M: N per group), an un-blocked fp64 textbook SparseGPT,
the OBS optimality of a single pruned weight against a least-squares solve,
and the running-average Hessian against its closed form.
"""
from __future__ import annotations

import math

import torch

from .gptq import hessian_inverse_factor

SGPT_PRECISION = torch.float32


def make_empty_hessian(num_columns: int):
    return torch.zeros((num_columns, num_columns), dtype=SGPT_PRECISION)


def accumulate_hessian(inp, H, num_samples: int):
    """Running average: after all calls ``H = (2/N) sum X^T X`` (sgpt_sparsify.py:19-56)."""
    if inp.ndim == 2:
        inp = inp.unsqueeze(0)
    added = inp.shape[0]
    x = inp.reshape(-1, inp.shape[-1]).t()  # [K, tokens]
    H *= num_samples / (num_samples + added)
    num_samples += added
    x = math.sqrt(2 / num_samples) * x.to(SGPT_PRECISION)
    H += x.matmul(x.t())
    return H, num_samples


def _saliency(w, d):
    return w ** 2 / d.reshape(1, -1) ** 2


def sparsify_weight(weight, hessian, sparsity, prune_n=0, prune_m=0, block_size=128, dampening_frac=0.01,
                    preserve_sparsity_mask=False):
    """sgpt_sparsify.py:59-213 for a Linear weight [R, K]; ``hessian`` is consumed.  Returns (loss, W)."""
    out_dtype = weight.dtype
    W = weight.clone().to(SGPT_PRECISION)
    H = hessian
    rows, cols = W.shape

    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    U, _ok = hessian_inverse_factor(H, dampening_frac)

    keep_zero = None
    if preserve_sparsity_mask:
        keep_zero = W == 0
        if keep_zero.sum() / W.numel() > sparsity:
            raise ValueError("The target sparsity is lower than the sparsity of the base model. Please retry "
                             "after turning preserve_sparsity_mask=False")

    losses = torch.zeros(rows)
    for c0 in range(0, cols, block_size):
        c1 = min(c0 + block_size, cols)
        n = c1 - c0
        Wb = W[:, c0:c1].clone()
        Qb = torch.zeros_like(Wb)
        Eb = torch.zeros_like(Wb)
        Lb = torch.zeros_like(Wb)
        Ub = U[c0:c1, c0:c1]
        dg = torch.diag(Ub)

        if prune_n == 0:
            k = int(Wb.numel() * sparsity)
            if keep_zero is not None:
                pruned = keep_zero[:, c0:c1]
                if k > pruned.sum():  # the target asks for more zeros than the pattern holds: extend it
                    score = (~keep_zero[:, c0:c1]) * Wb ** 2 / dg.reshape(1, -1) ** 2
                    pruned = score <= torch.sort(score.flatten())[0][k]
            else:
                score = _saliency(Wb, dg)
                pruned = score <= torch.sort(score.flatten())[0][k]
        else:
            pruned = keep_zero[:, c0:c1].clone() if keep_zero is not None else torch.zeros_like(Wb, dtype=torch.bool)

        for j in range(n):
            w = Wb[:, j]
            d = Ub[j, j]
            if prune_n != 0 and j % prune_m == 0:
                score = _saliency(Wb[:, j:j + prune_m], dg[j:j + prune_m])
                if keep_zero is not None:
                    score = score * (~keep_zero[:, c0 + j:c0 + j + prune_m])
                pick = torch.topk(score, prune_n, dim=1, largest=False)[1]
                pruned.scatter_(1, j + pick, True)
            q = w.clone()
            q[pruned[:, j]] = 0
            Qb[:, j] = q
            Lb[:, j] = (w - q) ** 2 / d ** 2
            e = (w - q) / d
            Wb[:, j:] -= e.unsqueeze(1).matmul(Ub[j, j:].unsqueeze(0))
            Eb[:, j] = e

        W[:, c0:c1] = Qb
        losses += torch.sum(Lb, 1) / 2
        far = Eb.matmul(U[c0:c1, c1:])
        if keep_zero is not None:
            far = (~keep_zero[:, c1:]) * far
        W[:, c1:] -= far

    return torch.sum(losses).item(), W.to(out_dtype)


def textbook_sparsegpt_fp64(W, H, masks, dampening_frac=0.01):
    """Un-blocked OBS elimination in fp64 with a given pruning mask [R, K] (Frantar & Alistarh 2023, Alg. 1
    without lazy batching, mask supplied): explicit inverse, explicit upper Cholesky factor, one column at a
    time.  Independent of the blocked restatement above; pins its indexing on tiny inputs."""
    W = W.double().clone()
    H = H.double().clone()
    K = W.shape[1]
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    H += torch.eye(K, dtype=torch.float64) * dampening_frac * torch.mean(torch.diag(H))
    U = torch.linalg.cholesky(torch.linalg.inv(H), upper=True)
    Q = torch.zeros_like(W)
    for j in range(K):
        q = torch.where(masks[:, j], torch.zeros_like(W[:, j]), W[:, j])
        Q[:, j] = q
        e = (W[:, j] - q) / U[j, j]
        W[:, j:] -= e.unsqueeze(1) * U[j, j:].unsqueeze(0)
    return Q
