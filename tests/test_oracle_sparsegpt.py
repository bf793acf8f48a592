"""The SparseGPT oracle pinned by mathematics (no reference-held vector exists for it)."""
import math

import pytest
import torch

from oracle import sparsegpt as S


def _hessian(K, T, seed, scale_cols=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, K, generator=g)
    if scale_cols:
        x = x * (0.25 + 2 * torch.rand(K, generator=g))
    return x, 2 * (x.t() @ x) / 1.0


def test_running_average_hessian_closed_form():
    g = torch.Generator().manual_seed(0)
    K = 24
    H, n = S.make_empty_hessian(K), 0
    xs = [torch.randn(b, 7, K, generator=g) for b in (1, 3, 2)] + [torch.randn(5, K, generator=g)]
    for x in xs:
        H, n = S.accumulate_hessian(x, H, n)
    assert n == 1 + 3 + 2 + 1  # a 2-D input counts as one sample
    flat = torch.cat([x.reshape(-1, K) for x in xs]).double()
    ref = 2.0 / n * (flat.t() @ flat)
    assert ((H.double() - ref).norm() / ref.norm()).item() < 1e-6


def test_diagonal_hessian_is_saliency_pruning_without_compensation():
    g = torch.Generator().manual_seed(1)
    R, K = 16, 64
    W = torch.randn(R, K, generator=g)
    h = 0.5 + torch.rand(K, generator=g)
    H = torch.diag(h)
    loss, Q = S.sparsify_weight(W, H.clone(), sparsity=0.5, block_size=32, dampening_frac=0.01)
    damp = 0.01 * h.mean()
    for c0 in (0, 32):
        blk = slice(c0, c0 + 32)
        score = (W[:, blk].double() ** 2) * (h[blk].double() + damp.double())  # w^2 / d^2, d = (h+damp)^-1/2
        k = int(R * 32 * 0.5)
        cut = torch.sort(score.flatten())[0][k]
        expect = torch.where(score <= cut, torch.zeros_like(W[:, blk]), W[:, blk])
        assert torch.equal(Q[:, blk], expect)  # survivors untouched: a diagonal U propagates nothing
    expect_loss = 0.5 * (((W - Q).double() ** 2) * (h + damp).double()).sum().item()
    assert abs(loss - expect_loss) / expect_loss < 1e-5


@pytest.mark.parametrize("sparsity,bs", [(0.5, 32), (0.7, 64), (0.25, 128)])
def test_unstructured_zero_count_per_block(sparsity, bs):
    R, K = 24, 128
    x, H = _hessian(K, 300, 2)
    W = torch.randn(R, K, generator=torch.Generator().manual_seed(3))
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=sparsity, block_size=bs)
    for c0 in range(0, K, bs):
        assert int((Q[:, c0:c0 + bs] == 0).sum()) == int(R * bs * sparsity) + 1  # "<= k-th smallest", no ties


@pytest.mark.parametrize("n,m", [(2, 4), (1, 2), (4, 8), (3, 4)])
def test_n_m_structure(n, m):
    R, K = 12, 64
    x, H = _hessian(K, 200, 4)
    W = torch.randn(R, K, generator=torch.Generator().manual_seed(5))
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=n / m, prune_n=n, prune_m=m, block_size=32)
    zeros = (Q == 0).reshape(R, K // m, m).sum(-1)
    assert torch.all(zeros == n)


def test_matches_unblocked_fp64_textbook_with_the_same_mask():
    R, K = 8, 48
    x, H = _hessian(K, 400, 6)
    W = torch.randn(R, K, generator=torch.Generator().manual_seed(7))
    for kw in (dict(sparsity=0.5, block_size=16), dict(sparsity=0.5, prune_n=2, prune_m=4, block_size=16),
               dict(sparsity=0.6, block_size=48)):
        _, Q = S.sparsify_weight(W, H.clone(), **kw)
        Qt = S.textbook_sparsegpt_fp64(W, H, Q == 0)
        assert ((Q.double() - Qt).norm() / Qt.norm()).item() < 1e-4
        assert torch.equal(Qt == 0, Q == 0)


def test_single_elimination_is_the_constrained_least_squares_optimum():
    """Pruning one weight at column j and compensating on the columns after it minimises
    delta^T H delta subject to delta_j = -w_j, delta_{<j} = 0 (the OBS step SparseGPT is built on)."""
    K = 12
    x, H = _hessian(K, 100, 8)
    W = torch.randn(1, K, generator=torch.Generator().manual_seed(9))
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=0.0, block_size=K, dampening_frac=0.01)
    j = int((Q[0] == 0).nonzero()[0])
    assert int((Q == 0).sum()) == 1
    assert torch.equal(Q[0, :j], W[0, :j])
    Hd = H.double() + torch.eye(K, dtype=torch.float64) * 0.01 * torch.diag(H).double().mean()
    rest = list(range(j + 1, K))
    dj = -W[0, j].double()
    d_rest = -torch.linalg.solve(Hd[rest][:, rest], Hd[rest, j] * dj)
    expect = W[0, rest].double() + d_rest
    assert ((Q[0, rest].double() - expect).norm() / expect.norm()).item() < 1e-4


def test_preserved_zeros_stay_and_count_towards_the_target():
    R, K = 16, 64
    x, H = _hessian(K, 300, 10)
    g = torch.Generator().manual_seed(11)
    W = torch.randn(R, K, generator=g)
    W[torch.rand(R, K, generator=g) < 0.3] = 0
    was_zero = W == 0
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=0.5, block_size=32, preserve_sparsity_mask=True)
    assert torch.all(Q[was_zero] == 0)
    for c0 in (0, 32):
        assert int((Q[:, c0:c0 + 32] == 0).sum()) == int(R * 32 * 0.5) + 1
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=0.5, prune_n=2, prune_m=4, block_size=32,
                             preserve_sparsity_mask=True)
    assert torch.all(Q[was_zero] == 0)
    assert torch.all((Q == 0).reshape(R, K // 4, 4).sum(-1) >= 2)
    with pytest.raises(ValueError):
        S.sparsify_weight(W, H.clone(), sparsity=0.1, preserve_sparsity_mask=True)


def test_dead_columns_and_identity_fallback():
    R, K = 4, 16
    x, H = _hessian(K, 50, 12)
    H[3, :] = 0
    H[:, 3] = 0
    W = torch.randn(R, K, generator=torch.Generator().manual_seed(13))
    _, Q = S.sparsify_weight(W, H.clone(), sparsity=0.5, block_size=16)
    assert torch.all(Q[:, 3] == 0)
    bad = -torch.eye(K)  # not positive definite: the factor falls back to the identity
    _, Q = S.sparsify_weight(W, bad, sparsity=0.5, block_size=16)
    score = W ** 2
    cut = torch.sort(score.flatten())[0][int(R * K * 0.5)]
    assert torch.equal(Q, torch.where(score <= cut, torch.zeros_like(W), W))
