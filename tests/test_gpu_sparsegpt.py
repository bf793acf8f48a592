"""SparseGPT column loop on the GPU against the CPU oracle (same seeded inputs) and through properties
at Llama-3-8B widths.  Tolerances: pruning mask >= 99.9 % identical, surviving weights within 1e-3 relative
(Frobenius) of the oracle's, loss within 1 %; zero counts and N:M structure exact."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import sparsegpt as S  # noqa: E402

DEV = "cuda"


def _problem(R, K, T, seed, wdtype=torch.bfloat16, zero_frac=0.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, K, generator=g) * (0.25 + 2 * torch.rand(K, generator=g))).bfloat16()
    W = (torch.randn(R, K, generator=g) * 0.05).to(wdtype)
    if zero_frac:
        W[torch.rand(R, K, generator=g) < zero_frac] = 0
    return x, W


def _gpu(x, W, n_samples, **kw):
    from llmcompressor_amd import ops

    K = W.shape[1]
    H = torch.zeros(K, K, device=DEV)
    ops.hessian_accumulate_(H, x.to(DEV))
    form = kw.pop("form", ops.FACTOR_INVERSE)
    U, dead, info = ops.gptq_hinv_(H, None, divisor=float(n_samples), percdamp=kw.pop("dampening_frac", 0.01),
                                   form=form)
    assert int(info.item()) == 0
    Q, loss = ops.sparsegpt_sparsify(W.to(DEV), U, dead=dead, form=form, **kw)
    return Q.cpu(), float(loss.item())


def _oracle(x, W, n_samples, **kw):
    K = W.shape[1]
    H, n = S.make_empty_hessian(K), 0
    for chunk in x.reshape(n_samples, -1, K):
        H, n = S.accumulate_hessian(chunk.unsqueeze(0), H, n)
    return S.sparsify_weight(W, H, kw.pop("sparsity"), kw.pop("prune_n", 0), kw.pop("prune_m", 0),
                             kw.pop("blocksize", 128), kw.pop("dampening_frac", 0.01),
                             kw.pop("preserve_sparsity_mask", False))


CASES = [
    dict(R=64, K=256, kw=dict(sparsity=0.5)),
    dict(R=48, K=256, kw=dict(sparsity=0.7, blocksize=64)),
    dict(R=40, K=200, kw=dict(sparsity=0.3, blocksize=32)),           # ragged last block
    dict(R=64, K=256, kw=dict(sparsity=0.5, prune_n=2, prune_m=4)),
    dict(R=32, K=256, kw=dict(sparsity=0.5, prune_n=4, prune_m=8, blocksize=64)),
    dict(R=32, K=128, kw=dict(sparsity=0.5, prune_n=1, prune_m=2)),
    dict(R=64, K=256, zero_frac=0.3, kw=dict(sparsity=0.5, preserve_sparsity_mask=True)),
    dict(R=64, K=256, zero_frac=0.6, kw=dict(sparsity=0.5, blocksize=64, preserve_sparsity_mask=True)),  # blocks already sparse enough
    dict(R=64, K=256, zero_frac=0.2, kw=dict(sparsity=0.5, prune_n=2, prune_m=4, preserve_sparsity_mask=True)),
    dict(R=32, K=256, wdtype=torch.float32, kw=dict(sparsity=0.5)),
    dict(R=32, K=256, wdtype=torch.float16, kw=dict(sparsity=0.9, dampening_frac=0.1)),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_sparsify_matches_oracle(case):
    R, K = case["R"], case["K"]
    x, W = _problem(R, K, 1024, 100 + R + K, case.get("wdtype", torch.bfloat16), case.get("zero_frac", 0.0))
    if case["kw"].get("preserve_sparsity_mask") and case.get("zero_frac", 0) > case["kw"]["sparsity"]:
        # the existing pattern may be denser than the target only block-wise, never overall: thin it out
        W[:, : K // 2] = torch.where(W[:, : K // 2] == 0, torch.full_like(W[:, : K // 2], 0.01), W[:, : K // 2])
    Qg, lg = _gpu(x, W, 8, **dict(case["kw"]))
    lo, Qo = _oracle(x, W, 8, **dict(case["kw"]))
    same_mask = ((Qg == 0) == (Qo == 0)).float().mean().item()
    assert same_mask >= 0.999, same_mask
    both = (Qg != 0) & (Qo != 0)
    rel = ((Qg.double() - Qo.double())[both].norm() / Qo.double()[both].norm()).item()
    assert rel < 1e-3 + (5e-3 if W.dtype != torch.float32 else 0), rel  # 16-bit outputs differ by an ulp here and there
    assert abs(lg - lo) <= 0.01 * abs(lo) + 1e-9
    kw = case["kw"]
    if kw.get("prune_n"):
        n, m = kw["prune_n"], kw["prune_m"]
        zeros = (Qg == 0).reshape(R, K // m, m).sum(-1)
        assert torch.all(zeros >= n) and (kw.get("preserve_sparsity_mask") or torch.all(zeros == n))
    elif not kw.get("preserve_sparsity_mask"):
        bs = kw.get("blocksize", 128)
        for c0 in range(0, K, bs):
            cnt = min(bs, K - c0)
            assert int((Qg[:, c0:c0 + cnt] == 0).sum()) == int(R * cnt * kw["sparsity"]) + 1
    if kw.get("preserve_sparsity_mask"):
        assert torch.all(Qg[W == 0] == 0)


GROUPED_FACTOR_CASES = [
    dict(R=64, K=1024, kw=dict(sparsity=0.5)),
    dict(R=96, K=1536, kw=dict(sparsity=0.5, prune_n=2, prune_m=4)),
    dict(R=64, K=1024, zero_frac=0.3, kw=dict(sparsity=0.6, preserve_sparsity_mask=True)),
    dict(R=48, K=1408, zero_frac=0.2, kw=dict(sparsity=0.5, preserve_sparsity_mask=True)),  # a first group of 384 columns
]


@pytest.mark.parametrize("case", GROUPED_FACTOR_CASES, ids=[str(i) for i in range(len(GROUPED_FACTOR_CASES))])
def test_sparsify_from_the_grouped_factor_matches_oracle(case):
    """The loop in its left-looking form (the Cholesky factor of H outside the 512-column diagonal blocks, what
    wide weights use) against the oracle's U-based loop, and against the other form on the device."""
    from llmcompressor_amd import ops

    R, K = case["R"], case["K"]
    x, W = _problem(R, K, 2 * K, 300 + R + K, torch.bfloat16, case.get("zero_frac", 0.0))
    Qg, lg = _gpu(x, W, 8, form=ops.FACTOR_GROUPS, **dict(case["kw"]))
    Qi, li = _gpu(x, W, 8, **dict(case["kw"]))
    lo, Qo = _oracle(x, W, 8, **dict(case["kw"]))
    for other, lother in ((Qo, lo), (Qi, li)):
        assert ((Qg == 0) == (other == 0)).float().mean().item() >= 0.999
        both = (Qg != 0) & (other != 0)
        rel = ((Qg.double() - other.double())[both].norm() / other.double()[both].norm()).item()
        assert rel < 6e-3, rel
        assert abs(lg - lother) <= 0.01 * abs(lother) + 1e-9
    if case["kw"].get("preserve_sparsity_mask"):
        assert torch.all(Qg[W == 0] == 0)
    if case["kw"].get("prune_n"):
        assert torch.all((Qg == 0).reshape(R, K // 4, 4).sum(-1) == 2)


def test_sparsify_rejects_unsupported_structures():
    from llmcompressor_amd import ops

    W = torch.randn(8, 128, device=DEV).bfloat16()
    U = torch.eye(128, device=DEV)
    with pytest.raises(ValueError):
        ops.sparsegpt_sparsify(W, U, 0.5, prune_n=2, prune_m=3)
    with pytest.raises(ValueError):
        ops.sparsegpt_sparsify(W, U, 1.0)
    with pytest.raises(ValueError):
        ops.sparsegpt_sparsify(W, U, 0.5, blocksize=256)


@pytest.mark.parametrize("kw", [dict(sparsity=0.5), dict(sparsity=0.5, prune_n=2, prune_m=4)])
def test_sparsify_full_size_properties(kw):
    """4096 x 4096 at 8192 tokens: exact zero counts / structure, and the compensated result reconstructs the
    layer output better than the same mask without compensation."""
    from llmcompressor_amd import ops

    torch.manual_seed(0)
    R = K = 4096
    # correlated features (a 64-dimensional common part), so that there is something to compensate
    x = (torch.randn(8192, K, device=DEV) * 0.3 + torch.randn(8192, 64, device=DEV) @ torch.randn(64, K, device=DEV) * 0.2
         ).bfloat16()
    W = (torch.randn(R, K, device=DEV) * 0.02).bfloat16()
    H = torch.zeros(K, K, device=DEV)
    ops.hessian_accumulate_(H, x)
    U, dead, info = ops.gptq_hinv_(H, None, divisor=4.0)
    assert int(info.item()) == 0
    Q, loss = ops.sparsegpt_sparsify(W, U, dead=dead, **kw)
    torch.cuda.synchronize()
    if kw.get("prune_n"):
        assert torch.all((Q == 0).reshape(R, K // 4, 4).sum(-1) == 2)
    else:
        per_block = (Q == 0).reshape(R, K // 128, 128).sum((0, 2))
        k = int(R * 128 * 0.5)  # everything tied with the k-th smallest goes too (bf16 weights tie in block 0)
        assert torch.all(per_block >= k + 1) and torch.all(per_block <= k + 64), per_block[:4]
    xs = x[:2048].float()
    masked_only = torch.where(Q == 0, torch.zeros_like(W), W)
    err_sgpt = (xs @ (W.float() - Q.float()).t()).norm().item()
    err_mask = (xs @ (W.float() - masked_only.float()).t()).norm().item()
    assert err_sgpt < 0.8 * err_mask, (err_sgpt, err_mask)
    assert loss.item() > 0
