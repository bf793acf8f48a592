"""GPU parity: Hessian accumulation through the C ABI vs the CPU oracle / fp64 closed form."""
import pytest
import torch

from oracle import gptq as G

pytestmark = pytest.mark.gpu

TOL = 1e-5  # relative Frobenius error stated by the north star for the Hessian


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


@pytest.mark.parametrize(
    "T,K",
    [(64, 128), (512, 256), (100, 96), (37, 200), (1, 8), (300, 520), (130, 1024), (64, 12)],
)
def test_hessian_matches_oracle(T, K):
    from llmcompressor_amd import ops

    torch.manual_seed(T * 1000 + K)
    x = torch.randn(T, K).bfloat16()
    x[:, K // 3] *= 20
    H0 = G.make_empty_hessian(K)
    Hc, _ = G.accumulate_hessian(x, H0.clone(), torch.zeros(()))
    Hc, _ = G.accumulate_hessian(x.flip(0) * 0.5, Hc, torch.zeros(()))
    Hg = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(Hg, x.cuda())
    ops.hessian_accumulate_(Hg, (x.flip(0) * 0.5).cuda())
    Hg = Hg.cpu()
    ref64 = 2 * x.double().t() @ x.double() * 1.25
    assert _rel(Hg, Hc) < TOL
    assert _rel(Hg, ref64) < TOL
    assert torch.equal(Hg, Hg.t())


def test_hessian_nonsymmetric_start_and_fp16():
    from llmcompressor_amd import ops

    torch.manual_seed(5)
    K, T = 384, 200
    x = torch.randn(T, K).half()
    H0 = torch.randn(K, K)
    Hg = H0.cuda()
    ops.hessian_accumulate_(Hg, x.cuda(), assume_symmetric=False)
    ref = H0.double() + 2 * x.double().t() @ x.double()
    assert _rel(Hg.cpu(), ref) < TOL


def test_hessian_config1_shape_additivity():
    """K=4096, 4 hook calls of [512,4096]: equals one call on the concatenation (sum over tokens)."""
    from llmcompressor_amd import ops

    torch.manual_seed(0)
    K = 4096
    xs = [torch.randn(512, K, device="cuda").bfloat16() for _ in range(4)]
    H1 = torch.zeros(K, K, device="cuda")
    for x in xs:
        ops.hessian_accumulate_(H1, x)
    H2 = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H2, torch.cat(xs))
    ref = 2 * torch.cat(xs).float().t() @ torch.cat(xs).float()
    assert _rel(H1, H2) < TOL and _rel(H1, ref) < TOL
    assert torch.equal(H1, H1.t())
    # K = 14336 takes the 256-wide tile path
    K = 14336
    x = torch.randn(256, K, device="cuda").bfloat16()
    H = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H, x)
    ref = 2 * x.float().t() @ x.float()
    assert _rel(H, ref) < TOL
    assert torch.equal(H, H.t())


@pytest.mark.parametrize("T,K", [(1024, 1024), (2048, 4096), (1100, 1288), (4096, 2304)])
def test_hessian_token_chunks(T, K):
    """Shapes whose tiles do not fill the chip: tiles are cut along the tokens, the partial tiles go
    through the workspace and are summed in fixed order.  Same tolerance, still bitwise symmetric and
    reproducible; without the workspace every tile is one workgroup."""
    from llmcompressor_amd import ops

    torch.manual_seed(T + K)
    x = torch.randn(T, K, device="cuda").bfloat16()
    x[:, 5] *= 30
    ref = 2 * (x.double().t() @ x.double())
    H = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H, x)
    assert _rel(H, ref) < TOL
    assert torch.equal(H, H.t())
    ops.hessian_accumulate_(H, x)  # a second launch on top of a mirrored result
    assert _rel(H, 2 * ref) < TOL
    assert torch.equal(H, H.t())
    Hd = [torch.zeros(K, K, device="cuda") for _ in range(2)]
    for h in Hd:
        ops.hessian_accumulate_(h, x)
        ops.hessian_accumulate_(h, x)
    assert torch.equal(Hd[0], Hd[1]) and torch.equal(Hd[0], H)
    Hn = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(Hn, x, use_workspace=False)
    assert _rel(Hn, ref) < TOL and torch.equal(Hn, Hn.t())
    Hu = torch.randn(K, K, device="cuda")  # not symmetric: both triangles are read-modify-written
    Hu0 = Hu.clone()
    ops.hessian_accumulate_(Hu, x, assume_symmetric=False)
    assert _rel(Hu - Hu0, ref) < 1e-4
    if T <= 2048 and K <= 1288:  # the CPU oracle at a size it finishes quickly
        Hc, _ = G.accumulate_hessian(x.cpu(), G.make_empty_hessian(K), torch.zeros(()))
        assert _rel(H.cpu(), 2 * Hc) < TOL


def test_hessian_full_size_token_chunks():
    """K = 14336 at 4096 tokens: 1536 whole tiles + 60 tiles in chunks; checked on sampled rows."""
    from llmcompressor_amd import ops

    torch.manual_seed(1)
    K, T = 14336, 4096
    x = torch.randn(T, K, device="cuda").bfloat16()
    H = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H, x)
    rows = torch.tensor([0, 255, 256, 4095, 7000, 13000, 14080, 14335], device="cuda")
    ref = 2 * (x[:, rows].double().t() @ x.double())
    assert _rel(H[rows], ref) < TOL
    assert torch.equal(H, H.t())


def test_hessian_grouped_moe_shapes():
    """Config-5 shapes: 128 experts with routed token counts (some zero), widths 2048 and 768, one launch
    per projection; each expert's Hessian equals the single-problem entry point's, bit for bit where that
    one also runs whole tiles, and an expert without tokens keeps its Hessian."""
    from llmcompressor_amd import ops

    g = torch.Generator().manual_seed(0)
    E = 128
    w = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.1
    idx = torch.multinomial(w / w.sum(), 4096 * 8, replacement=True, generator=g)
    n_e = torch.bincount(idx, minlength=E)
    n_e[5] = 0
    n_e[77] = 0
    for K in (2048, 768):
        x_all = torch.randn(int(n_e.sum()), K, generator=g).bfloat16().cuda()
        offs = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(n_e, 0)])
        xs = [x_all[int(offs[e]): int(offs[e + 1])] for e in range(E)]
        H = torch.zeros(E, K, K, device="cuda")
        H[5] = 3.0  # must stay as it is
        ops.hessian_accumulate_grouped_([H[e] for e in range(E)], xs)
        assert torch.equal(H[5], torch.full_like(H[5], 3.0)) and torch.count_nonzero(H[77]) == 0
        for e in (0, 1, 17, 64, 127):
            ref = 2 * (xs[e].double().t() @ xs[e].double())
            if n_e[e] > 0:
                assert _rel(H[e], ref) < TOL, (K, e)
            assert torch.equal(H[e], H[e].t())
            single = torch.zeros(K, K, device="cuda")
            if n_e[e] > 0:
                ops.hessian_accumulate_(single, xs[e], use_workspace=False)
            assert _rel(H[e], single) < 1e-6 if n_e[e] > 0 else torch.count_nonzero(H[e]) == 0
        # second launch accumulates on top
        ops.hessian_accumulate_grouped_([H[e] for e in range(E)], xs)
        ref = 4 * (xs[0].double().t() @ xs[0].double())
        assert _rel(H[0], ref) < TOL
    # the oracle on a small grouped case, f16 inputs, more problems than one launch holds
    K, E = 96, 150
    xs = [torch.randn(int(t), K, generator=g).half().cuda() for t in torch.randint(0, 40, (E,), generator=g)]
    Hs = [torch.zeros(K, K, device="cuda") for _ in range(E)]
    ops.hessian_accumulate_grouped_(Hs, xs)
    for e in (0, 3, 129, 149):
        Hc, _ = G.accumulate_hessian(xs[e].cpu(), G.make_empty_hessian(K), torch.zeros(()))
        if xs[e].shape[0]:
            assert _rel(Hs[e].cpu(), Hc) < TOL
        else:
            assert torch.count_nonzero(Hs[e]) == 0


@pytest.mark.parametrize("K,seg,nseg,last,dtype", [
    (1024, 64, 5, 64, torch.bfloat16),      # every slab in a buffer of its own
    (1288, 128, 7, 100, torch.bfloat16),    # ragged last buffer, K not a multiple of the tile
    (4096, 256, 9, 256, torch.float16),     # tiles cut along the tokens: chunk starts inside a buffer list
    (2304, 192, 64, 1, torch.bfloat16),     # the maximum number of buffers, a single row in the last
    (512, 2048, 1, 777, torch.bfloat16),    # one buffer only
])
def test_hessian_segments_match_concatenation(K, seg, nseg, last, dtype):
    """llmc_hessian_accumulate_segments on separately allocated buffers is bit-identical to
    llmc_hessian_accumulate on their concatenation (same plan, same summation order)."""
    from llmcompressor_amd import ops

    torch.manual_seed(K + seg)
    xs = []
    for i in range(nseg):
        rows = last if i == nseg - 1 else seg
        # separate allocations in shuffled address order, padded rows (row stride > K)
        buf = torch.randn(rows, K + 8, device="cuda").to(dtype)
        xs.append(buf[:, :K])
        _ = torch.empty(1000 * (i % 3 + 1), device="cuda")
    cat = torch.cat([x.contiguous() for x in xs], 0)
    ref = 2 * (cat.double().t() @ cat.double())
    H0 = torch.randn(K, K, device="cuda")
    H0 = H0 + H0.t()
    Ha, Hb = H0.clone(), H0.clone()
    ops.hessian_accumulate_(Ha, cat)
    ops.hessian_accumulate_segments_(Hb, xs)
    assert torch.equal(Ha, Hb)
    assert _rel(Hb - H0, ref) < 2e-5
    assert torch.equal(Hb, Hb.t())
    # more buffers than one launch takes: split by the wrapper
    if nseg == 64:
        Hc = H0.clone()
        ops.hessian_accumulate_segments_(Hc, xs[:-1] + [xs[0]] * 3 + [xs[-1]])
        cat2 = torch.cat([cat[:-last], xs[0], xs[0], xs[0], cat[-last:]], 0)
        assert _rel(Hc - H0, 2 * (cat2.double().t() @ cat2.double())) < 2e-5
    with pytest.raises(ValueError):
        ops.hessian_accumulate_segments_(Hb, [xs[0][:63], xs[0][:63]])  # rows per buffer not a multiple of 64


def test_hessian_segments_full_size():
    """K = 14336, 32 buffers of 2048 tokens (one staged launch of the bench): bit-identical to the
    concatenated launch."""
    from llmcompressor_amd import ops

    torch.manual_seed(3)
    K, seg, nseg = 14336, 2048, 32
    big = torch.randn(nseg + 1, seg, K, device="cuda").bfloat16()
    xs = [big[i] for i in range(nseg)]
    xs = [xs[(7 * i) % nseg] for i in range(nseg)]  # buffers out of address order
    cat = torch.cat(xs, 0)
    Ha = torch.zeros(K, K, device="cuda")
    Hb = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(Ha, cat)
    ops.hessian_accumulate_segments_(Hb, xs)
    assert torch.equal(Ha, Hb)
    rows = torch.tensor([0, 255, 256, 7000, 14335], device="cuda")
    ref = 2 * (cat[:, rows].double().t() @ cat.double())
    assert _rel(Hb[rows], ref) < TOL


@pytest.mark.parametrize("T,K", [(64, 128), (100, 96), (37, 201), (1, 8), (300, 520), (2048, 1024), (513, 67)])
def test_hessian_fp32_activations(T, K):
    """fp32 activations (the reference's ``inp.float()`` path with nothing to cast, gptq_quantize.py:57-62)
    take the fp32 matrix-core product: the oracle and the fp64 closed form within the Hessian tolerance, a
    non-symmetric start is read-modify-written everywhere, a symmetric one stays bitwise symmetric, and a
    row-strided view of the activations is accepted."""
    from llmcompressor_amd import ops

    torch.manual_seed(T * 7 + K)
    wide = torch.randn(T, K + 5)
    wide[:, K // 3] *= 20
    x = wide[:, :K]
    Hc, _ = G.accumulate_hessian(x.contiguous(), G.make_empty_hessian(K), torch.zeros(()))
    Hc, _ = G.accumulate_hessian(x.flip(0).contiguous() * 0.5, Hc, torch.zeros(()))
    Hg = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(Hg, wide.cuda()[:, :K])
    ops.hessian_accumulate_(Hg, (x.flip(0) * 0.5).cuda())
    ref64 = 2 * x.double().t() @ x.double() * 1.25
    assert _rel(Hg.cpu(), Hc) < TOL
    assert _rel(Hg.cpu(), ref64) < TOL
    assert torch.equal(Hg, Hg.t())
    H0 = torch.randn(K, K)
    Hn = H0.cuda()
    ops.hessian_accumulate_(Hn, x.cuda().contiguous(), assume_symmetric=False)
    assert _rel(Hn.cpu(), H0.double() + 2 * x.double().t() @ x.double()) < TOL
