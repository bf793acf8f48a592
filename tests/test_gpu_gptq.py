"""GPU parity: damped Cholesky chain and the GPTQ column loop through the C ABI vs the CPU oracle.

Tolerances (north star): GPTQ codes agree on >= 99.9 % of the weights and the layer
reconstruction error ||(W - Q) X|| is within 1 % of the oracle's.
"""
import pytest
import torch

from oracle import gptq as G
from oracle import observers as O
from oracle import qformat as F

pytestmark = pytest.mark.gpu

CODE_AGREEMENT = 0.999
RECON_TOL = 0.01


def _hessian(K, T, seed, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, K, generator=g)
    if outliers:
        idx = torch.randperm(K, generator=g)[: max(1, K // 100)]
        x[:, idx] *= 20
    x = x.bfloat16().float()
    return 2 * x.t() @ x, x


@pytest.mark.parametrize("K", [24, 64, 96, 200, 512, 1000, 1536])
@pytest.mark.parametrize("use_perm", [False, True])
def test_hinv_matches_fp64_and_oracle(K, use_perm):
    from llmcompressor_amd import ops

    H, _ = _hessian(K, 4 * K, K)
    n = 7.0
    perm = torch.argsort(torch.diag(H), descending=True) if use_perm else None
    Hd = (H / n).double()
    if use_perm:
        Hd = Hd[perm][:, perm]
    Hd = Hd + 0.01 * Hd.diag().mean() * torch.eye(K, dtype=torch.float64)
    U64 = torch.linalg.cholesky(torch.linalg.inv(Hd), upper=True)
    Ho = H / n
    if use_perm:
        Ho = Ho[perm][:, perm]
    Uo, ok = G.hessian_inverse_factor(Ho.clone(), 0.01)
    assert ok
    Ug, dead, info = ops.gptq_hinv_(H.clone().cuda(), perm.cuda() if use_perm else None, divisor=n, percdamp=0.01)
    Ug = Ug.cpu()
    assert info.item() == 0 and dead.sum().item() == 0
    assert torch.equal(Ug, torch.triu(Ug))
    err_g = ((Ug.double() - U64).norm() / U64.norm()).item()
    err_o = ((Uo.double() - U64).norm() / U64.norm()).item()
    # at least as close to the exact factor as the reference's three-step fp32 route (x4 slack)
    assert err_g <= max(4 * err_o, 1e-5), (err_g, err_o)
    ident = Ug.double().t() @ Ug.double() @ Hd
    assert (ident - torch.eye(K, dtype=torch.float64)).abs().max() < 5e-3


def test_hinv_failure_and_dead_columns():
    from llmcompressor_amd import ops

    K = 130
    U, dead, info = ops.gptq_hinv_((-torch.eye(K)).cuda())
    assert info.item() != 0
    assert torch.equal(U.cpu(), torch.eye(K))
    H, _ = _hessian(K, 4 * K, 3)
    H[5, :] = 0
    H[:, 5] = 0
    H[77, :] = 0
    H[:, 77] = 0
    Uo, ok = G.hessian_inverse_factor(_fix_dead(H.clone()), 0.01)
    Ug, dead, info = ops.gptq_hinv_(H.clone().cuda())
    assert info.item() == 0
    assert dead.nonzero().flatten().tolist() == [5, 77]
    assert torch.allclose(Ug.cpu(), Uo, rtol=1e-3, atol=1e-5)
    # all-zero Hessian: every column dead, factor of (1 + 0.01) I
    Ug, dead, info = ops.gptq_hinv_(torch.zeros(K, K).cuda())
    assert dead.all() and info.item() == 0
    assert torch.allclose(Ug.cpu(), torch.eye(K) / (1.01 ** 0.5), atol=1e-6)


def _fix_dead(H):
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    return H


def _codes(wq, scale, g):
    s = scale.float().repeat_interleave(g, dim=1)
    return torch.round(wq.float() / s)


def _run_both(R, K, g, actorder, seed, bits=4, symmetric=True, blocksize=128, T=None, form=0):
    from llmcompressor_amd import ops

    torch.manual_seed(seed)
    w = (torch.randn(R, K) * 0.02).bfloat16()
    H, x = _hessian(K, T or 2 * K, seed + 1)
    n = 4.0
    args = F.QArgs(num_bits=bits, strategy="group", group_size=g, symmetric=symmetric, actorder=actorder)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    scale, zp = F.calculate_qparams(obs.min_vals, obs.max_vals, args)
    loss_o, out_o, info_o = G.quantize_weight(w, obs, args, (H / n).clone(), blocksize=blocksize)
    assert info_o["ok"]

    Hg = H.clone().cuda()
    perm = None
    if actorder:
        perm = torch.argsort(torch.diag(H / n), descending=True)
    g_idx = torch.arange(K, dtype=torch.int32) // g
    if actorder == "weight":
        g_idx = g_idx[perm]
    assert actorder != "group"
    U, dead, info = ops.gptq_hinv_(Hg, perm.cuda() if perm is not None else None, divisor=n, form=form)
    zpa = None if symmetric else zp.to(torch.int8).cuda()
    wq, loss = ops.gptq_quantize(w.cuda(), U, scale.cuda(), zpa, ops.FMT_INT, bits, 1, K // g, g_idx=g_idx.cuda(),
                                 perm=perm.cuda() if perm is not None else None, dead=dead, blocksize=blocksize,
                                 form=form)
    return w, x, scale, out_o["weight"], wq.cpu(), loss_o, loss.item()


@pytest.mark.parametrize(
    "R,K,g,actorder,kw",
    [
        (64, 256, 128, None, {}),
        (48, 384, 128, "weight", {}),
        (33, 200, 8, None, dict(blocksize=32)),
        (128, 512, 32, None, dict(symmetric=False)),
        (100, 512, 128, "weight", dict(bits=8)),
        (256, 1024, 128, None, {}),
    ],
)
def test_gptq_quantize_matches_oracle(R, K, g, actorder, kw):
    w, x, scale, wo, wg, loss_o, loss_g = _run_both(R, K, g, actorder, seed=R + K, **kw)
    agree = (wo == wg).float().mean().item()
    eo = ((w.float() - wo.float()) @ x.t()).norm().item()
    eg = ((w.float() - wg.float()) @ x.t()).norm().item()
    print(f"agreement {agree:.5f}  recon oracle {eo:.4f} gpu {eg:.4f}  loss {loss_o:.5g} {loss_g:.5g}")
    assert agree >= CODE_AGREEMENT
    assert abs(eg - eo) <= RECON_TOL * eo
    assert abs(loss_g - loss_o) <= 0.01 * abs(loss_o) + 1e-9


def test_gptq_diagonal_hessian_is_rtn_bit_exact():
    """Reference fixture (diagonal Hessian, distinct entries): no propagation, GPTQ == RTN exactly."""
    from llmcompressor_amd import ops

    torch.manual_seed(0)
    R, K, g = 6, 8, 2
    w = torch.nn.Linear(K, R, bias=False).weight.data.bfloat16()
    args = F.QArgs(num_bits=4, strategy="group", group_size=g)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    scale, zp = F.calculate_qparams(obs.min_vals, obs.max_vals, args)
    H = torch.diag(torch.arange(1, K + 1, dtype=torch.float32))
    U, dead, info = ops.gptq_hinv_(H.cuda())
    g_idx = torch.arange(K, dtype=torch.int32) // g
    wq, loss = ops.gptq_quantize(w.cuda(), U, scale.cuda(), None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx.cuda(), dead=dead)
    rtn = F.fake_quantize(w.float(), scale, zp, args).to(torch.bfloat16)
    assert torch.equal(wq.cpu(), rtn)
    assert loss.item() >= 0


def test_gptq_extreme_magnitudes_take_the_plain_division_route():
    """The column loop divides through hoisted reciprocals and falls back to plain divisions when a scale or a
    quotient leaves the range in which the short form is exact.  Tiny weights beside ordinary ones, whole
    groups of tiny weights (scale below 2^-60) and exact zeros force that route; with a diagonal Hessian the
    result must still be round-to-nearest bit for bit."""
    from llmcompressor_amd import ops

    torch.manual_seed(3)
    R, K, g = 24, 256, 32
    w = torch.randn(R, K)
    mag = torch.ones(R, K)
    mag[:, 32:64] = 1e-30                      # a whole group far below the reciprocal's range
    mag[:, 64:96:3] = 1e-20                    # tiny values beside ordinary ones: quotients below 2^-40
    mag[:, 130:140] = 0.0                      # exact zeros: zero dividends
    mag[5] = 1e-25
    w = (w * mag).bfloat16()
    args = F.QArgs(num_bits=4, strategy="group", group_size=g)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    scale, zp = F.calculate_qparams(obs.min_vals, obs.max_vals, args)
    H = torch.diag(torch.linspace(1.0, 3.0, K))
    U, dead, info = ops.gptq_hinv_(H.cuda())
    g_idx = torch.arange(K, dtype=torch.int32) // g
    wq, loss = ops.gptq_quantize(w.cuda(), U, scale.cuda(), None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx.cuda(), dead=dead)
    rtn = F.fake_quantize(w.float(), scale, zp, args).to(torch.bfloat16)
    assert torch.isfinite(wq.float()).all() and torch.isfinite(loss).all()
    assert torch.equal(wq.cpu(), rtn)


@pytest.mark.parametrize("K", [2048, 16640])
def test_gptq_permuted_columns_on_a_diagonal_hessian_are_rtn(K):
    """Activation ordering with a diagonal Hessian of distinct entries: the column loop runs in the permuted
    order, nothing propagates, and the result written back through the inverse permutation must be
    round-to-nearest bit for bit.  K = 2048 takes the gather / scatter kernels that move whole rows through
    LDS, K = 16640 is wider than they stage and takes the element-wise ones."""
    from llmcompressor_amd import ops

    torch.manual_seed(K)
    R, g = 8, 128
    w = (torch.randn(R, K) * 0.05).bfloat16()
    args = F.QArgs(num_bits=4, strategy="group", group_size=g)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    scale, zp = F.calculate_qparams(obs.min_vals, obs.max_vals, args)
    d = torch.rand(K) + 0.5
    perm = torch.argsort(d, descending=True).to(torch.int32)
    U, dead, info = ops.gptq_hinv_(torch.diag(d).cuda(), perm.cuda())
    assert info.item() == 0
    g_idx = (torch.arange(K, dtype=torch.int32) // g)[perm.long()]
    wq, loss = ops.gptq_quantize(w.cuda(), U, scale.cuda(), None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx.cuda(),
                                 perm=perm.cuda(), dead=dead)
    rtn = F.fake_quantize(w.float(), scale, zp, args).to(torch.bfloat16)
    assert torch.equal(wq.cpu(), rtn)
    # the factor of a diagonal matrix in the permuted order: 1 / sqrt(d + damp) on the diagonal
    damp = 0.01 * d.mean()
    expect = 1.0 / torch.sqrt(d[perm.long()] + damp)
    assert torch.allclose(torch.diagonal(U).cpu(), expect, rtol=1e-5)
    assert torch.count_nonzero(U.cpu() - torch.diag(torch.diagonal(U).cpu())) == 0


def test_gptq_zero_hessian_zeroes_weight_and_failure_is_rtn():
    from llmcompressor_amd import ops

    torch.manual_seed(1)
    R, K, g = 32, 256, 128
    w = (torch.randn(R, K) * 0.02).bfloat16()
    args = F.QArgs(num_bits=4, strategy="group", group_size=g)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    scale, zp = F.calculate_qparams(obs.min_vals, obs.max_vals, args)
    g_idx = (torch.arange(K, dtype=torch.int32) // g).cuda()
    U, dead, info = ops.gptq_hinv_(torch.zeros(K, K).cuda())
    wq, _ = ops.gptq_quantize(w.cuda(), U, scale.cuda(), None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx, dead=dead)
    assert torch.count_nonzero(wq) == 0
    U, dead, info = ops.gptq_hinv_((-torch.eye(K)).cuda())
    wq, _ = ops.gptq_quantize(w.cuda(), U, scale.cuda(), None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx, dead=dead)
    rtn = F.fake_quantize(w.float(), scale, zp, args).to(torch.bfloat16)
    assert torch.equal(wq.cpu(), rtn)


@pytest.mark.parametrize("R,K,T", [(1024, 4096, 8192), (512, 14336, 32768)])
def test_gptq_full_size_properties(R, K, T):
    """Llama-3-8B widths (the oracle would take minutes here): size-independent properties.
    Every output value lies on its group's int4 grid; GPTQ's layer reconstruction error beats
    round-to-nearest's; rescaling H leaves the codes unchanged; a narrower block width regroups the
    same fp32 sums (>= 99.9 % identical); U^T U (H/n + damp I) = I on sampled columns."""
    from llmcompressor_amd import ops

    torch.manual_seed(K)
    g = 128
    w = (torch.randn(R, K, device="cuda") * 0.02).bfloat16()
    x = torch.randn(T, K, device="cuda")
    x[:, torch.randperm(K, device="cuda")[: K // 100]] *= 20
    x = x.bfloat16()
    H = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H, x)
    mn, mx = ops.minmax_groups(w, g)
    scale, _, _ = ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, True)
    perm = torch.argsort(torch.diag(H), descending=True)
    g_idx = (torch.arange(K, dtype=torch.int32, device="cuda") // g)[perm]

    def run(Hin, blocksize=128, divisor=float(T)):
        U, dead, info = ops.gptq_hinv_(Hin.clone(), perm, divisor=divisor)
        assert int(info.item()) == 0
        wq, loss = ops.gptq_quantize(w, U, scale, None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx, perm=perm, dead=dead,
                                     blocksize=blocksize)
        return wq, loss, U

    wq, loss, U = run(H)
    # grid membership: q = wq / scale is an integer in [-8, 7] and q * scale reproduces wq in bf16
    s_full = scale.repeat_interleave(g, dim=1)
    q = (wq.float() / s_full.float()).round()
    assert q.min() >= -8 and q.max() <= 7
    assert torch.equal((q.to(torch.bfloat16) * s_full), wq)
    # reconstruction error vs round-to-nearest with the same scales
    rtn = ops.quantize(w, scale, None, ops.FMT_INT, 4, 1, K // g, g)
    xs = x.float()
    e_gptq = ((w.float() - wq.float()) @ xs.t()).norm().item()
    e_rtn = ((w.float() - rtn.float()) @ xs.t()).norm().item()
    assert e_gptq < 0.9 * e_rtn, (e_gptq, e_rtn)
    assert float(loss) > 0
    # codes are invariant to a positive rescaling of H (damping is relative)
    wq_s, _, _ = run(H * 3.0)
    assert (wq_s == wq).float().mean().item() >= CODE_AGREEMENT
    # block width only regroups fp32 sums
    wq_b, _, _ = run(H, blocksize=64)
    assert (wq_b == wq).float().mean().item() >= CODE_AGREEMENT
    # U^T U = (P^T H P / n + damp I)^-1 on sampled columns
    Hp = (H[perm][:, perm] / T).double()
    damp = 0.01 * torch.diag(Hp).mean()
    Hp += damp * torch.eye(K, device="cuda", dtype=torch.float64)
    cols = torch.tensor([0, 1, K // 2, K - 2, K - 1], device="cuda")
    Ud = U.double()
    got = Ud.t() @ (Ud @ Hp[:, cols])
    want = torch.eye(K, device="cuda", dtype=torch.float64)[:, cols]
    assert (got - want).abs().max().item() < 5e-3


@pytest.mark.parametrize("K,n,actorder", [(768, 5, False), (2048, 3, True), (200, 4, True)])
def test_hinv_grouped_is_bit_identical_to_single_calls(K, n, actorder):
    """llmc_gptq_hinv_grouped: the lock-step chain over n problems gives exactly the factors, dead-column
    flags and failure flags of n single calls (one problem is made indefinite, one has dead columns)."""
    from llmcompressor_amd import ops

    torch.manual_seed(K + n)
    Hs = []
    for b in range(n):
        x = torch.randn(3 * K if b != 1 else K // 2, K, device="cuda").bfloat16()
        H = torch.zeros(K, K, device="cuda")
        ops.hessian_accumulate_(H, x)
        if b == 2:
            H[5, :] = 0
            H[:, 5] = 0
        if b == n - 1:
            H = -H  # not positive definite: identity fallback, info != 0
        Hs.append(H)
    perms = torch.stack([torch.argsort(torch.diagonal(H), descending=True) for H in Hs]).to(torch.int32) if actorder else None
    divs = [float(b + 1) for b in range(n)]
    U, dead, info = ops.gptq_hinv_grouped(Hs, perms, divs, 0.01)
    for b in range(n):
        Hc = Hs[b].clone()
        Ub, db, ib = ops.gptq_hinv_(Hc, perms[b] if actorder else None, divisor=divs[b], percdamp=0.01)
        assert torch.equal(U[b], Ub), b
        assert torch.equal(dead[b], db)
        assert int(info[b]) == int(ib)
    assert int(info[n - 1]) != 0 and int(info[0]) == 0


@pytest.mark.parametrize("R,K,n,fmt_case", [(96, 768, 5, "int4_sym"), (64, 512, 4, "int4_asym_actorder"),
                                            (48, 256, 3, "nvfp4"), (1024, 4096, 2, "int4_sym"),
                                            (1024, 4608, 2, "int4_asym_actorder"),
                                            (3072, 512, 3, "int4_asym_actorder"), (3080, 256, 3, "nvfp4")])
def test_gptq_quantize_grouped_is_bit_identical_to_single_calls(R, K, n, fmt_case):
    """llmc_gptq_quantize_grouped on the factors of llmc_gptq_hinv_grouped: identical weights and losses to n
    single calls (int4 symmetric g128, int4 asymmetric g64 with activation ordering, NVFP4 with global scales).
    The two 1024-row cases reach the split-bf16 products of the trailing updates (the small ones stay on the fp32
    matrix instructions), whose choice must not depend on how many problems a call carries.  In the last two the
    grouped call carries more than 8192 rows and runs the block kernel with four lanes per row while the single
    calls use sixteen: the two layouts must give the same bits (3080 rows: a last workgroup that is partly empty in
    both)."""
    from llmcompressor_amd import ops

    torch.manual_seed(R + K)
    Ws = [(torch.randn(R, K, device="cuda") * 0.05).bfloat16() for _ in range(n)]
    Hs = []
    for b in range(n):
        x = torch.randn(2 * K, K, device="cuda").bfloat16()
        H = torch.zeros(K, K, device="cuda")
        ops.hessian_accumulate_(H, x)
        Hs.append(H)
    actorder = "actorder" in fmt_case
    perms = torch.stack([torch.argsort(torch.diagonal(H), descending=True) for H in Hs]).to(torch.int32) if actorder else None
    scales, zps, gss, gidx = [], [], [], []
    for b, W in enumerate(Ws):
        if fmt_case == "nvfp4":
            mn, mx = ops.minmax_groups(W, 16)
            gs = ops.global_scale_from_stats([(mn, mx)])
            s, _, _ = ops.calculate_qparams(mn, mx, ops.FMT_FP4, 4, True, ops.SCALE_NVFP4, gs)
            scales.append(s.float() if s.dtype not in (torch.float32, torch.bfloat16, torch.float16) else s)
            gss.append(gs)
            group = 16
        else:
            group = 64 if actorder else 128
            mn, mx = ops.minmax_groups(W, group)
            s, z, _ = ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, not actorder)
            scales.append(s)
            zps.append(z.to(torch.int8))
        g = torch.arange(K, dtype=torch.int32, device="cuda") // group
        gidx.append(g[perms[b].long()] if actorder else g)
    fmt = ops.FMT_FP4 if fmt_case == "nvfp4" else ops.FMT_INT
    zp_arg = zps if actorder else None
    gs_arg = gss if fmt_case == "nvfp4" else None
    U, dead, info = ops.gptq_hinv_grouped(Hs, perms, [2.0] * n, 0.01)
    assert int(info.abs().sum()) == 0
    outs, loss = ops.gptq_quantize_grouped(Ws, U, scales, zp_arg, fmt, 4, 1, K // group, g_idxs=gidx, perms=perms,
                                           dead=dead, global_scales=gs_arg)
    for b in range(n):
        ob, lb = ops.gptq_quantize(Ws[b], U[b], scales[b], zp_arg[b] if zp_arg else None, fmt, 4, 1, K // group,
                                   g_idx=gidx[b], perm=perms[b] if actorder else None, dead=dead[b],
                                   global_scale=gs_arg[b] if gs_arg else None)
        assert torch.equal(outs[b], ob), b
        assert torch.equal(loss[b:b + 1], lb)


@pytest.mark.parametrize("R,K", [(768, 2048), (2048, 768)])
def test_gptq_grouped_at_moe_layer_size(R, K):
    """128 expert Linears of one MoE layer (Qwen3-30B-A3B expert shapes, Zipf-routed token counts, two experts
    never routed) in one lock-step call: sampled problems equal the single-problem path bit for bit, every
    output lies on its group's int4 grid, idle experts come out zeroed with zero loss, and every expert with at
    least K tokens reports a positive finite loss."""
    from llmcompressor_amd import ops

    n, T, group = 128, 4096, 128
    gen = torch.Generator(device="cuda").manual_seed(R)
    logits = torch.randn(T, n, device="cuda", generator=gen) + torch.log(
        1.0 / torch.arange(1, n + 1, device="cuda").float() ** 1.1)
    logits[:, [17, 127]] = -1e9  # idle experts: no token, Hessian stays zero
    idx = torch.topk(logits, 8, -1).indices
    x_all = torch.randn(T, K, device="cuda", generator=gen).bfloat16()
    Ws = [(torch.randn(R, K, device="cuda", generator=gen) * 0.02).bfloat16() for _ in range(n)]
    Hs = [torch.zeros(K, K, device="cuda") for _ in range(n)]
    xs = [x_all[(idx == e).any(-1)] for e in range(n)]
    ops.hessian_accumulate_grouped_(Hs, xs, alpha=2.0)
    counts = [int(x.shape[0]) for x in xs]
    assert counts[17] == 0 and counts[127] == 0 and max(counts) > 8 * min(c for c in counts if c)
    perms = torch.stack([torch.argsort(torch.diagonal(H), descending=True) for H in Hs]).to(torch.int32)
    scales, gidx = [], []
    base = torch.arange(K, dtype=torch.int32, device="cuda") // group
    for b, W in enumerate(Ws):
        mn, mx = ops.minmax_groups(W, group)
        s, _, _ = ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, True)
        scales.append(s)
        gidx.append(base[perms[b].long()])
    U, dead, info = ops.gptq_hinv_grouped([H.clone() for H in Hs], perms, [1.0] * n, 0.01)
    assert int(info.abs().sum()) == 0
    outs, loss = ops.gptq_quantize_grouped(Ws, U, scales, None, ops.FMT_INT, 4, 1, K // group, g_idxs=gidx,
                                           perms=perms, dead=dead)
    torch.cuda.synchronize()
    for b in (0, 17, 64, 126):
        Ub, db, ib = ops.gptq_hinv_(Hs[b].clone(), perms[b], divisor=1.0)
        assert torch.equal(Ub, U[b]) and torch.equal(db, dead[b])
        ob, lb = ops.gptq_quantize(Ws[b], Ub, scales[b], None, ops.FMT_INT, 4, 1, K // group, g_idx=gidx[b],
                                   perm=perms[b], dead=db)
        assert torch.equal(outs[b], ob), b
        assert torch.equal(loss[b:b + 1], lb)
    assert torch.count_nonzero(outs[17]) == 0 and torch.count_nonzero(outs[127]) == 0
    assert bool(dead[17].all()) and bool(dead[127].all())
    for b in (0, 5, 64, 126):  # grid membership: out / scale is an integer code in [-8, 7]
        s = scales[b].float().repeat_interleave(group, dim=1)
        code = outs[b].float() / s
        live = ~dead[b].bool()
        # dequantised values are rounded to bf16 after code * scale: compare against the rounded grid
        nearest = torch.round(code).clamp(-8, 7)
        regrid = (nearest * s).bfloat16().float()
        assert torch.equal(regrid[:, live], outs[b].float()[:, live]), b
        assert torch.count_nonzero(outs[b][:, ~live]) == 0
    assert torch.isfinite(loss).all() and float(loss[17]) == 0.0
    routed = [b for b in range(n) if counts[b] >= K]
    assert all(float(loss[b]) > 0 for b in routed)


@pytest.mark.parametrize("K,n", [(64, 1), (1000, 3), (4096, 6), (14336, 1), (16384, 2), (2048, 300)])
def test_diag_argsort_is_torchs_stable_descending_argsort(K, n):
    """The column order of the activation ordering from one launch: equal to
    ``torch.argsort(diag, descending=True, stable=True)`` (the reference sorts with torch's unstable argsort,
    gptq_quantize.py:131-140, which agrees wherever no two entries are equal), including runs of exact ties,
    zeros of either sign, infinities and NaN."""
    from llmcompressor_amd import ops

    g = torch.Generator().manual_seed(K + n)
    Hs = []
    for b in range(n):
        d = torch.rand(K, generator=g) * 10
        d[torch.randperm(K, generator=g)[: K // 5]] = 3.25      # a run of exact ties
        d[torch.randperm(K, generator=g)[: K // 9]] = 0.0
        d[torch.randperm(K, generator=g)[: K // 11]] = -0.0
        if b % 2 and K > 100:
            d[7], d[K - 3], d[K // 2] = float("inf"), float("-inf"), float("nan")
            d[11] = float("nan")
        H = torch.randn(K, K, generator=g) if K <= 4096 else torch.zeros(K, K)
        H.diagonal().copy_(d)
        Hs.append(H.to("cuda"))
    got = ops.diag_argsort_desc(Hs)
    want = torch.argsort(torch.stack([torch.diagonal(H) for H in Hs]), dim=1, descending=True, stable=True)
    assert got.dtype == torch.int64 and got.shape == (n, K)
    assert torch.equal(got, want)


# ---- the factor in groups: Cholesky factor of H outside 512-column diagonal blocks, its inverse inside ----------

def test_factor_form_choice():
    from llmcompressor_amd import ops

    assert ops.gptq_factor_form(14336, 128) == ops.FACTOR_GROUPS
    assert ops.gptq_factor_form(8192, 512) == ops.FACTOR_GROUPS
    assert ops.gptq_factor_form(4096, 128) == ops.FACTOR_INVERSE   # the chain's saving does not pay for the loop's cost
    assert ops.gptq_factor_form(11008 + 8192, 128) == ops.FACTOR_GROUPS  # not a multiple of 512: a short first group
    assert ops.gptq_factor_form(14336 + 64, 128) == ops.FACTOR_INVERSE   # 128-column blocks would straddle two groups
    assert ops.gptq_factor_form(14336, 64) == ops.FACTOR_INVERSE   # narrower column blocks


def test_factor_form_is_checked_by_every_entry_point():
    """A form the width or the column blocks do not allow, or a number that names no form, is refused by the
    library before anything is launched (the weight and the Hessian stay as they were)."""
    from llmcompressor_amd import ops

    K = 192  # not a multiple of 128
    H = _hessian(K, 3 * K, 3)[0].cuda()
    keep = H.clone()
    with pytest.raises(ValueError, match="llmc_gptq_hinv: argument 7"):
        ops.gptq_hinv_(H, form=ops.FACTOR_GROUPS)
    with pytest.raises(ValueError, match="llmc_gptq_hinv: argument 7"):
        ops.gptq_hinv_(H, form=5)
    with pytest.raises(ValueError, match="llmc_gptq_hinv_grouped: argument 8"):
        ops.gptq_hinv_grouped([H, H.clone()], form=ops.FACTOR_GROUPS)
    assert torch.equal(H, keep)
    K = 256
    H = _hessian(K, 3 * K, 4)[0].cuda()
    U, dead, _ = ops.gptq_hinv_(H.clone(), form=ops.FACTOR_GROUPS)
    W = (torch.randn(8, K, device="cuda") * 0.05).bfloat16()
    Wkeep = W.clone()
    scale = torch.full((8, K // 128), 0.01, device="cuda", dtype=torch.bfloat16)
    g_idx = (torch.arange(K, dtype=torch.int32) // 128).cuda()
    args = (W, U, scale, None, ops.FMT_INT, 4, 1, K // 128, g_idx)
    with pytest.raises(ValueError, match="llmc_gptq_quantize: argument 20"):
        ops.gptq_quantize(*args, dead=dead, blocksize=64, form=ops.FACTOR_GROUPS)  # blocks narrower than 128
    with pytest.raises(ValueError, match="llmc_gptq_quantize: argument 20"):
        ops.gptq_quantize(*args, dead=dead, form=3)
    with pytest.raises(ValueError, match="llmc_sparsegpt_sparsify: argument 13"):
        ops.sparsegpt_sparsify(W, U, 0.5, dead=dead, blocksize=64, form=ops.FACTOR_GROUPS)  # exactly 128 there
    assert torch.equal(W, Wkeep)
    out, _ = ops.gptq_quantize(*args, dead=dead, form=ops.FACTOR_GROUPS)
    assert out.shape == W.shape and torch.isfinite(out.float()).all()


def _groups(K):
    """Column ranges of the diagonal blocks: 512 wide, aligned to the last column, the first one what is left."""
    first = K % 512 or 512
    edges = [0] + list(range(first, K + 1, 512))
    return list(zip(edges[:-1], edges[1:]))


@pytest.mark.parametrize("K,use_perm", [(1024, False), (1536, True), (2048, True), (1152, True), (1920, False)])
def test_grouped_factor_is_the_cholesky_factor_outside_the_diagonal_blocks(K, use_perm):
    """form = FACTOR_GROUPS against fp64: V V^T = H (V upper) outside the 512-blocks (aligned to the last column; a
    width that is not a multiple of 512 starts with a short one), inv(V[G, G]) inside; the diagonal blocks agree
    with the other form's U to fp32 rounding."""
    from llmcompressor_amd import ops

    H, _ = _hessian(K, 3 * K, K + 1)
    n = 5.0
    perm = torch.argsort(torch.diag(H), descending=True) if use_perm else None
    Hd = (H / n).double()
    if use_perm:
        Hd = Hd[perm][:, perm]
    Hd = Hd + 0.01 * Hd.diag().mean() * torch.eye(K, dtype=torch.float64)
    V64 = torch.flip(torch.linalg.cholesky(torch.flip(Hd, (0, 1))), (0, 1))  # upper, V V^T = H
    assert (V64 @ V64.t() - Hd).abs().max() / Hd.abs().max() < 1e-12 and torch.equal(V64, torch.triu(V64))
    want = V64.clone()
    for g0, g1 in _groups(K):
        want[g0:g1, g0:g1] = torch.linalg.inv(V64[g0:g1, g0:g1])
    pg = perm.cuda() if use_perm else None
    M, dead, info = ops.gptq_hinv_(H.clone().cuda(), pg, divisor=n, percdamp=0.01, form=ops.FACTOR_GROUPS)
    U, _, _ = ops.gptq_hinv_(H.clone().cuda(), pg, divisor=n, percdamp=0.01)
    M, U = M.cpu(), U.cpu()
    assert info.item() == 0 and dead.sum().item() == 0 and torch.equal(M, torch.triu(M))
    for g0, g1 in _groups(K):
        G_ = slice(g0, g1)
        blk, ref = M[G_, G_].double(), want[G_, G_]
        assert ((blk - ref).norm() / ref.norm()).item() < 2e-5
        assert ((blk - U[G_, G_].double()).norm() / ref.norm()).item() < 2e-5
        if g0:
            off, ref = M[:g0, G_].double(), want[:g0, G_]
            assert ((off - ref).norm() / ref.norm()).item() < 1e-5
    # a failed factorisation leaves the identity in this form too
    Mf, _, inf = ops.gptq_hinv_((-torch.eye(K)).cuda(), form=ops.FACTOR_GROUPS)
    assert inf.item() != 0 and torch.equal(Mf.cpu(), torch.eye(K))


@pytest.mark.parametrize(
    "R,K,g,actorder,kw",
    [
        (96, 1024, 128, None, {}),
        (200, 1536, 128, "weight", dict(symmetric=False)),
        (128, 2048, 32, "weight", {}),
        (256, 1024, 128, None, dict(bits=8)),
        (96, 1152, 128, "weight", {}),                       # a first group of 128 columns, then two of 512
        (64, 1920, 64, None, dict(symmetric=False)),         # a first group of 384 columns
        # fewer tokens than columns: only the damping keeps H regular, and an fp32 factor is then ~1e-5 from the exact
        # one whoever computes it (the fp32 oracle itself agrees with its fp64 run on 99.81 % of these 8-bit codes,
        # this form on 99.79 %, the other on 99.75 %): the bar of the rank-deficient expert Hessians
        (256, 1024, 128, None, dict(bits=8, T=700, bar=0.997)),
    ],
)
def test_gptq_from_the_grouped_factor_matches_the_oracle(R, K, g, actorder, kw):
    """The column loop in its left-looking form (what every group owes to earlier columns comes from the Cholesky
    factor of H) against the oracle, which follows the reference's U-based loop: same bar as the other form."""
    from llmcompressor_amd import ops

    kw = dict(kw)
    bar = kw.pop("bar", CODE_AGREEMENT)
    w, x, scale, wo, wg, loss_o, loss_g = _run_both(R, K, g, actorder, seed=R + K, form=ops.FACTOR_GROUPS, **kw)
    agree = (wo == wg).float().mean().item()
    eo = ((w.float() - wo.float()) @ x.t()).norm().item()
    eg = ((w.float() - wg.float()) @ x.t()).norm().item()
    print(f"agreement {agree:.5f}  recon oracle {eo:.4f} gpu {eg:.4f}  loss {loss_o:.5g} {loss_g:.5g}")
    assert agree >= bar
    assert abs(eg - eo) <= RECON_TOL * eo
    assert abs(loss_g - loss_o) <= 0.01 * abs(loss_o) + 1e-9


@pytest.mark.parametrize("R,K", [(8192, 3072), (1024, 4096), (4096, 5120), (2048, 11008)])
def test_both_factor_forms_give_the_same_weights_at_size(R, K):
    """Sizes at which the contraction over the earlier columns is cut into pieces (8192 rows: four pieces at most,
    so the five groups before the last one of 3072 columns go 2 + 2 + 1, a shorter last piece)."""
    from llmcompressor_amd import ops

    torch.manual_seed(K + R)
    g = 128
    T = 2 * K
    w = (torch.randn(R, K, device="cuda") * 0.02).bfloat16()
    x = torch.randn(T, K, device="cuda")
    x[:, torch.randperm(K, device="cuda")[: K // 100]] *= 20
    x = x.bfloat16()
    H = torch.zeros(K, K, device="cuda")
    ops.hessian_accumulate_(H, x)
    mn, mx = ops.minmax_groups(w, g)
    scale, _, _ = ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, True)
    perm = torch.argsort(torch.diag(H), descending=True)
    g_idx = (torch.arange(K, dtype=torch.int32, device="cuda") // g)[perm]
    got = {}
    for form in (ops.FACTOR_INVERSE, ops.FACTOR_GROUPS):
        U, dead, info = ops.gptq_hinv_(H.clone(), perm, divisor=float(T), form=form)
        assert int(info.item()) == 0
        got[form] = ops.gptq_quantize(w, U, scale, None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx, perm=perm, dead=dead,
                                      form=form)
    (wa, la), (wb, lb) = got[0], got[1]
    assert (wa == wb).float().mean().item() >= CODE_AGREEMENT
    assert abs(float(la) - float(lb)) <= 2e-3 * abs(float(la))
    xs = x.float()
    ea = ((w.float() - wa.float()) @ xs.t()).norm().item()
    eb = ((w.float() - wb.float()) @ xs.t()).norm().item()
    assert abs(ea - eb) <= RECON_TOL * ea


def test_grouped_calls_give_the_bits_of_single_calls_in_the_grouped_factor_form():
    from llmcompressor_amd import ops

    torch.manual_seed(5)
    n, R, K, g = 3, 256, 1536, 128
    Hs, Ws, scales, gidx = [], [], [], []
    for b in range(n):
        H, _ = _hessian(K, 2 * K, 100 + b)
        Hs.append(H.cuda())
        w = (torch.randn(R, K) * 0.02).bfloat16().cuda()
        Ws.append(w)
        mn, mx = ops.minmax_groups(w, g)
        scales.append(ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, True)[0])
    perms = torch.stack([torch.argsort(torch.diag(H), descending=True, stable=True) for H in Hs]).to(torch.int32)
    gidx = [(torch.arange(K, dtype=torch.int32, device="cuda") // g)[perms[b].long()] for b in range(n)]
    form = ops.FACTOR_GROUPS
    U, dead, info = ops.gptq_hinv_grouped([H.clone() for H in Hs], perms, [2.0] * n, 0.01, form=form)
    assert int(info.abs().sum()) == 0
    outs, loss = ops.gptq_quantize_grouped(Ws, U, scales, None, ops.FMT_INT, 4, 1, K // g, g_idxs=gidx, perms=perms,
                                           dead=dead, form=form)
    for b in range(n):
        Ub, db, ib = ops.gptq_hinv_(Hs[b].clone(), perms[b], divisor=2.0, form=form)
        assert torch.equal(Ub, U[b]) and torch.equal(db, dead[b])
        ob, lb = ops.gptq_quantize(Ws[b], Ub, scales[b], None, ops.FMT_INT, 4, 1, K // g, g_idx=gidx[b], perm=perms[b],
                                   dead=db, form=form)
        assert torch.equal(ob, outs[b]) and torch.equal(lb.reshape(()), loss[b])


def _grid_values(fmt_name, bits):
    if fmt_name == "fp4":
        pos = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
        return torch.cat([-pos.flip(0), pos])
    return torch.arange(-(1 << (bits - 1)), 1 << (bits - 1)).float()


@pytest.mark.parametrize(
    "R,K,fmt_name,bits,group,sym,actorder,dead_cols,n",
    [
        (1, 1024, "int", 4, 128, True, False, 0, 1),        # a single row: every product on the fp32 instruction
        (17, 1536, "int", 4, 32, False, True, 3, 1),        # zero points, permuted columns, dead columns
        (100, 9216, "int", 4, 128, True, True, 0, 1),       # 17 earlier groups in 9 pieces, the last one shorter
        (513, 1024, "int", 8, 1024, True, False, 0, 1),     # per-channel scales, rows one past a tile
        (64, 2048, "fp4", 4, 16, True, False, 5, 2),        # NVFP4 grid with a global scale, two problems in lock-step
        (130, 1536, "fp8", 8, 1536, True, True, 0, 3),      # fp8 codes per channel, three problems
        (72, 1664, "int", 4, 128, True, True, 2, 2),        # a first group of 128 columns, two problems in lock-step
    ],
)
def test_factor_forms_agree_over_shapes_and_formats(R, K, fmt_name, bits, group, sym, actorder, dead_cols, n):
    """Edge shapes of the left-looking loop against the right-looking one on the device (which the oracle tests
    pin): >= 99.9 % identical weights, values on the format's grid, equal losses, dead columns zeroed -- for single
    and grouped calls."""
    from llmcompressor_amd import ops

    torch.manual_seed(R * 7 + K)
    dev = "cuda"
    fmt = {"int": ops.FMT_INT, "fp4": ops.FMT_FP4, "fp8": ops.FMT_FP8}[fmt_name]
    T = max(2 * K, 2048)
    Hs, Ws, scales, zps, gss, perms, gidx = [], [], [], [], [], [], []
    for b in range(n):
        x = torch.randn(T, K, device=dev) * (0.25 + 2 * torch.rand(K, device=dev))
        if dead_cols:
            x[:, torch.randperm(K, device=dev)[:dead_cols]] = 0
        x = x.bfloat16()
        H = torch.zeros(K, K, device=dev)
        ops.hessian_accumulate_(H, x)
        Hs.append(H)
        w = (torch.randn(R, K, device=dev) * 0.02).bfloat16()
        Ws.append(w)
        mn, mx = ops.minmax_groups(w, group)
        gs = None
        if fmt_name == "fp4":
            gs = (448.0 * 6.0 / w.abs().max().float()).reshape(1)
            s, z, _ = ops.calculate_qparams(mn, mx, fmt, bits, True, ops.SCALE_NVFP4, gs)
        else:
            s, z, _ = ops.calculate_qparams(mn, mx, fmt, bits, sym)
        scales.append(s)
        zps.append(None if sym else z.to(torch.int8))
        gss.append(gs)
        perm = torch.argsort(torch.diag(H), descending=True, stable=True).to(torch.int32) if actorder else None
        perms.append(perm)
        g = torch.arange(K, dtype=torch.int32, device=dev) // group
        gidx.append(g[perm.long()] if actorder else g)
    pstack = torch.stack(perms) if actorder else None
    results = {}
    for form in (ops.FACTOR_INVERSE, ops.FACTOR_GROUPS):
        if n == 1:
            U, dead, info = ops.gptq_hinv_(Hs[0].clone(), perms[0], divisor=3.0, form=form)
            wq, loss = ops.gptq_quantize(Ws[0], U, scales[0], zps[0], fmt, bits, 1, K // group, g_idx=gidx[0],
                                         perm=perms[0], dead=dead, global_scale=gss[0], form=form)
            outs, losses, deads = [wq], loss.reshape(1), dead.reshape(1, K)
        else:
            U, deads, info = ops.gptq_hinv_grouped([H.clone() for H in Hs], pstack, [3.0] * n, 0.01, form=form)
            outs, losses = ops.gptq_quantize_grouped(
                Ws, U, scales, None if sym else zps, fmt, bits, 1, K // group, g_idxs=gidx, perms=pstack, dead=deads,
                global_scales=gss if fmt_name == "fp4" else None, form=form)
        assert int(info.abs().sum()) == 0
        results[form] = ([o.clone() for o in outs], losses.clone(), deads.clone())
    (oa, la, da), (ob, lb, db) = results[ops.FACTOR_INVERSE], results[ops.FACTOR_GROUPS]
    assert torch.equal(da, db) and int(da.sum()) == dead_cols * n
    grid = _grid_values(fmt_name, bits).to(dev) if fmt_name != "fp8" else None
    for b in range(n):
        agree = (oa[b] == ob[b]).float().mean().item()
        assert agree >= CODE_AGREEMENT, (b, agree)
        assert abs(float(la[b]) - float(lb[b])) <= 5e-3 * abs(float(la[b])) + 1e-12
        if actorder:
            inv = torch.empty(K, dtype=torch.long, device=dev)
            inv[perms[b].long()] = torch.arange(K, device=dev)
            dead_orig = db[b].bool()[inv]
        else:
            dead_orig = db[b].bool()
        assert torch.count_nonzero(ob[b][:, dead_orig]) == 0
        if grid is not None and sym and fmt_name == "int":
            s_full = scales[b].float().repeat_interleave(group, dim=1)[:, :K]
            q = ob[b].float() / s_full
            # q * scale was rounded to bf16: the quotient is an integer to within 2^-8 of its magnitude
            assert torch.all((q - q.round()).abs() <= 0.005 * q.abs() + 1e-6)
            assert q.round().min() >= grid.min() and q.round().max() <= grid.max()
