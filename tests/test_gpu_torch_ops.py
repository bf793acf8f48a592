"""GPU: the ``torch.ops.llmc.*`` registration of the C ABI, op by op against the CPU oracle."""
import pytest
import torch

from oracle import gptq as G
from oracle import observers as O
from oracle import pack as P
from oracle import qformat as F

pytestmark = pytest.mark.gpu


def test_torch_ops_run_the_hot_path_end_to_end():
    from llmcompressor_amd import ops, torch_ops  # noqa: F401

    llmc = torch.ops.llmc
    torch.manual_seed(3)
    R, K, g, T = 192, 512, 64, 1536
    w = (torch.randn(R, K) * 0.02).bfloat16()
    x = torch.randn(3, T // 3, K)
    x[:, :, 5] *= 12
    x = x.bfloat16()
    Ho, n = G.make_empty_hessian(K), torch.zeros(())
    Ho, n = G.accumulate_hessian(x, Ho, n)
    args = F.QArgs(num_bits=4, strategy="group", group_size=g)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    mn_o, mx_o = obs.min_vals.clone(), obs.max_vals.clone()
    scale_o, zp_o = F.calculate_qparams(mn_o, mx_o, args)
    _, exp, info = G.quantize_weight(w, obs, args, (Ho / n).clone())
    assert info["ok"]

    H = torch.zeros(K, K, device="cuda")
    for b in range(3):
        assert llmc.hessian_accum_(H, x[b].cuda()) is None  # in place
    assert ((H.cpu().double() - Ho.double()).norm() / Ho.double().norm()).item() <= 1e-5
    H2 = torch.zeros(K, K, device="cuda")
    llmc.hessian_accum_segments_(H2, [x[b].cuda() for b in range(3)])
    assert ((H2.cpu().double() - Ho.double()).norm() / Ho.double().norm()).item() <= 1e-5
    mn, mx = llmc.minmax_observe(w.cuda(), g)
    assert torch.equal(mn.cpu(), mn_o.reshape(mn.shape)) and torch.equal(mx.cpu(), mx_o.reshape(mx.shape))
    scale, zp, codes = llmc.qparams(mn, mx, ops.FMT_INT, 4, True)
    assert codes is None and torch.equal(scale.cpu(), scale_o)
    dead, inf = llmc.gptq_prepare_hinv_(H, None, float(n), 0.01)
    assert inf.item() == 0 and not dead.any()
    g_idx = (torch.arange(K, dtype=torch.int32) // g).cuda()
    wq, loss = llmc.gptq_quantize(w.cuda(), H, scale, None, ops.FMT_INT, 4, 1, K // g, g_idx=g_idx, dead=dead)
    assert (wq.cpu() == exp["weight"]).float().mean().item() >= 0.999
    packed = llmc.quant_pack(wq, scale, None, ops.FMT_INT, 4, 1, K // g, g, ops.OUT_PACKED)
    codes_g = F.quantize(wq.cpu(), scale_o, zp_o, args, dtype=torch.int8)
    assert torch.equal(packed.cpu(), P.pack_to_int32(codes_g, 4))
    # MSE observer and dynamic per-token through the dispatcher
    m_mn, m_mx = llmc.mse_observe(w.cuda(), g, ops.FMT_INT, 4, True)
    e_mn, e_mx = O.grid_search_mse(O.flatten_for_calibration(w, "weight", args), args)
    assert torch.equal(m_mn.cpu().reshape(-1), e_mn.reshape(-1)) and torch.equal(m_mx.cpu().reshape(-1), e_mx.reshape(-1))
    xa = x.reshape(-1, K)[:257].contiguous()
    out, s = llmc.fp8_dynamic_per_token(xa.cuda())
    targs = F.QArgs(num_bits=8, type="float", strategy="token", dynamic=True)
    want, want_scale = F.forward_quantize_dynamic(xa.unsqueeze(0), targs)
    assert torch.equal(out.cpu(), want[0]) and torch.equal(s.cpu().reshape(-1), want_scale.reshape(-1))


def test_torch_ops_refuse_host_tensors():
    from llmcompressor_amd import torch_ops  # noqa: F401

    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.llmc.minmax_observe(torch.zeros(4, 8, dtype=torch.bfloat16), 8)


def test_workspaces_are_per_thread_and_go_away_with_the_thread():
    """A call's scratch buffer is cached per (device, stream, host thread) in thread-local storage: a worker thread
    that has ended no longer pins its buffer, and release_workspaces() drops the buffers of the live threads."""
    import gc
    import threading

    import torch

    from llmcompressor_amd import ops

    ops.release_workspaces()
    w = torch.randn(64, 256, device="cuda").bfloat16()
    ops.minmax_groups(w, 64)
    mine = [s for s in ops._ws_stores if s]
    assert len(mine) == 1 and len(mine[0]) == 1
    seen = []

    def worker():
        ops.minmax_groups(w, 64)
        seen.append(len([s for s in ops._ws_stores if s]))

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen == [2]  # the worker had a buffer of its own
    del t
    gc.collect()
    assert len([s for s in ops._ws_stores if s]) == 1  # ... which went away with the thread
    ops.release_workspaces()
    assert not [s for s in ops._ws_stores if s]
    mn, mx = ops.minmax_groups(w, 64)  # and the next call simply allocates again
    assert torch.equal(mn, w.unflatten(-1, (-1, 64)).amin(-1))
