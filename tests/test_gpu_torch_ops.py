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
