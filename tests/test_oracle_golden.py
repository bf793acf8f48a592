"""Pins the CPU oracle against every value-level vector the reference's own tests hold."""
import math

import pytest
import torch

from oracle import observers as O
from oracle import qformat as F


def _args(d):
    d = dict(d)
    if "scale_dtype" in d:
        d["scale_dtype"] = getattr(torch, d["scale_dtype"])
    return F.QArgs(**d)


def _weight_qdq(weight, args, observer="memoryless_minmax"):
    obs = O.Observer(observer, "weight", args)
    obs(weight)
    mn, mx = obs.min_vals.clone(), obs.max_vals.clone()
    qp = obs.get_qparams()
    out = F.fake_quantize(weight, qp["scale"], qp["zero_point"], args, global_scale=qp["global_scale"])
    return mn, mx, out, qp


@pytest.mark.parametrize("idx", range(5))
def test_lifecycle_weight_goldens(golden, idx):
    case = golden["lifecycle_weight"]["cases"][idx]
    args = _args(case["args"])
    weight = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    mn, mx, out, _ = _weight_qdq(weight, args)
    assert torch.equal(mn, torch.tensor(case["min"], dtype=mn.dtype))
    assert torch.equal(mx, torch.tensor(case["max"], dtype=mx.dtype))
    exp = torch.tensor(case["quant"], dtype=torch.float32).to(torch.bfloat16)
    # the reference asserts allclose on a bf16 matmul-with-identity output; the
    # goldens are printed to 4 decimals, so compare after rounding both to bf16
    assert torch.equal(out.to(torch.bfloat16), exp), (out, exp)
    assert torch.nn.functional.mse_loss(out.float(), weight.float()) <= case["loss"]


def test_lifecycle_activation_tensor_golden(golden):
    case = golden["lifecycle_activation"]["cases"][0]
    args = _args(case["args"])
    x = torch.arange(12, dtype=torch.bfloat16).reshape(1, 2, 6)
    obs = O.Observer("minmax", "input", args)
    obs(x)
    assert torch.equal(obs.min_vals, torch.tensor(case["min"], dtype=torch.bfloat16))
    assert torch.equal(obs.max_vals, torch.tensor(case["max"], dtype=torch.bfloat16))
    qp = obs.get_qparams()
    out = F.fake_quantize(x, qp["scale"], qp["zero_point"], args)
    exp = torch.tensor(case["quant"]).to(torch.bfloat16)
    assert torch.equal(out, exp)


def test_lifecycle_activation_nvfp4_dynamic_local_golden(golden):
    case = golden["lifecycle_activation"]["cases"][1]
    args = _args(case["args"])
    x = torch.arange(12, dtype=torch.bfloat16).reshape(1, 2, 6)
    obs = O.Observer("minmax", "input", args)
    obs(x)
    gs = obs.get_qparams()["global_scale"]
    assert gs.dtype == torch.float32 and gs.item() == 244.0
    out, scale = F.forward_quantize_dynamic(x, args, global_scale=gs)
    exp = torch.tensor(case["quant"]).to(torch.bfloat16)
    assert torch.equal(out, exp), out
    assert scale.flatten().tolist() == [80.0, 208.0, 320.0, 448.0]


def test_lifecycle_attention_golden(golden):
    case = golden["lifecycle_attention"]
    args = _args(case["args"])
    x = torch.arange(12, dtype=torch.bfloat16).reshape(1, 2, 2, 3)
    obs = O.Observer("minmax", "k", args)
    obs(x)
    assert obs.min_vals.tolist() == case["min"] and obs.max_vals.tolist() == case["max"]
    qp = obs.get_qparams()
    out = F.fake_quantize(x, qp["scale"], qp["zero_point"], args)
    assert torch.equal(out, torch.tensor(case["quant"]).to(torch.bfloat16))


def test_nvfp4_weight_golden_scales():
    # discriminating vector: the global scale must be divided in bf16 (2688/23 -> 117.0)
    args = F.QArgs(num_bits=4, type="float", strategy="tensor_group", group_size=3, scale_dtype=torch.float8_e4m3fn)
    weight = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    _, _, out, qp = _weight_qdq(weight, args)
    assert qp["global_scale"].item() == 117.0
    assert qp["scale"].tolist() == [[40, 96], [160, 208], [288, 320], [384, 448]]
    assert out[2, 1].item() == 14.75


def test_mse_known_answers(golden):
    g = golden["mse_observer"]
    tensor = torch.arange(24).reshape((6, 4)) / 24
    for strategy, symmetric, exp_loss in g["cases"]:
        args = F.QArgs(
            num_bits=g["num_bits"],
            strategy=strategy,
            symmetric=symmetric,
            group_size=(2 if strategy == "group" else None),
            block_structure=([3, 2] if strategy == "block" else None),
            observer="mse",
        )
        obs = O.Observer("mse", "weight", args)
        qp = obs(tensor).get_qparams()
        q = F.fake_quantize(tensor, qp["scale"], qp["zero_point"], args)
        loss = torch.sum((tensor - q).abs().pow(2)) / tensor.numel()
        assert loss.item() == pytest.approx(exp_loss, abs=g["abs_tol"]), (strategy, symmetric)


def test_mse_fp4(golden):
    w = torch.arange(24, dtype=torch.bfloat16).reshape((4, 6)) / 24
    args = F.QArgs(num_bits=4, type="float", strategy="tensor_group", group_size=3)
    qp = O.Observer("mse", "weight", args)(w).get_qparams()
    q = F.fake_quantize(w, qp["scale"], qp["zero_point"], args, global_scale=qp["global_scale"])
    assert torch.nn.functional.mse_loss(q.float(), w.float()) <= golden["mse_fp4"]["max_mse"]


def test_minmax_qparams(golden):
    g = golden["minmax_qparams"]
    for symmetric, exp_scale, exp_zp in g["cases"]:
        args = F.QArgs(num_bits=8, symmetric=symmetric, observer="minmax")
        qp = O.Observer("minmax", "weight", args)(torch.tensor(g["tensor"])).get_qparams()
        assert round(qp["scale"].item(), 4) == exp_scale
        assert round(qp["zero_point"].item(), 4) == exp_zp


def test_minmax_ema_trajectory(golden):
    g = golden["minmax_ema"]
    inp = torch.tensor([[1, 1, 1, 1, 1]])
    seq = [inp, inp, torch.tensor([[127, 1, 1, 1, 1]]), inp, torch.tensor([[-128, 1, 1, 1, 1]])]
    obs = O.Observer("minmax", "input", F.QArgs(num_bits=8, strategy="tensor"))
    cmax, cmin = 1, 1
    for i, t in enumerate(seq):
        obs(t)
        cmax = max(obs.max_vals[0], cmax)
        cmin = min(obs.min_vals[0], cmin)
        if i < 2:
            assert cmax == 1 and cmin == 1
        elif i < 4:
            assert abs(cmax - g["max_after_update"]) < g["delta"] and cmin == 1
        else:
            assert abs(cmax - g["max_after_update"]) < g["delta"]
            assert abs(cmin - g["min_after_update"]) < g["delta"]


def test_observer_trajectories(golden):
    g = golden["observer_trajectories"]
    observed = torch.tensor(g["observed"])
    for name, kwargs, exp_min, exp_max in g["cases"]:
        obs = O.Observer(name, "input", F.QArgs(strategy="tensor"), **kwargs)
        mins, maxs = [], []
        for row in observed:
            obs(row)
            mins.append(obs.min_vals)
            maxs.append(obs.max_vals)
        assert torch.allclose(torch.stack(mins), torch.tensor(exp_min)), name
        assert torch.allclose(torch.stack(maxs), torch.tensor(exp_max)), name


@pytest.mark.parametrize(
    "kw,scale_shape",
    [
        (dict(strategy="tensor"), (1,)),
        (dict(strategy="channel"), (10, 1)),
        (dict(strategy="group", group_size=4), (10, 2)),
        (dict(strategy="tensor_group", group_size=4), (10, 2)),
        (dict(strategy="block", block_structure=[5, 4]), (2, 2)),
        (dict(strategy="block", block_structure=[3, 3]), (4, 3)),
    ],
)
def test_flatten_weight_shape_contract(kw, scale_shape):
    # reference: tests/llmcompressor/observers/test_helpers.py:37-59 (Linear(8, 10))
    w = torch.empty(10, 8)
    flat = O.flatten_for_calibration(w, "weight", F.QArgs(**kw))
    assert tuple(flat.shape[1:-1]) == scale_shape


def test_flatten_input_shape_contract():
    x = torch.empty(3, 5, 8)
    assert tuple(O.flatten_for_calibration(x, "input", F.QArgs(strategy="tensor")).shape[1:-1]) == (1,)
    assert tuple(
        O.flatten_for_calibration(x, "input", F.QArgs(strategy="tensor_group", group_size=4)).shape[1:-1]
    ) == (2,)


def test_fused_global_scale_closed_form():
    # reference: tests/llmcompressor/modifiers/utils/test_update_fused_layer_weights.py:72-120
    torch.manual_seed(0)
    ws = [torch.randn(8, 16).bfloat16() * s for s in (1.0, 3.0, 0.5)]
    args = [F.QArgs(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype=torch.float8_e4m3fn) for _ in ws]
    obs = [O.Observer("memoryless_minmax", "weight", a) for a in args]
    O.Observer.fuse(zip(obs, ws))
    gs = [o(w).get_qparams()["global_scale"] for o, w in zip(obs, ws)]
    absmax = max(w.abs().max().item() for w in ws)
    for g in gs:
        assert g.item() == pytest.approx(448 * 6 / absmax, rel=1e-2)
        assert g.item() == gs[0].item()
    assert all(not o.has_statistics for o in obs)


def test_fp8_cast_saturates_before_cast():
    # torch's e4m3 cast gives NaN above 448: the format path must clamp first
    x = torch.tensor([500.0, -1000.0, 448.0, 464.0])
    args = F.QArgs(num_bits=8, type="float")
    out = F.round_to_qtype(x, args, -448.0, 448.0)
    assert out.tolist() == [448.0, -448.0, 448.0, 448.0]


def test_cast_to_fp4_matches_torch_e2m1_table():
    # every bf16 value in [-6, 6] against an exhaustive nearest/ties-to-even-mantissa search
    grid = torch.tensor(F.E2M1_VALUES)
    xs = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    xs = xs[torch.isfinite(xs) & (xs.abs() <= 6)]
    got = F.cast_to_fp4(xs)
    d = (xs.abs().unsqueeze(-1) - grid).abs()
    mn = d.min(dim=-1, keepdim=True).values
    tie = (d == mn).sum(-1) > 1
    near = grid[d.argmin(-1)]
    # ties go to the even mantissa: grid indices 0,2,4,6 (0,1,2,4)
    even = torch.tensor([True, False, True, False, True, False, True, False])
    cand = torch.where((d == mn) & even, grid, torch.full_like(d, -1.0)).max(-1).values
    exp = torch.where(tie, cand, near)
    assert torch.equal(got.abs(), exp)
    assert torch.equal(torch.signbit(got), (xs < 0))


def test_generate_gparam_is_reciprocal_then_product():
    """``float / Tensor`` is ``Tensor.reciprocal() * float`` in torch, so the global scale of bf16 statistics
    carries two roundings; a single correctly rounded division differs for some absmax values (40.0)."""
    for v, want in ((40.0, 67.5), (23.0, 117.0), (11.0, 244.0)):
        t = torch.tensor([v], dtype=torch.bfloat16)
        gs = F.generate_gparam(-t, t)
        assert gs.dtype == torch.float32 and gs.item() == want
        assert gs.item() == (t.reciprocal() * 2688.0).float().item()
    assert (torch.tensor([2688.0]).bfloat16() / torch.tensor([40.0]).bfloat16()).item() == 67.0


# ---- what mathematics and the installed libraries can still say about the unpinned format rules -----------------

def _all_positive_normal_bf16():
    # exponent fields 3..253: every normal bf16 for which neither rule leaves the E8M0 range
    bits = torch.arange(3 << 7, 254 << 7, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def test_mxfp4_exponent_rule_against_the_ocp_mx_definition_over_every_bf16_maximum():
    """OCP Microscaling v1.0 (section 6.3): shared exponent = floor(log2(max|x|)) - emax(e2m1) with emax = 2.
    The oracle follows the bf16 bit-pattern rule of compressed-tensors (a rounding bump of 0x20 before the mantissa
    is dropped).  Brute force over every positive normal bf16 maximum (exponent fields 3..253): the two rules agree whenever the three
    leading mantissa bits are below 0b110; for mantissas >= 1.75 the bump carries into the exponent and the
    bit-pattern rule gives one more -- exactly those, nothing else.  (Which rule compressed-tensors' release
    applies cannot be confirmed without the package: the function stays parity unpinned.)"""
    amax = _all_positive_normal_bf16()
    got = F.mxfp4_scale_exponent(amax).to(torch.int32)
    ocp = (torch.floor(torch.log2(amax.double())) - 2 + 127).to(torch.int32)
    mant = amax.view(torch.int16).to(torch.int32) & 0x7F
    carries = mant >= 0x60  # 1.75 and above
    assert torch.equal(got[~carries], ocp[~carries])
    assert torch.equal(got[carries], ocp[carries] + 1)
    assert 0.24 < carries.float().mean().item() < 0.26
    # either way the scaled maximum amax / 2^(e-127) stays inside what e2m1 can round to 6 without clipping more
    # than its top step: OCP gives [4, 8), the bump rule [3.5, 7)
    ratio_bump = amax.double() / torch.pow(2.0, got.double() - 127)
    ratio_ocp = amax.double() / torch.pow(2.0, ocp.double() - 127)
    assert ratio_ocp.min() >= 4 and ratio_ocp.max() < 8
    assert ratio_bump.min() >= 3.5 and ratio_bump.max() < 7


def test_e8m0_code_is_the_byte_of_torch_float8_e8m0fnu():
    """The stored MXFP4 scale byte e stands for 2^(e-127): the same byte torch's float8_e8m0fnu cast produces
    for that power of two, for every exponent the rule can emit."""
    e = torch.arange(1, 255, dtype=torch.int32)
    value = torch.pow(2.0, (e - 127).double()).to(torch.float32)
    as_e8m0 = value.to(torch.float8_e8m0fnu).view(torch.uint8).to(torch.int32)
    assert torch.equal(as_e8m0, e)
    back = F.mxfp4_scale_from_exponent(e.float(), dtype=torch.float32)
    assert torch.equal(back, value)


def test_per_token_dynamic_fp8_against_the_consumer_side_definition():
    """Cross-check, not the oracle: an HF-side consumer of FP8 activations quantises per row with fp32 scales,
    scale = where(rowmax > 0, rowmax, 1) / 448, q = clamp(x / scale, +-448).to(e4m3)
    (transformers/integrations/compressed_tensors.py, the per-row FP8 helper).  The calibration-time path keeps the scale in
    the activation dtype (bf16).  On N(0,1) rows with outliers the two agree on the reduce dimension (one scale
    per token: the bf16 scale is the fp32 one rounded to bf16, row by row) and on >= 95 % of the code bytes; every
    differing byte is one e4m3 step away.  The remaining per-token rule (keepdim shape, dtype of the scale) is
    still parity unpinned."""
    torch.manual_seed(4)
    x = torch.randn(64, 512)
    x[::7, ::31] *= 15
    x = x.bfloat16()
    args = F.QArgs(num_bits=8, type="float", strategy="token", dynamic=True)
    scale, zp = F.compute_dynamic_scales_and_zp(x.unsqueeze(0), args)
    assert scale.shape == (1, 64, 1) and scale.dtype == torch.bfloat16
    rowmax = x.float().abs().amax(dim=-1, keepdim=True)
    s32 = torch.where(rowmax > 0, rowmax, torch.ones_like(rowmax)) / 448.0
    assert torch.equal(scale.reshape(-1), s32.to(torch.bfloat16).reshape(-1))
    q_consumer = torch.clamp(x.float() / s32, -448, 448).to(torch.float8_e4m3fn)
    q_oracle = F.quantize(x.unsqueeze(0), scale, zp, args, dtype=torch.float8_e4m3fn)[0]
    a, b = q_consumer.view(torch.uint8).to(torch.int32), q_oracle.view(torch.uint8).to(torch.int32)
    same = (a == b).float().mean().item()
    assert same >= 0.95
    assert ((a - b).abs() <= 1).all()
