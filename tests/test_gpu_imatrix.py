"""iMatrix (importance-weighted MSE) observer on the GPU against the CPU oracle.

The search compares fp32 sums whose order differs between the kernel and torch's reductions, so two
candidates whose errors agree to the last bits may swap: groups identical >= 99 %, and every differing group
must have picked a candidate whose weighted error is within 1e-5 of the oracle's choice."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import observers as O  # noqa: E402
from oracle.qformat import QArgs, calculate_qparams, fake_quantize  # noqa: E402

DEV = "cuda"


def _err(obs, args, mn, mx, imp, norm):
    token = args.copy(strategy="token")
    a = args.copy(scale_dtype=None) if args.strategy == "tensor_group" else args
    token = token.copy(scale_dtype=None) if args.strategy == "tensor_group" else token
    s, z = calculate_qparams(mn, mx, a)
    q = fake_quantize(obs, s.unsqueeze(-1), z.unsqueeze(-1), token)
    return ((q.double() - obs.double()).abs() ** norm * imp.double()).sum(dim=(0, -1))


@pytest.mark.parametrize("case", [
    dict(strategy="group", group_size=32, num_bits=4, symmetric=True),
    dict(strategy="group", group_size=128, num_bits=4, symmetric=False),
    dict(strategy="channel", num_bits=4, symmetric=True),
    dict(strategy="channel", num_bits=8, symmetric=True, kw=dict(norm=2.4, maxshrink=0.5, grid=40)),
    dict(strategy="tensor_group", group_size=16, num_bits=4, type="float", symmetric=True, scale_dtype=torch.float8_e4m3fn),
    dict(strategy="group", group_size=32, num_bits=4, symmetric=True, dtype=torch.float32, kw=dict(patience=0)),
    dict(strategy="group", group_size=64, num_bits=4, symmetric=True, dtype=torch.float16, uniform=True),
], ids=lambda c: f"{c['strategy']}-{c.get('group_size')}-{c.get('num_bits')}")
def test_imatrix_observer_matches_oracle(case):
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs

    case = dict(case)
    kw = case.pop("kw", {})
    dtype = case.pop("dtype", torch.bfloat16)
    uniform = case.pop("uniform", False)
    R, K = 96, 512
    g = torch.Generator().manual_seed(17)
    w = (torch.randn(R, K, generator=g) * 0.05).to(dtype)
    imp_raw = torch.rand(K, generator=g) ** 4 * 10 + 1e-3
    qa = QuantizationArgs(observer="imatrix_mse", observer_kwargs=dict(kw), **case)
    lin = torch.nn.Linear(K, R, bias=False, dtype=dtype, device=DEV)
    lin.weight.data.copy_(w)
    obs = Observer.load_from_registry("imatrix_mse", base_name="weight", args=qa)
    obs.attach(lin)
    if not uniform:
        obs._imatrix_sum = imp_raw.to(DEV) * 3
        obs._imatrix_count = torch.tensor(3, dtype=torch.int64, device=DEV)
    obs(lin.weight)
    mn_g, mx_g = obs.min_vals.cpu(), obs.max_vals.cpu()

    oa = QArgs(**{k: v for k, v in case.items()})
    observed = O.flatten_for_calibration(w, "weight", oa)
    imp = O.prepare_importance(imp_raw * 3, 3, observed, oa) if not uniform else None
    mn_o, mx_o = O.imatrix_grid_search(observed, oa, importance_weights=imp, **kw)
    mn_o, mx_o = mn_o.reshape(mn_g.shape), mx_o.reshape(mx_g.shape)
    same = (mn_g == mn_o) & (mx_g == mx_o)
    assert same.float().mean().item() >= 0.99, same.float().mean().item()
    if not bool(same.all()):
        ones = torch.ones_like(observed, dtype=torch.float32) if imp is None else imp
        norm = kw.get("norm", 3.0)
        shp = torch.amin(observed, dim=(0, -1)).shape
        e_g = _err(observed, oa, mn_g.reshape(shp), mx_g.reshape(shp), ones, norm).reshape(mn_g.shape)
        e_o = _err(observed, oa, mn_o.reshape(shp), mx_o.reshape(shp), ones, norm).reshape(mn_g.shape)
        assert bool((((e_g - e_o).abs() / e_o)[~same] < 1e-5).all())
    # qparams come out finite and the statistics (importance included) are dropped afterwards
    qp = obs.get_qparams()
    assert bool(torch.isfinite(qp["scale"].float()).all())
    assert not obs.has_statistics and not hasattr(obs, "_imatrix_sum")


def test_imatrix_hook_collects_sum_of_squares():
    """The forward-pre hook accumulates sum x^2 per input channel and the token count (imatrix.py:93-111);
    nothing is collected while hooks are disabled."""
    from llmcompressor_amd.modifiers.utils.hooks import HooksMixin
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs

    K = 1288
    lin = torch.nn.Linear(K, 16, bias=False, dtype=torch.bfloat16, device=DEV)
    qa = QuantizationArgs(num_bits=4, symmetric=True, strategy="group", group_size=8, observer="imatrix_mse")
    obs = Observer.load_from_registry("imatrix_mse", base_name="weight", args=qa)
    obs.attach(lin)
    xs = [torch.randn(2, 77, K, generator=torch.Generator().manual_seed(i)).bfloat16() for i in range(3)]
    xs.append(torch.randn(5, K, generator=torch.Generator().manual_seed(9)).bfloat16())
    for x in xs:
        lin(x.to(DEV))
    with HooksMixin.disable_hooks():
        lin(xs[0].to(DEV))
    flat = torch.cat([x.reshape(-1, K) for x in xs]).double()
    ref = (flat ** 2).sum(0)
    assert int(obs._imatrix_count.item()) == flat.shape[0]
    assert ((obs._imatrix_sum.cpu().double() - ref).abs() / ref).max().item() < 1e-5
    obs.detach(lin)
    lin(xs[0].to(DEV))
    assert int(obs._imatrix_count.item()) == flat.shape[0]


def test_imatrix_fallbacks_and_strict():
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs

    lin = torch.nn.Linear(64, 8, bias=False, dtype=torch.bfloat16, device=DEV)
    base = dict(num_bits=4, symmetric=True, strategy="channel", observer="imatrix_mse")
    obs = Observer.load_from_registry("imatrix_mse", base_name="weight", args=QuantizationArgs(**base))
    obs.attach(lin)
    assert bool(torch.isfinite(obs(lin.weight).get_qparams()["scale"].float()).all())  # no data: uniform search
    strict = Observer.load_from_registry("imatrix_mse", base_name="weight",
                                         args=QuantizationArgs(observer_kwargs=dict(strict=True), **base))
    strict.attach(lin)
    with pytest.raises(ValueError, match="no importance data"):
        strict(lin.weight)
    strict._imatrix_sum = torch.ones(32, device=DEV)
    strict._imatrix_count = torch.tensor(1, device=DEV)
    with pytest.raises(ValueError, match="size mismatch"):
        strict(lin.weight)
    strict._imatrix_sum = -torch.ones(64, device=DEV)
    with pytest.raises(ValueError, match="negative"):
        strict(lin.weight)
    for bad in (dict(norm=float("nan")), dict(norm=-1.0), dict(grid=0), dict(patience=-1), dict(maxshrink=1.5)):
        with pytest.raises(ValueError):
            Observer.load_from_registry("imatrix_mse", base_name="weight",
                                        args=QuantizationArgs(observer_kwargs=bad, **base))


def test_imatrix_block_and_activation_fall_back_to_uniform_search():
    """Block-wise weights and non-weight observers take the uniform fp32-error search (imatrix.py:141-245;
    reference test_block_strategy / test_non_weight_base_name_non_strict_falls_back)."""
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs

    g = torch.Generator().manual_seed(3)
    w = (torch.randn(96, 160, generator=g) * 0.05).bfloat16()
    lin = torch.nn.Linear(160, 96, bias=False, dtype=torch.bfloat16, device=DEV)
    lin.weight.data.copy_(w)
    qa = QuantizationArgs(num_bits=4, symmetric=True, strategy="block", block_structure=[32, 64],
                          observer="imatrix_mse")
    obs = Observer.load_from_registry("imatrix_mse", base_name="weight", args=qa)
    obs.attach(lin)
    obs._imatrix_sum = torch.rand(160, device=DEV) + 0.1
    obs._imatrix_count = torch.tensor(1, dtype=torch.int64, device=DEV)
    obs(lin.weight)
    oa = QArgs(num_bits=4, symmetric=True, strategy="block", block_structure=[32, 64])
    observed = O.flatten_for_calibration(w, "weight", oa)
    mn_o, mx_o = O.imatrix_grid_search(observed, oa)
    same = (obs.min_vals.cpu() == mn_o.reshape(obs.min_vals.shape)) & (obs.max_vals.cpu() == mx_o.reshape(obs.max_vals.shape))
    assert same.float().mean().item() >= 0.9  # 15 blocks: at most one near-tie may swap

    x = (torch.randn(4, 33, 64, generator=g)).bfloat16()
    qa = QuantizationArgs(num_bits=8, symmetric=True, strategy="tensor", observer="imatrix_mse")
    aobs = Observer.load_from_registry("imatrix_mse", base_name="input", args=qa)
    aobs(x.to(DEV))
    oa = QArgs(num_bits=8, symmetric=True, strategy="tensor")
    mn_o, mx_o = O.imatrix_grid_search(O.flatten_for_calibration(x, "input", oa), oa)
    assert torch.equal(aobs.min_vals.cpu().reshape(-1), mn_o.reshape(-1))
    assert torch.equal(aobs.max_vals.cpu().reshape(-1), mx_o.reshape(-1))
