"""GPU parity: MSE grid-search observer through the C ABI vs the CPU oracle.

fp32 inputs reproduce the reference's eight known-answer losses (tests/llmcompressor/observers/
test_mse.py:9-42) to the reference's own abs=1e-10.  For bf16 weights every intermediate is
rounded to bf16, so near-ties between neighbouring shrink steps are common; the kernels form
|e|^2.4 as exp2(2.4 log2 e) in extended precision and fall back to powf only where the 16-bit
rounding of the two could differ, so the search picks the oracle's (min, max) for every group:
the fixed cases below assert equality (as the 60-case sweep in test_gpu_sweeps.py does).
"""
import pytest
import torch

from oracle import observers as O
from oracle import qformat as F

pytestmark = pytest.mark.gpu



def _gpu_minmax(w, args, **kw):
    from llmcompressor_amd import ops

    fmt = ops.FMT_INT if args.type == "int" else (ops.FMT_FP8 if args.num_bits == 8 else ops.FMT_FP4)
    mode = ops.SCALE_MXFP4 if args.is_mx else ops.SCALE_PLAIN
    wg = w.cuda()
    R, K = w.shape
    s = args.strategy
    if s == "tensor":
        mn, mx = ops.mse_observe_groups(wg.reshape(1, -1), R * K, fmt, args.num_bits, args.symmetric, mode, **kw)
        return mn.view(1), mx.view(1)
    if s == "channel":
        return ops.mse_observe_groups(wg, K, fmt, args.num_bits, args.symmetric, mode, **kw)
    if s in ("group", "tensor_group"):
        return ops.mse_observe_groups(wg, args.group_size, fmt, args.num_bits, args.symmetric, mode, **kw)
    bh, bw = args.block_structure
    return ops.mse_observe_blocks(wg, bh, bw, fmt, args.num_bits, args.symmetric, mode, **kw)


def test_known_answer_losses_fp32(golden):
    g = golden["mse_observer"]
    tensor = torch.arange(24).reshape((6, 4)) / 24
    for strategy, symmetric, exp_loss in g["cases"]:
        args = F.QArgs(num_bits=8, strategy=strategy, symmetric=symmetric,
                       group_size=(2 if strategy == "group" else None),
                       block_structure=([3, 2] if strategy == "block" else None))
        mn, mx = _gpu_minmax(tensor, args)
        scale, zp = F.calculate_qparams(mn.cpu(), mx.cpu(), args)
        q = F.fake_quantize(tensor, scale, zp, args)
        loss = torch.sum((tensor - q).abs().pow(2)) / tensor.numel()
        assert loss.item() == pytest.approx(exp_loss, abs=g["abs_tol"]), (strategy, symmetric)


CASES = {
    "int4_g128": (dict(num_bits=4, strategy="group", group_size=128), {}),
    "int4_g32_asym": (dict(num_bits=4, strategy="group", group_size=32, symmetric=False), {}),
    "nvfp4_g16_classic": (dict(num_bits=4, type="float", strategy="tensor_group", group_size=16,
                               scale_dtype=torch.float8_e4m3fn), dict(maxshrink=0.8, patience=100)),
    "mxfp4_g32_classic": (dict(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype=torch.uint8),
                          dict(maxshrink=0.8, patience=100)),
    "fp8_channel": (dict(num_bits=8, type="float", strategy="channel"), {}),
    "int8_tensor": (dict(num_bits=8, strategy="tensor"), {}),
    "nvfp4_expanded": (dict(num_bits=4, type="float", strategy="tensor_group", group_size=16,
                            scale_dtype=torch.float8_e4m3fn),
                       dict(expand=1.8, maxshrink=1 - 0.8 / 1.8, grid=200.0, patience=1000)),
}


@pytest.mark.parametrize("name", list(CASES))
def test_mse_matches_oracle_bf16(name):
    akw, okw = CASES[name]
    args = F.QArgs(**akw)
    torch.manual_seed(len(name))
    w = (torch.randn(64, 512) * 0.05).bfloat16()
    w[3, 17] = 1.5
    flat = O.flatten_for_calibration(w, "weight", args)
    emn, emx = O.grid_search_mse(flat, args, **{**dict(maxshrink=0.2, patience=5, grid=100.0, norm=2.4, expand=1.0), **okw})
    mn, mx = _gpu_minmax(w, args, **okw)
    mn, mx = mn.cpu().reshape(emn.shape), mx.cpu().reshape(emx.shape)
    same = ((mn == emn) & (mx == emx)).float().mean().item()
    print(f"{name}: groups identical {same:.4f}")
    assert torch.equal(mn, emn) and torch.equal(mx, emx), same

    # the chosen ranges are as good as the oracle's
    def qerr(a, b):
        sargs = args.copy(scale_dtype=None) if args.strategy == "tensor_group" else args
        s, z = F.calculate_qparams(a, b, sargs)
        q = F.fake_quantize(flat, s.unsqueeze(-1), z.unsqueeze(-1), sargs.copy(strategy="token"))
        return (q.float() - flat.float()).abs().pow(2.4).sum().item()

    assert qerr(mn, mx) <= 1.02 * qerr(emn, emx)


def test_global_patience_stop_is_reproduced():
    """A group that keeps improving late must be cut off by the global stop exactly like the host loop."""
    args = F.QArgs(num_bits=4, strategy="group", group_size=16)
    torch.manual_seed(0)
    w = (torch.randn(8, 64) * 0.02).bfloat16()
    for patience in (1, 2, 3, 5, 50):
        flat = O.flatten_for_calibration(w, "weight", args)
        emn, emx = O.grid_search_mse(flat, args, maxshrink=0.8, patience=patience)
        mn, mx = _gpu_minmax(w, args, maxshrink=0.8, patience=patience)
        assert torch.equal(mn.cpu().reshape(emn.shape), emn) and torch.equal(mx.cpu().reshape(emx.shape), emx), patience
