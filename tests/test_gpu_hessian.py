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
