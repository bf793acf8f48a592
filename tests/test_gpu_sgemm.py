"""GPU: llmc_sgemm, the fp32 product of the lazy trailing updates (W[:, i2:] -= Err1 @ Hinv[i1:i2, i2:],
gptq_quantize.py:245, and the products inside the Cholesky chain), through the C ABI against an fp64 product.

Tolerance: relative Frobenius error <= 2e-6 (fp32 accumulation over up to 2048 terms), and the split product on
the 16-bit matrix cores must be at least as accurate as 1.5 x the fp32 matrix instruction's error on the same
operands -- the property that lets it stand in for fp32 inside the Cholesky chain."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _operands(M, N, Kc, trans_b, flags, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    # rows of very different magnitude, as the panels of a Cholesky factor have
    A = torch.randn(M, Kc, device="cuda", generator=g) * torch.exp(2 * torch.randn(M, 1, device="cuda", generator=g))
    Bp = torch.randn(Kc, N, device="cuda", generator=g)
    if flags & 2:
        A = torch.tril(A)
    if flags & 4:
        Bp = torch.tril(Bp)
    B = Bp.t().contiguous() if trans_b else Bp.contiguous()
    C0 = torch.randn(M, N, device="cuda", generator=g)
    return A, B, Bp, C0


@pytest.mark.parametrize("M,N,Kc,trans_b,flags,alpha,beta", [
    (256, 512, 128, True, 0, -1.0, 1.0),      # 128-wide tiles, split
    (256, 512, 128, False, 0, -1.0, 1.0),
    (2048, 4096, 512, False, 0, -1.0, 1.0),   # 256-wide tiles, split: the rank-512 update of the column loop
    (4096, 4096, 256, True, 1, -1.0, 1.0),    # trailing update of the factorisation (lower triangle only)
    (1024, 2048, 2048, False, 4, 1.0, 0.0),   # inverse, first product (B lower triangular)
    (1024, 2048, 1024, False, 2, -1.0, 0.0),  # inverse, second product (A lower triangular)
    (200, 328, 72, True, 0, 0.5, 2.0),        # ragged: fp32 matrix instruction
    (64, 64, 64, False, 0, 1.0, 0.0),         # too small to split
])
def test_sgemm_matches_fp64(M, N, Kc, trans_b, flags, alpha, beta):
    from llmcompressor_amd import ops

    A, B, Bp, C0 = _operands(M, N, Kc, trans_b, flags, seed=M + N + Kc + flags)
    ref = alpha * (A.double() @ Bp.double()) + beta * C0.double()
    errs = {}
    for name, extra in (("auto", 0), ("fp32", ops.SGEMM_FP32_MFMA)):
        C = C0.clone()
        ops.sgemm_(C, A, B, alpha, beta, trans_b, flags | extra)
        if flags & ops.SGEMM_C_LOWER:
            low = torch.tril(torch.ones(M, N, dtype=torch.bool, device="cuda"))
            assert torch.equal(C[~low], C0[~low])  # nothing above the diagonal is written
            errs[name] = ((C.double() - ref)[low].norm() / ref[low].norm()).item()
        else:
            errs[name] = ((C.double() - ref).norm() / ref.norm()).item()
    print(f"rel err auto {errs['auto']:.2e} fp32 {errs['fp32']:.2e}")
    assert errs["auto"] <= 2e-6 and errs["fp32"] <= 2e-6
    assert errs["auto"] <= 1.5 * errs["fp32"] + 1e-8


def test_sgemm_rejects_bad_arguments():
    from llmcompressor_amd import _lib

    lib = _lib.lib()
    a = torch.zeros(8, 8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.llmc_sgemm(0, 8, a.data_ptr(), 8, a.data_ptr(), 8, 8, 8, 8, 1.0, 0.0, 0, 0, st) == -1
    assert lib.llmc_sgemm(a.data_ptr(), 8, a.data_ptr(), 8, a.data_ptr(), 4, 8, 8, 8, 1.0, 0.0, 0, 0, st) == -5
    assert lib.llmc_sgemm(a.data_ptr(), 8, a.data_ptr(), 8, a.data_ptr(), 8, 8, 8, 8, 1.0, 0.0, 0, 64, st) == -13
