"""The quantise kernels form bf16(x / s) for bf16 x and s as bf16(x * y) with y within one ulp of 1/s
(csrc/qformat.h).  Exhaustive check of that claim on the host: every pair of bf16 significands, the quotient
in the normal range, y at the correctly rounded reciprocal and one ulp either side of it."""
import numpy as np
import torch


def _bf16_values(exponent):
    bits = (np.uint32(127 + exponent) << np.uint32(23)) | (np.arange(128, dtype=np.uint32) << np.uint32(16))
    return bits.view(np.float32)


def test_one_multiply_quotient_rounds_like_the_ieee_quotient():
    bad = 0
    for ex in (-20, -3, 0, 5):
        for es in (-17, -7, 0, 1, 9):
            x = _bf16_values(ex)[:, None]
            s = _bf16_values(es)[None, :]
            want = torch.from_numpy(x / s).to(torch.bfloat16)
            y0 = (np.float32(1.0) / s).astype(np.float32)
            for y in (y0, np.nextafter(y0, np.float32(np.inf)), np.nextafter(y0, np.float32(-np.inf))):
                for sign in (1.0, -1.0):
                    got = torch.from_numpy((np.float32(sign) * x * y).astype(np.float32)).to(torch.bfloat16)
                    bad += (got != sign * want).sum().item()
    assert bad == 0
