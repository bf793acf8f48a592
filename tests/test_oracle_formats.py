"""Pins the oracle's storage formats (``oracle/pack.py``, the fp8 / e2m1 casts of ``oracle/qformat.py``) against
independent definitions that are importable here: the consumer-side MXFP4 decode of ``transformers``
(``transformers.integrations.mxfp4``: nibble order, sign bit, E8M0 bias), triton's OCP reference encoder
(``triton.tools.mxfp``, plain torch code), torch's own ``float8_e4m3fn`` / ``float8_e8m0fnu`` dtypes, and decodes
written here from the formats' bit fields.  Every test names the mistake it would catch and checks that the mistake
does fail (swapped nibbles, a dropped sign of -0, a wrong shift order, truncation instead of round-to-nearest-even).

Reference call sites of these formats: ``src/llmcompressor/transformers/compression/compressed_tensors_utils.py:134-138``,
``src/llmcompressor/entrypoints/model_free/process.py:125,205,226``; BLOCK inside the column loop:
``src/llmcompressor/modifiers/gptq/gptq_quantize.py:213-223``.
"""
import json
import os

import pytest
import torch

from oracle import gptq as G
from oracle import observers as O
from oracle import pack as P
from oracle import qformat as F


def _bits16(t):
    return t.contiguous().view(torch.int16)


def _all_bf16():
    return torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


# ---- e2m1 nibbles and E8M0 bytes: the consumer's decode must give back fake_quantize --------------------------------

def _mx_args():
    return F.QArgs(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype=torch.uint8)


def _mx_case(seed=0, R=24, K=256):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(R, K, generator=g) * torch.logspace(-6, 4, R).unsqueeze(1)
    w[3, 5:40] = 0.0                      # zeros of both signs inside a group
    w[3, 7] = -0.0
    w[5, ::2] *= -1e-3                    # tiny negatives: they round to -0
    w = w.bfloat16()
    args = _mx_args()
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    qp = obs.get_qparams()
    return w, args, qp


def test_mxfp4_bytes_decode_to_the_fake_quant_weight_with_the_transformers_consumer():
    mx = pytest.importorskip("transformers.integrations.mxfp4")
    w, args, qp = _mx_case()
    R, K = w.shape
    fq = F.fake_quantize(w, qp["scale"], qp["zero_point"], args)
    st = P.compress_weight(w, qp["scale"], qp["zero_point"], args)
    blocks = st["weight_packed"].reshape(1, R, K // 32, 16)
    scales = st["weight_scale"].reshape(1, R, K // 32)
    assert st["weight_scale"].dtype == torch.uint8 and st["weight_packed"].dtype == torch.uint8

    def consumer(b, s):
        # [1, R, G, 16] bytes + [1, R, G] exponents -> [1, K, R] values; back to [R, K]
        return mx._convert_moe_packed_tensors(b, s, dtype=torch.bfloat16)[0].t().contiguous()

    got = consumer(blocks, scales)
    # bit patterns, so that -0 is told from +0
    assert torch.equal(_bits16(got), _bits16(fq))
    assert (got == 0).any() and (torch.signbit(got) & (got == 0)).any(), "the case must exercise the -0 nibble"

    # the mistakes this has to catch
    swapped = ((blocks & 0xF) << 4) | (blocks >> 4)
    assert not torch.equal(_bits16(consumer(swapped, scales)), _bits16(fq)), "swapped nibbles went unnoticed"
    nosign0 = blocks.clone()
    lo, hi = nosign0 & 0xF, nosign0 >> 4
    lo = torch.where(lo == 8, torch.zeros_like(lo), lo)
    hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
    assert not torch.equal(_bits16(consumer(lo | (hi << 4), scales)), _bits16(fq)), "-0 stored as +0 went unnoticed"
    assert not torch.equal(_bits16(consumer(blocks, scales + 1)), _bits16(fq)), "an E8M0 bias off by one went unnoticed"


def test_e2m1_rounding_and_nibble_codes_against_the_ocp_reference_encoder_over_every_bf16():
    """triton.tools.mxfp.MXFP4Tensor is a brute-force nearest / ties-to-even-mantissa encoder with the OCP bit
    fields (sign<<3 | exponent<<1 | mantissa).  Every bf16 value of magnitude <= 6 (both zeros included) must get the
    same nibble from ``pack_fp4_to_uint8(cast_to_fp4(x))``, and the same byte when packed in pairs."""
    mxfp = pytest.importorskip("triton.tools.mxfp")
    x = _all_bf16()
    # the input -0.0 itself is left out: the cast is ``|x| rounded * sign(x)`` and torch's sign(-0.0) is +0, so it
    # codes as +0 (checked below); in the quantise chain the zeros zero point has turned it into +0 before anyway.
    # Negative values that round to zero keep their sign (nibble 8) in both encoders.
    x = x[torch.isfinite(x) & (x.abs() <= 6) & ~((x == 0) & torch.signbit(x))]
    if x.numel() % 2:
        x = x[:-1]
    assert P.pack_fp4_to_uint8(F.cast_to_fp4(torch.tensor([[-0.0, -0.1]]))).item() == 0x80
    want = mxfp.MXFP4Tensor(data=x.float().clone())
    nib_want = want.data.to(torch.int32)
    packed = P.pack_fp4_to_uint8(F.cast_to_fp4(x).reshape(1, -1)).reshape(-1).to(torch.int32)
    nib_got = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(-1)
    assert torch.equal(nib_got, nib_want)
    assert torch.equal(packed, want.to_packed_tensor(dim=0).to(torch.int32))
    # the decode side: both libraries' tables give back the rounded value, sign of zero included
    back = P.unpack_fp4_from_uint8(packed.to(torch.uint8).reshape(1, -1), dtype=torch.float32).reshape(-1)
    assert torch.equal(back.view(torch.int32), want.to(torch.float32).view(torch.int32))
    # ties: 0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4 (even mantissa)
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    assert F.cast_to_fp4(ties).tolist() == [0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0]


def test_nvfp4_bytes_scales_and_global_scale_decode_to_the_fake_quant_weight():
    """NVFP4 consumers form ``e2m1(nibble) * e4m3(scale byte) / global_scale``; the nibble table is the one
    transformers ships for MXFP4 (same e2m1 element format)."""
    mx = pytest.importorskip("transformers.integrations.mxfp4")
    torch.manual_seed(1)
    R, K = 16, 128
    w = (torch.randn(R, K) * torch.logspace(-3, 1, R).unsqueeze(1)).bfloat16()
    w[2, :16] = 0
    args = F.QArgs(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype=torch.float8_e4m3fn)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    qp = obs.get_qparams()
    fq = F.fake_quantize(w, qp["scale"], qp["zero_point"], args, global_scale=qp["global_scale"])
    st = P.compress_weight(w, qp["scale"], qp["zero_point"], args, global_scale=qp["global_scale"])
    assert st["weight_scale"].dtype == torch.float8_e4m3fn
    lut = torch.tensor(mx.FP4_VALUES, dtype=torch.float32)
    b = st["weight_packed"].to(torch.int64)
    vals = torch.stack([lut[b & 0xF], lut[b >> 4]], dim=-1).reshape(R, K)
    s = st["weight_scale"].to(torch.float32) / st["weight_global_scale"].to(torch.float32)
    got = (vals.reshape(R, K // 16, 16) * s.unsqueeze(-1)).reshape(R, K).to(torch.bfloat16)
    assert torch.equal(_bits16(got), _bits16(fq))
    # scales must survive the e4m3 byte unchanged (they were rounded to e4m3 when they were computed)
    assert torch.equal(st["weight_scale"].to(qp["scale"].dtype), qp["scale"])


# ---- fp8 storage: nearest-even over a decode of the 256 byte values written from the bit fields ----------------------

def _e4m3fn_table():
    """value of every e4m3fn byte from its fields: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities,
    S.1111.111 is NaN."""
    vals = []
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 0xF, b & 7
        if e == 0xF and m == 7:
            v = float("nan")
        elif e == 0:
            v = (m / 8.0) * 2.0 ** (-6)
        else:
            v = (1 + m / 8.0) * 2.0 ** (e - 7)
        vals.append(-v if s else v)
    return torch.tensor(vals, dtype=torch.float64)


def test_fp8_storage_bytes_are_nearest_even_e4m3fn_over_every_bf16_input():
    table = _e4m3fn_table()
    assert table[0x7E].item() == 448.0 and torch.isnan(table[0x7F])
    # torch's dtype decodes the bytes the same way
    tb = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).to(torch.float64)
    assert torch.equal(torch.nan_to_num(tb, nan=-1.0), torch.nan_to_num(table, nan=-1.0))

    x = _all_bf16()
    x = x[torch.isfinite(x)]
    args = F.QArgs(num_bits=8, type="float", strategy="tensor")
    one = torch.ones(1, dtype=torch.bfloat16)
    zp = torch.zeros(1, dtype=torch.bfloat16)
    got = F.quantize(x, one, zp, args, dtype=torch.float8_e4m3fn).view(torch.uint8).to(torch.int64)
    # the reference expression of the storage cast (process.py / CT float-quantized: clamp, then cast)
    direct = torch.clamp(x, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8).to(torch.int64)
    # x + 0 (the zeros zero point) turns -0 into +0; nothing else may differ
    assert torch.equal(got[x != 0], direct[x != 0])
    assert (got[x == 0] == 0).all()

    # nearest, ties to the even mantissa, saturating at +-448, by brute force over the finite codes
    finite = ~torch.isnan(table)
    codes = torch.arange(256)[finite]
    tv = table[finite]
    xc = torch.clamp(x.double(), -448, 448)
    d = (xc.unsqueeze(-1) - tv).abs()
    dmin = d.min(dim=-1, keepdim=True).values
    tie = d == dmin
    even = (codes & 1) == 0
    # among the nearest codes prefer the even one; +0 over -0 for x == 0 (x + 0.0)
    score = tie.to(torch.int64) * 4 + (tie & even).to(torch.int64) * 2 + (tie & (codes < 128)).to(torch.int64)
    score = torch.where((xc == 0).unsqueeze(-1), score, tie.to(torch.int64) * 4 + (tie & even).to(torch.int64) * 2
                        + (tie & ((codes < 128) == (xc >= 0).unsqueeze(-1))).to(torch.int64))
    want = codes[score.argmax(dim=-1)]
    assert torch.equal(got, want)
    # truncation toward zero would differ on close to half of the inputs in e4m3's normal range: not a vacuous check
    trunc = codes[torch.where(tv.abs().unsqueeze(0) <= xc.abs().unsqueeze(-1), tv.abs().unsqueeze(0), -1.0)
                  .argmax(dim=-1)]
    normal = (xc.abs() >= 2.0 ** -6) & (xc.abs() < 448)
    assert (trunc != (want & 0x7F))[normal].float().mean() > 0.4


# ---- pack-quantized: int codes in int32 words ----------------------------------------------------------------------

def _decode_words(words, num_bits, cols):
    """independent decode from the published definition: ``pack_factor = 32 // num_bits`` codes per word, code j of
    a word in bits [j*num_bits, (j+1)*num_bits), stored with an offset of 2^(num_bits-1)."""
    pf = 32 // num_bits
    out = []
    for row in words.tolist():
        vals = []
        for wd in row:
            u = wd & 0xFFFFFFFF
            for j in range(pf):
                vals.append(((u >> (j * num_bits)) & ((1 << num_bits) - 1)) - (1 << (num_bits - 1)))
        out.append(vals[:cols])
    return torch.tensor(out, dtype=torch.int8)


@pytest.mark.parametrize("num_bits", [4, 8, 2])
def test_pack_to_int32_every_code_in_every_slot(num_bits):
    pf = 32 // num_bits
    lo, hi = -(1 << (num_bits - 1)), (1 << (num_bits - 1)) - 1
    n_codes = hi - lo + 1
    # row r: code (r mod n_codes) in slot (r div n_codes) of the first word, a second word of a fixed pattern, and a ragged tail
    rows = []
    for slot in range(pf):
        for c in range(lo, hi + 1):
            r = [lo] * pf
            r[slot] = c
            rows.append(r + [((slot + c + j) % n_codes) + lo for j in range(pf)] + [hi, lo, hi][: min(3, pf - 1)])
    codes = torch.tensor(rows, dtype=torch.int8)
    words = P.pack_to_int32(codes, num_bits)
    assert words.dtype == torch.int32 and words.shape == (len(rows), 3)
    assert torch.equal(_decode_words(words, num_bits, codes.shape[1]), codes)
    assert torch.equal(P.unpack_from_int32(words, num_bits, codes.shape), codes)
    # explicit words: slot j holds bits j*num_bits...; the highest slot lands in the sign bit of the int32
    r = [lo] * pf
    r[0] = hi
    w0 = P.pack_to_int32(torch.tensor([r], dtype=torch.int8), num_bits)[0, 0].item()
    assert w0 == (1 << num_bits) - 1
    r = [lo] * pf
    r[pf - 1] = hi
    w1 = P.pack_to_int32(torch.tensor([r], dtype=torch.int8), num_bits)[0, 0].item()
    assert (w1 & 0xFFFFFFFF) == ((1 << num_bits) - 1) << (32 - num_bits) and w1 < 0
    # a big-endian slot order is a different word for every asymmetric row: the decode above would catch it
    rev = P.pack_to_int32(codes.reshape(len(rows), -1)[:, :pf].flip(1), num_bits)[:, 0]
    assert (rev != words[:, 0]).any()


def test_pack_quantized_store_of_a_reference_held_matrix(golden):
    """the reference's int4 group golden (tests/llmcompressor/modifiers/calibration/test_lifecycle.py:78-98): its
    fake-quant values divided by the scales are the codes; the packed words must decode to exactly those."""
    case = golden["lifecycle_weight"]["cases"][2]
    args = F.QArgs(num_bits=4, strategy="group", group_size=3)
    w = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    qp = obs.get_qparams()
    st = P.compress_weight(w, qp["scale"], qp["zero_point"], args)
    codes = _decode_words(st["weight_packed"], 4, 6)
    deq = (codes.float().reshape(4, 2, 3) * qp["scale"].float().unsqueeze(-1)).reshape(4, 6).to(torch.bfloat16)
    assert torch.equal(deq, torch.tensor(case["quant"], dtype=torch.float32).to(torch.bfloat16))
    assert st["weight_shape"].tolist() == [4, 6]


# ---- BLOCK strategy inside the GPTQ column loop --------------------------------------------------------------------

def test_block_strategy_in_the_column_loop_reproduces_the_reference_block_golden(golden):
    """With a diagonal Hessian no error reaches another column, so ``quantize_weight`` must return the round-to-nearest
    result, and for block [2, 3] on arange(24) that result is held by the reference
    (test_lifecycle.py:78-98, last case).  A wrong scale row or column index in the BLOCK branch changes it."""
    case = golden["lifecycle_weight"]["cases"][4]
    assert case["args"]["strategy"] == "block"
    args = F.QArgs(num_bits=4, strategy="block", block_structure=[2, 3])
    w = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    want = torch.tensor(case["quant"], dtype=torch.float32).to(torch.bfloat16)
    for diag in (torch.ones(6), torch.tensor([3.0, 0.5, 7.0, 1.0, 2.0, 9.0])):
        obs = O.Observer("memoryless_minmax", "weight", args)
        obs(w)
        loss, out, info = G.quantize_weight(w, obs, args, torch.diag(diag).float(), blocksize=4)
        assert info["ok"]
        assert torch.equal(out["weight"], want), out["weight"]
        assert tuple(out["weight_scale"].shape) == (2, 2)
    # and with a dense Hessian the result still lies on each block's own grid (scale of its block row and column)
    torch.manual_seed(0)
    x = torch.randn(64, 6)
    obs = O.Observer("memoryless_minmax", "weight", args)
    obs(w)
    _, out, _ = G.quantize_weight(w, obs, args, (x.t() @ x).float(), blocksize=4)
    s = out["weight_scale"].float().repeat_interleave(2, 0).repeat_interleave(3, 1)
    q = out["weight"].float() / s
    # (the result is stored in bf16, so a code times its scale is off the grid by at most one bf16 rounding)
    assert ((q - q.round()).abs() <= q.abs() * 2.0 ** -8).all() and q.round().max() <= 7 and q.round().min() >= -8
