// Element-format arithmetic shared by the observer, quantise/pack, MSE-search and GPTQ kernels.
//
// The reference evaluates these formulas as chains of eager tensor ops, so every
// intermediate is rounded to the tensor's dtype.  Each function below takes the
// dtype of each intermediate explicitly (LLMC_BF16 / LLMC_F16 / LLMC_F32) and
// rounds at exactly those points, computing in fp32 in between (which is what
// the eager kernels do for 16-bit types).
#pragma once
#include "common.h"

__device__ __forceinline__ float round_rt(float f, int dt) {
  if (dt == LLMC_BF16) return round_bf16(f);
  if (dt == LLMC_F16) return (float)(_Float16)f;
  return f;
}

__device__ __forceinline__ float load_rt(const void* p, int64_t i, int dt) {
  if (dt == LLMC_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  if (dt == LLMC_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

__device__ __forceinline__ void store_rt(void* p, int64_t i, float f, int dt) {
  if (dt == LLMC_BF16)
    ((uint16_t*)p)[i] = f32_to_bf16_bits(f);
  else if (dt == LLMC_F16)
    ((uint16_t*)p)[i] = f32_to_f16_bits(f);
  else
    ((float*)p)[i] = f;
}

__device__ __forceinline__ float dtype_eps(int dt) {
  return dt == LLMC_BF16 ? 0.0078125f : dt == LLMC_F16 ? 0.0009765625f : 1.1920928955078125e-07f;
}

// ---- float8 e4m3fn (max 448, no inf), round-to-nearest-even; |x| <= 448 on entry
__device__ __forceinline__ float e4m3_round(float x) {
  const float a = fabsf(x);
  float r;
  if (a >= 0.015625f) {  // normal range: keep 3 mantissa bits
    uint32_t u = __float_as_uint(a);
    u += 0x7ffffu + ((u >> 20) & 1u);
    u &= 0xfff00000u;
    r = __uint_as_float(u);
  } else {  // subnormal: multiples of 2^-9
    r = rintf(a * 512.0f) * 0.001953125f;
  }
  return copysignf(r, x);
}

// byte encoding of a value already on the e4m3 grid
__device__ __forceinline__ uint8_t e4m3_encode(float v) {
  const uint32_t u = __float_as_uint(v);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  const float a = fabsf(v);
  if (a == 0.f) return sign;
  if (a < 0.015625f) return sign | (uint8_t)(a * 512.0f);
  const uint32_t e = ((u >> 23) & 0xffu) - 127u + 7u;
  return sign | (uint8_t)((e << 3) | ((u >> 20) & 7u));
}

__device__ __forceinline__ float e4m3_decode(uint8_t b) {
  const uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
  float a = e == 0 ? (float)m * 0.001953125f : __uint_as_float(((e - 7u + 127u) << 23) | (m << 20));
  return (b & 0x80u) ? -a : a;
}

// ---- float4 e2m1 grid {0,.5,1,1.5,2,3,4,6}; ties to the even mantissa; |x| <= 6 on entry.
// Returns the magnitude; the sign is the sign of x when x != 0 (a negative value that
// rounds to zero keeps its sign bit, -0.0 itself does not).
__device__ __forceinline__ float e2m1_round_abs(float a) {
  float r = 6.0f;
  r = a <= 5.0f ? 4.0f : r;
  r = a < 3.5f ? 3.0f : r;
  r = a <= 2.5f ? 2.0f : r;
  r = a < 1.75f ? 1.5f : r;
  r = a <= 1.25f ? 1.0f : r;
  r = a < 0.75f ? 0.5f : r;
  r = a <= 0.25f ? 0.0f : r;
  return r;
}
__device__ __forceinline__ uint8_t e2m1_index(float mag) {
  // 0,.5,1,1.5 -> 0..3 ; 2,3 -> 4,5 ; 4 -> 6 ; 6 -> 7
  return mag < 2.0f ? (uint8_t)(mag * 2.0f) : mag < 4.0f ? (uint8_t)(mag + 2.0f) : mag == 4.0f ? 6 : 7;
}

// ---- gfx950 conversion instructions.  v_cvt_pk_fp8_f32 rounds to OCP e4m3fn (nearest even) and
// v_cvt_scalef32_pk_fp4_f32 to e2m1 (ties to the even mantissa); on inputs already clamped to the
// format's range both give the same bytes as e4m3_encode(e4m3_round(v)) and the e2m1_index /
// sign-bit-3 nibble above, including the sign bit of a negative value that rounds to zero.
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two e4m3 bytes: a in bits 7:0, b in bits 15:8
__device__ __forceinline__ uint32_t hw_e4m3_pair(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ f32x2_t hw_e4m3_pair_decode(uint32_t w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
}
// two e2m1 nibbles in one byte: a in bits 3:0, b in bits 7:4
__device__ __forceinline__ uint32_t hw_e2m1_pair(float a, float b) {
  return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, a, b, 1.0f, 0) & 0xffu;
}
__device__ __forceinline__ f32x2_t hw_e2m1_pair_decode(uint32_t byte) {
  return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(byte, 1.0f, 0);
}

// two fp32 values rounded (nearest even) to the 16-bit type DT, packed lo | hi << 16; bf16 goes
// through the packed conversion instruction
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <int DT>
__device__ __forceinline__ uint32_t pack16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  uint32_t w;
  if (DT == LLMC_BF16) {
    const bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
    __builtin_memcpy(&w, &b, 4);
  } else {
    const f16x2_t h = __builtin_convertvector(v, f16x2_t);
    __builtin_memcpy(&w, &h, 4);
  }
  return w;
}
template <int DT>
__device__ __forceinline__ float round16_finite(float f) {
  if (DT == LLMC_BF16) return (float)(__bf16)f;
  return (float)(_Float16)f;
}

// ---- division by a value shared by many elements.  The steps are those of the correctly
// rounded fp32 division sequence (reciprocal with one Newton step, quotient with two residual
// corrections) with the divisor's part hoisted; they give the IEEE quotient whenever nothing
// under- or overflows on the way, which `ok` and fastdiv_trusted() bound from the divisor's and
// the quotient's magnitudes.  Callers redo the division with `/` when the bound fails.
struct FastDiv {
  float s, y;
  bool ok;
};
__device__ __forceinline__ FastDiv make_fastdiv(float s) {
  FastDiv d;
  d.s = s;
  const float y0 = __builtin_amdgcn_rcpf(s);
  const float e = fmaf(-s, y0, 1.0f);
  d.y = fmaf(e, y0, y0);
  const float a = fabsf(s);
  d.ok = a > 0x1p-60f && a < 0x1p60f;
  return d;
}
__device__ __forceinline__ float fastdiv(float x, const FastDiv& d) {
  float q = x * d.y;
  float r = fmaf(-d.s, q, x);
  q = fmaf(r, d.y, q);
  r = fmaf(-d.s, q, x);
  return fmaf(r, d.y, q);
}
// quotient magnitudes for which fastdiv() is exact given d.ok: below 2^100 nothing overflowed
// (NaN fails the test too); from 2^-40 up the residuals stayed normal.  An exact zero quotient
// of a zero dividend is exact as well.
__device__ __forceinline__ bool fastdiv_big_ok(float q) { return fabsf(q) < 0x1p100f; }
__device__ __forceinline__ bool fastdiv_small(float q) { return fabsf(q) < 0x1p-40f; }

// ---- bf16 / bf16 quotient rounded to bf16, with one multiply.  For x and s both bf16 (8-bit
// significands X, S in [128, 255]) the exact quotient X/S is never a rounding midpoint of bf16 (a midpoint
// has a 9-bit odd significand M, and M*S' = X*2^k has no solution with M >= 257 > X), and it lies at
// least 2^-16 (relative) away from the nearest one: |256 X - M S| >= 1 over 256 S.  x * y with y the
// reciprocal of make_fastdiv() is within 2^-22 of the quotient, so bf16(x * y) == bf16(x / s) whenever the
// quotient is a normal bf16 number and nothing overflows.  bf16_inputs_plain() bounds that from the inputs:
// every nonzero |x| lies in [2^-96, 2^96) (which also excludes inf and NaN), and bf16_scale_plain() asks
// |s| in (2^-30, 2^30), so |x / s| lies in (2^-126, 2^126).  A zero dividend gives an exact zero.
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
struct Bf16Range {
  u16x2_t mx, mn;
};
__device__ __forceinline__ Bf16Range bf16_range_init() {
  Bf16Range r;
  r.mx = (u16x2_t){0, 0};
  r.mn = (u16x2_t){0xffff, 0xffff};
  return r;
}
// fold the two bf16 values of one 32-bit word into the running magnitude range (zeros do not lower it)
__device__ __forceinline__ void bf16_range_add(Bf16Range& r, uint32_t w) {
  const uint32_t a = w & 0x7fff7fffu;
  u16x2_t m;
  __builtin_memcpy(&m, &a, 4);
  r.mx = __builtin_elementwise_max(r.mx, m);
  r.mn = __builtin_elementwise_min(r.mn, (u16x2_t)(m - (u16x2_t){1, 1}));
}
__device__ __forceinline__ bool bf16_inputs_plain(const Bf16Range& r) {
  constexpr uint32_t LO = (127u - 96u) << 7, HI = (127u + 96u) << 7;  // bit patterns of 2^-96 and 2^96
  const uint32_t mx = max((uint32_t)r.mx.x, (uint32_t)r.mx.y), mn = min((uint32_t)r.mn.x, (uint32_t)r.mn.y);
  return mx < HI && mn >= LO - 1u;
}
__device__ __forceinline__ bool bf16_scale_plain(float s) {
  const float a = fabsf(s);
  return a > 0x1p-30f && a < 0x1p30f;
}

struct QFormat {
  int fmt;   // LLMC_FMT_*
  float qmin, qmax;
};

__host__ __device__ __forceinline__ QFormat make_qformat(int fmt, int bits) {
  QFormat f;
  f.fmt = fmt;
  if (fmt == LLMC_FMT_INT) {
    const float half = (float)(1 << (bits - 1));
    f.qmin = -half;
    f.qmax = half - 1.0f;
  } else if (fmt == LLMC_FMT_FP8) {
    f.qmin = -448.0f;
    f.qmax = 448.0f;
  } else {
    f.qmin = -6.0f;
    f.qmax = 6.0f;
  }
  return f;
}

// clamp + round onto the element grid; result is the (signed) grid value
__device__ __forceinline__ float round_to_grid(float v, const QFormat& f) {
  v = fminf(fmaxf(v, f.qmin), f.qmax);
  if (f.fmt == LLMC_FMT_INT) return rintf(v);
  if (f.fmt == LLMC_FMT_FP8) return e4m3_round(v);
  const float m = e2m1_round_abs(fabsf(v));
  return v < 0.f ? -m : m;  // -0.0f when a negative value rounds to zero
}

// quantise one value: x (dtype xd) / scale -> (+zp) -> grid.  pd = dtype of the quotient
// (promotion of x's and the scale's dtypes).
__device__ __forceinline__ float quantize_value(float x, float s, float zp, bool has_zp, int pd,
                                               const QFormat& f) {
  float v = round_rt(x / s, pd);
  // the reference always adds a zero-point tensor (zeros when symmetric), which turns a
  // -0.0 quotient into +0.0; x + 0.0f is not foldable under IEEE semantics
  v = has_zp ? round_rt(v + zp, pd) : v + 0.0f;
  return round_to_grid(v, f);
}

// dequantise a grid value in the scale's dtype sd
__device__ __forceinline__ float dequantize_value(float q, float s, float zp, bool has_zp, int sd) {
  float d = q;
  if (has_zp) d = round_rt(d - zp, sd);
  return round_rt(d * s, sd);
}

// scale (and zero point) from an observed min/max pair, statistics in dtype sd.
//   symmetric : scale = absmax / (range/2);  asymmetric: scale = (max-min)/range,
//   zp = clamp(qmin - min/scale) rounded to an integer (int8 storage).
// scale_mode NVFP4: scale = e4m3(global_scale * scale) as fp32; MXFP4: 2^(e-127), *e_out = e.
__device__ __forceinline__ void qparams_from_minmax(float mn, float mx, int sd, const QFormat& f,
                                                    bool symmetric, int scale_mode, float gscale,
                                                    float* scale_out, float* zp_out, int* e_out) {
  mn = fminf(mn, 0.f);
  mx = fmaxf(mx, 0.f);
  const float range = f.qmax - f.qmin;
  float s, zp = 0.f;
  *e_out = 0;
  if (symmetric) {
    const float amax = fmaxf(fabsf(mn), fabsf(mx));
    if (scale_mode == LLMC_SCALE_MXFP4) {
      // power-of-two scale from the bf16 bit pattern of absmax: bump by half an e2m1
      // mantissa step, drop the mantissa, exponent - 2 (emax of e2m1), biased by 127
      const uint32_t bits = (uint32_t)f32_to_bf16_bits(amax);
      const uint32_t p2 = (bits + 32u) & 0xff80u;
      const float p2f = bf16_bits_to_f32((uint16_t)p2);
      float e = 127.0f + floorf(log2f(p2f)) - 2.0f;  // p2f is an exact power of two (or 0 -> -inf)
      e = fminf(fmaxf(e, 0.f), 255.f);
      *e_out = (int)e;
      s = round_rt(exp2f(e - 127.0f), sd);
    } else {
      s = round_rt(amax / (range * 0.5f), sd);
    }
  } else {
    s = round_rt(round_rt(mx - mn, sd) / range, sd);
    zp = round_rt(f.qmin - round_rt(mn / s, sd), sd);
    // an all-zero group has scale 0 -> min/scale = NaN, which the reference's clamp keeps and
    // its integer cast turns into 0
    zp = (zp != zp) ? 0.f : fminf(fmaxf(zp, f.qmin), f.qmax);
    zp = rintf(fminf(fmaxf(zp, -128.f), 127.f));
  }
  float eps = dtype_eps(sd);
  if (scale_mode == LLMC_SCALE_NVFP4) {
    s = gscale * s;  // fp32 [1] tensor times 16-bit tensor promotes to fp32
    s = e4m3_round(fminf(fmaxf(s, -448.f), 448.f));
    eps = 0.125f;
  }
  if (s == 0.f) s = eps;
  *scale_out = s;
  *zp_out = zp;
}
