// Quantise / fake-quantise / pack kernels (bandwidth-bound: one pass, 16-byte coalesced loads).
//
// One thread owns 8 consecutive columns of a row: it loads them with one
// 16-byte access (16-bit inputs), looks the scale up once when the 8 columns
// share a group, and emits either the dequantised values, one byte per code,
// or the packed storage word (eight int4 fields in one int32, two int8 words,
// eight e4m3 bytes, or four bytes of e2m1 nibble pairs).
#include "qformat.h"

namespace {

struct QuantParams {
  const void* x;
  int x_dt;
  int64_t R, K, ldx;
  const void* scale;
  int scale_dt;
  const int8_t* zp;
  const int32_t* g_idx;
  const float* gscale;
  int fmt, bits;
  int64_t rdiv, srow, cdiv;  // scale index = (r / rdiv) * srow + (g_idx ? g_idx[c] : c / cdiv)
  int pd;                    // dtype of the quotient x / scale
  int sd;                    // dtype the dequantised value is formed in
  int out_mode;
  void* out;
  int out_dt;
  int64_t ldo;  // leading dimension of `out` in its own elements
};

__device__ __forceinline__ uint32_t code_bits(float q, const QFormat& f, int bits) {
  if (f.fmt == LLMC_FMT_INT) return (uint32_t)((int)q + (1 << (bits - 1))) & ((1u << bits) - 1u);
  if (f.fmt == LLMC_FMT_FP8) return e4m3_encode(q);
  return (uint32_t)e2m1_index(fabsf(q)) | (signbit(q) ? 8u : 0u);
}

template <bool VEC>
__global__ __launch_bounds__(256) void quantize_kernel(QuantParams p) {
  const int64_t per_row = (p.K + 7) / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= p.R * per_row) return;
  const int64_t r = gid / per_row;
  const int64_t c0 = (gid % per_row) * 8;
  const QFormat f = make_qformat(p.fmt, p.bits);
  const float gs = p.gscale ? p.gscale[0] : 1.f;

  float xv[8];
  if (VEC && p.x_dt != LLMC_F32) {
    const uint4 v = *(const uint4*)((const uint16_t*)p.x + r * p.ldx + c0);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (p.x_dt == LLMC_BF16) {
        xv[2 * j] = __uint_as_float(w[j] << 16);
        xv[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      } else {
        xv[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
        xv[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) xv[j] = (c0 + j < p.K) ? load_rt(p.x, r * p.ldx + c0 + j, p.x_dt) : 0.f;
  }

  const int64_t srow_off = (r / p.rdiv) * p.srow;
  float s = 1.f, zp = 0.f;
  const bool has_zp = p.zp != nullptr;
  auto fetch = [&](int64_t c) {
    const int64_t si = srow_off + (p.g_idx ? (int64_t)p.g_idx[c] : c / p.cdiv);
    s = load_rt(p.scale, si, p.scale_dt);
    if (p.gscale) s = s / gs;  // stored scale (as fp32) / global_scale
    if (has_zp) zp = (float)p.zp[si];
  };
  if (VEC) fetch(c0);

  float qv[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if (!VEC) {
      if (c0 + j >= p.K) {
        qv[j] = 0.f;
        continue;
      }
      fetch(c0 + j);
    }
    qv[j] = quantize_value(xv[j], s, zp, has_zp, p.pd, f);
    if (p.out_mode == LLMC_OUT_FAKEQUANT) qv[j] = dequantize_value(qv[j], s, zp, has_zp, p.sd);
  }

  if (p.out_mode == LLMC_OUT_FAKEQUANT) {
    if (VEC && p.out_dt != LLMC_F32) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = p.out_dt == LLMC_BF16 ? f32_to_bf16_bits(qv[2 * j]) : f32_to_f16_bits(qv[2 * j]);
        const uint32_t hi = p.out_dt == LLMC_BF16 ? f32_to_bf16_bits(qv[2 * j + 1]) : f32_to_f16_bits(qv[2 * j + 1]);
        w[j] = lo | (hi << 16);
      }
      *(uint4*)((uint16_t*)p.out + r * p.ldo + c0) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (c0 + j < p.K) store_rt(p.out, r * p.ldo + c0 + j, qv[j], p.out_dt);
    }
    return;
  }

  uint32_t cb[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) cb[j] = (c0 + j < p.K) ? code_bits(qv[j], f, p.bits) : 0u;

  if (p.out_mode == LLMC_OUT_CODES) {
    // one byte per element: int8 code, e4m3 byte, or e2m1 nibble (sign in bit 3)
    uint8_t* o = (uint8_t*)p.out + r * p.ldo + c0;
    if (VEC) {
      uint32_t w0 = 0, w1 = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t b0 = f.fmt == LLMC_FMT_INT ? (uint32_t)(uint8_t)(int8_t)(int)qv[j] : cb[j];
        const uint32_t b1 = f.fmt == LLMC_FMT_INT ? (uint32_t)(uint8_t)(int8_t)(int)qv[j + 4] : cb[j + 4];
        w0 |= b0 << (8 * j);
        w1 |= b1 << (8 * j);
      }
      *(uint2*)o = make_uint2(w0, w1);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (c0 + j < p.K) o[j] = f.fmt == LLMC_FMT_INT ? (uint8_t)(int8_t)(int)qv[j] : (uint8_t)cb[j];
    }
    return;
  }

  // LLMC_OUT_PACKED
  if (f.fmt == LLMC_FMT_FP4) {
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) w |= cb[j] << (4 * j);  // even column in the low nibble of each byte
    uint8_t* o = (uint8_t*)p.out + r * p.ldo + c0 / 2;
    if (VEC) {
      *(uint32_t*)o = w;
    } else {
      for (int j = 0; j < 4; ++j)
        if (c0 + 2 * j < p.K) o[j] = (uint8_t)(w >> (8 * j));
    }
  } else if (f.fmt == LLMC_FMT_FP8) {
    uint8_t* o = (uint8_t*)p.out + r * p.ldo + c0;
    for (int j = 0; j < 8; ++j)
      if (c0 + j < p.K) o[j] = (uint8_t)cb[j];
  } else {
    // offset-binary fields, element j of a word at bit j*bits, 32/bits elements per int32 word
    const int pf = 32 / p.bits;
    uint32_t* o = (uint32_t*)p.out + r * p.ldo;
    if (pf == 8) {
      uint32_t w = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) w |= cb[j] << (4 * j);
      o[c0 / 8] = w;
    } else if (pf == 4) {
      uint32_t w0 = 0, w1 = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        w0 |= cb[j] << (8 * j);
        w1 |= cb[j + 4] << (8 * j);
      }
      o[c0 / 4] = w0;
      if (c0 + 4 < p.K) o[c0 / 4 + 1] = w1;
    } else {
      // other widths (pf = 16, 10, 6, 5): a word may straddle this thread's 8 columns
      for (int j = 0; j < 8; ++j)
        if (c0 + j < p.K) atomicOr(&o[(c0 + j) / pf], cb[j] << (((c0 + j) % pf) * p.bits));
    }
  }
}

// ---- the common case: 16-bit input with K % 8 == 0, scales in the input's dtype or fp32,
// power-of-two (or whole-row) column groups, no g_idx, 4/8-bit ints, e4m3 or e2m1.
// One workgroup walks one row in 16-byte chunks with 32-bit index arithmetic; everything the
// format decides is a template parameter so the per-element path is branch-free: shared-divisor
// division, rounding to the quotient's dtype, clamp, and the hardware e4m3/e2m1 conversions.
template <int XDT>
__device__ __forceinline__ void unpack8(const uint4& v, float* x) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (XDT == LLMC_BF16) {
      x[2 * j] = __uint_as_float(w[j] << 16);
      x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    } else {
      x[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
      x[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
    }
  }
}

// SM: 0 = scales in the input's 16-bit dtype, 1 = fp32 scales, 2 = stored scale / global scale (fp32)
// A lane handles 16 consecutive columns (two 16-byte loads), which share one scale.
template <int XDT, int SM, int FMT, bool HAS_ZP, int OUT>
__global__ __launch_bounds__(256) void quantize_rows_kernel(QuantParams p, int cshift) {
  constexpr bool S32 = SM != 0;
  constexpr int PD = S32 ? LLMC_F32 : XDT;  // dtype of the quotient and of the dequantised value
  constexpr int E = 16;
  const int64_t r = blockIdx.x;
  const int upr = (int)(p.K >> 4);
  const uint16_t* xr = (const uint16_t*)p.x + r * p.ldx;
  const int64_t srow_off = (p.rdiv == 1 ? r : r / p.rdiv) * p.srow;
  const QFormat f = make_qformat(FMT, p.bits);
  float gs = 1.f;
  if (SM == 2) gs = p.gscale[0];

  for (int u = threadIdx.x; u < upr; u += 256) {
    const uint4 raw0 = *(const uint4*)(xr + (u << 4));
    const uint4 raw1 = *(const uint4*)(xr + (u << 4) + 8);
    const int64_t si = srow_off + ((u << 4) >> cshift);
    float s;
    if (SM == 0)
      s = load_as_f32<XDT>(p.scale, si);
    else if (SM == 1)
      s = ((const float*)p.scale)[si];
    else
      s = load_rt(p.scale, si, p.scale_dt) / gs;
    const float zp = HAS_ZP ? (float)p.zp[si] : 0.f;
    float x[E], v[E];
    unpack8<XDT>(raw0, x);
    unpack8<XDT>(raw1, x + 8);
    const FastDiv d = make_fastdiv(s);
    bool redo;
    if (XDT == LLMC_BF16 && SM == 0) {
      // bf16 values over a bf16 scale: the rounded quotient is one multiply away (see qformat.h)
      Bf16Range rg = bf16_range_init();
      bf16_range_add(rg, raw0.x); bf16_range_add(rg, raw0.y); bf16_range_add(rg, raw0.z); bf16_range_add(rg, raw0.w);
      bf16_range_add(rg, raw1.x); bf16_range_add(rg, raw1.y); bf16_range_add(rg, raw1.z); bf16_range_add(rg, raw1.w);
      redo = !(bf16_inputs_plain(rg) & bf16_scale_plain(s));
#pragma unroll
      for (int j = 0; j < E; ++j) v[j] = x[j] * d.y;
    } else {
      bool big = false, small = false;
#pragma unroll
      for (int j = 0; j < E; ++j) {
        v[j] = fastdiv(x[j], d);
        big = big | !fastdiv_big_ok(v[j]);
        small = small | fastdiv_small(v[j]);
      }
      redo = big | !d.ok;
      if (small) {
#pragma unroll
        for (int j = 0; j < E; ++j) redo = redo | (fastdiv_small(v[j]) & (x[j] != 0.f));
      }
    }
    if (redo) {
      // out-of-range divisor or quotient, NaN: the plain division, then the same tail
#pragma unroll
      for (int j = 0; j < E; ++j) {
        v[j] = round_rt(x[j] / s, PD);
        v[j] = HAS_ZP ? round_rt(v[j] + zp, PD) : v[j] + 0.0f;
        v[j] = fminf(fmaxf(v[j], f.qmin), f.qmax);
      }
    } else {
#pragma unroll
      for (int j = 0; j < E; ++j) {
        if (!S32) v[j] = round16_finite<XDT>(v[j]);
        if (HAS_ZP)
          v[j] = S32 ? v[j] + zp : round16_finite<XDT>(v[j] + zp);
        else if (FMT != LLMC_FMT_INT || OUT == LLMC_OUT_FAKEQUANT)
          v[j] = v[j] + 0.0f;  // the reference adds a zero zero-point: -0.0 becomes +0.0
        v[j] = __builtin_amdgcn_fmed3f(v[j], f.qmin, f.qmax);
      }
    }

    // element codes: e4m3 bytes / e2m1 nibbles via the conversion instructions
    uint32_t fp8w[4] = {0u, 0u, 0u, 0u}, fp4w[2] = {0u, 0u};
    if (FMT == LLMC_FMT_FP8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) fp8w[j >> 1] |= hw_e4m3_pair(v[2 * j], v[2 * j + 1]) << (16 * (j & 1));
    } else if (FMT == LLMC_FMT_FP4) {
#pragma unroll
      for (int j = 0; j < 8; ++j) fp4w[j >> 2] |= hw_e2m1_pair(v[2 * j], v[2 * j + 1]) << (8 * (j & 3));
    }

    if (OUT == LLMC_OUT_FAKEQUANT) {
      if (FMT == LLMC_FMT_INT) {
#pragma unroll
        for (int j = 0; j < E; ++j) v[j] = rintf(v[j]);
      } else if (FMT == LLMC_FMT_FP8) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const f32x2_t t = hw_e4m3_pair_decode(fp8w[j >> 1] >> (16 * (j & 1)));
          v[2 * j] = t.x;
          v[2 * j + 1] = t.y;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const f32x2_t t = hw_e2m1_pair_decode(fp4w[j >> 2] >> (8 * (j & 3)));
          v[2 * j] = t.x;
          v[2 * j + 1] = t.y;
        }
      }
#pragma unroll
      for (int j = 0; j < E; ++j) {
        if (HAS_ZP) v[j] = round_rt(v[j] - zp, PD);
        v[j] *= s;  // rounding to PD, then to the output's dtype, is one rounding
      }
      uint16_t* o = (uint16_t*)p.out + r * p.ldo + (u << 4);
      *(uint4*)o = make_uint4(pack16<XDT>(v[0], v[1]), pack16<XDT>(v[2], v[3]), pack16<XDT>(v[4], v[5]),
                              pack16<XDT>(v[6], v[7]));
      *(uint4*)(o + 8) = make_uint4(pack16<XDT>(v[8], v[9]), pack16<XDT>(v[10], v[11]),
                                    pack16<XDT>(v[12], v[13]), pack16<XDT>(v[14], v[15]));
      continue;
    }

    if (FMT == LLMC_FMT_FP8) {  // bytes either way
      *(uint4*)((uint8_t*)p.out + r * p.ldo + (u << 4)) = make_uint4(fp8w[0], fp8w[1], fp8w[2], fp8w[3]);
    } else if (FMT == LLMC_FMT_FP4) {
      if (OUT == LLMC_OUT_PACKED) {
        *(uint2*)((uint8_t*)p.out + r * p.ldo + (u << 3)) = make_uint2(fp4w[0], fp4w[1]);
      } else {  // one nibble per byte
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint32_t h = (fp4w[k >> 1] >> (16 * (k & 1))) & 0xffffu;
          w[k] = (h & 0xfu) | ((h & 0xf0u) << 4) | ((h & 0xf00u) << 8) | ((h & 0xf000u) << 12);
        }
        *(uint4*)((uint8_t*)p.out + r * p.ldo + (u << 4)) = make_uint4(w[0], w[1], w[2], w[3]);
      }
    } else {
      // v + 1.5*2^23 rounds v to the nearest-even integer and leaves it, two's complement, in the
      // low mantissa bits; funnel shifts collect the low 4 or 8 bits of each element
      uint32_t q[E];
#pragma unroll
      for (int j = 0; j < E; ++j) q[j] = __float_as_uint(v[j] + 12582912.0f);
      if (OUT == LLMC_OUT_CODES || p.bits == 8) {
        // int8 codes, or int8 fields (offset binary) four to a word: the same byte positions
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < E; ++j) w[j >> 2] = __builtin_amdgcn_alignbit(q[j], w[j >> 2], 8);
        if (OUT == LLMC_OUT_CODES) {
          *(uint4*)((uint8_t*)p.out + r * p.ldo + (u << 4)) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
          const uint32_t m = 0x80808080u;
          *(uint4*)((uint32_t*)p.out + r * p.ldo + (u << 2)) = make_uint4(w[0] ^ m, w[1] ^ m, w[2] ^ m, w[3] ^ m);
        }
      } else {  // sixteen 4-bit fields, offset binary
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < E; ++j) w[j >> 3] = __builtin_amdgcn_alignbit(q[j], w[j >> 3], 4);
        *(uint2*)((uint32_t*)p.out + r * p.ldo + (u << 1)) = make_uint2(w[0] ^ 0x88888888u, w[1] ^ 0x88888888u);
      }
    }
  }
}

template <int XDT, int SM, int FMT, bool HAS_ZP>
void launch_rows_out(const QuantParams& p, int cshift, hipStream_t st) {
  const dim3 grid((unsigned)p.R), block(256);
  if (p.out_mode == LLMC_OUT_FAKEQUANT)
    hipLaunchKernelGGL((quantize_rows_kernel<XDT, SM, FMT, HAS_ZP, LLMC_OUT_FAKEQUANT>), grid, block, 0, st, p, cshift);
  else if (p.out_mode == LLMC_OUT_CODES)
    hipLaunchKernelGGL((quantize_rows_kernel<XDT, SM, FMT, HAS_ZP, LLMC_OUT_CODES>), grid, block, 0, st, p, cshift);
  else
    hipLaunchKernelGGL((quantize_rows_kernel<XDT, SM, FMT, HAS_ZP, LLMC_OUT_PACKED>), grid, block, 0, st, p, cshift);
}

template <int XDT, int SM>
void launch_rows_fmt(const QuantParams& p, int cshift, hipStream_t st) {
  if (p.fmt == LLMC_FMT_INT) {
    if (p.zp)
      launch_rows_out<XDT, SM, LLMC_FMT_INT, true>(p, cshift, st);
    else
      launch_rows_out<XDT, SM, LLMC_FMT_INT, false>(p, cshift, st);
  } else if (p.fmt == LLMC_FMT_FP8) {
    launch_rows_out<XDT, SM, LLMC_FMT_FP8, false>(p, cshift, st);
  } else {
    launch_rows_out<XDT, SM, LLMC_FMT_FP4, false>(p, cshift, st);
  }
}

// launches the row kernel when the call fits its assumptions; false = use the general kernel
bool try_launch_rows(const QuantParams& p, hipStream_t st) {
  if (p.x_dt == LLMC_F32 || p.g_idx || p.K % 16 || p.ldx % 8 || ((uintptr_t)p.x & 15)) return false;
  if (p.R > 0x7fffffffLL || p.K > (1LL << 30)) return false;
  const int eff = p.gscale ? LLMC_F32 : p.scale_dt;
  if (eff != LLMC_F32 && eff != p.x_dt) return false;
  if (p.zp && p.fmt != LLMC_FMT_INT) return false;
  if (p.fmt == LLMC_FMT_INT && p.bits != 4 && p.bits != 8) return false;
  int cshift;
  if (p.cdiv >= p.K) {
    cshift = 31;
  } else {
    if (p.cdiv < 16 || (p.cdiv & (p.cdiv - 1))) return false;
    cshift = 0;
    while ((1LL << cshift) < p.cdiv) ++cshift;
  }
  if (p.out_mode == LLMC_OUT_FAKEQUANT) {
    if (p.out_dt != p.x_dt || p.ldo % 8 || ((uintptr_t)p.out & 15)) return false;
  } else if (p.out_mode == LLMC_OUT_CODES || p.fmt == LLMC_FMT_FP8) {
    if (p.ldo % 16 || ((uintptr_t)p.out & 15)) return false;  // 16 bytes per lane
  } else if (p.fmt == LLMC_FMT_FP4) {
    if (p.ldo % 8 || ((uintptr_t)p.out & 7)) return false;  // 8 bytes per lane
  } else if (p.bits == 8) {
    if (p.ldo % 4 || ((uintptr_t)p.out & 15)) return false;  // four int32 words per lane
  } else {
    if (p.ldo % 2 || ((uintptr_t)p.out & 7)) return false;  // two int32 words per lane
  }
  const int sm = p.gscale ? 2 : (eff == LLMC_F32 ? 1 : 0);
  if (p.x_dt == LLMC_BF16) {
    if (sm == 0) launch_rows_fmt<LLMC_BF16, 0>(p, cshift, st);
    else if (sm == 1) launch_rows_fmt<LLMC_BF16, 1>(p, cshift, st);
    else launch_rows_fmt<LLMC_BF16, 2>(p, cshift, st);
  } else {
    if (sm == 0) launch_rows_fmt<LLMC_F16, 0>(p, cshift, st);
    else if (sm == 1) launch_rows_fmt<LLMC_F16, 1>(p, cshift, st);
    else launch_rows_fmt<LLMC_F16, 2>(p, cshift, st);
  }
  return true;
}

// Per-token dynamic quantisation: one workgroup per row.  The row is staged in LDS while
// its absmax is reduced, so HBM sees one read and one write per element.
template <int DT>
__global__ __launch_bounds__(256) void dynamic_token_kernel(const void* __restrict__ x, int64_t ldx, int K,
                                                            int fmt, int bits, int out_mode,
                                                            void* __restrict__ out, int64_t ldo,
                                                            void* __restrict__ scale_out) {
  extern __shared__ __attribute__((aligned(16))) uint16_t row[];
  __shared__ float wred[4];
  const int64_t r = blockIdx.x;
  const uint16_t* xr = (const uint16_t*)x + r * ldx;
  const bool vec = (K % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)x & 15) == 0);
  float amax = 0.f;
  if (vec) {
    for (int c = threadIdx.x * 8; c < K; c += 256 * 8) {
      const uint4 v = *(const uint4*)(xr + c);
      *(uint4*)(row + c) = v;
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float lo = load_as_f32<DT>(&w[j], 0), hi = load_as_f32<DT>(&w[j], 1);
        amax = fmaxf(amax, fmaxf(fabsf(lo), fabsf(hi)));
      }
    }
  } else {
    for (int c = threadIdx.x; c < K; c += 256) {
      row[c] = xr[c];
      amax = fmaxf(amax, fabsf(load_as_f32<DT>(xr, c)));
    }
  }
  amax = wave_max(amax);
  if ((threadIdx.x & 63) == 0) wred[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wred[0], wred[1]), fmaxf(wred[2], wred[3]));
  const QFormat f = make_qformat(fmt, bits);
  float s = round_to<DT>(amax / ((f.qmax - f.qmin) * 0.5f));
  if (s == 0.f) s = dtype_eps(DT);
  if (threadIdx.x == 0) store_from_f32<DT>(scale_out, r, s);
  for (int c = threadIdx.x * 8; c < K; c += 256 * 8) {
    float q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float xv = (c + j < K) ? load_as_f32<DT>(row, c + j) : 0.f;
      q[j] = quantize_value(xv, s, 0.f, false, DT, f);
    }
    if (out_mode == LLMC_OUT_FAKEQUANT) {
      uint16_t o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float d = dequantize_value(q[j], s, 0.f, false, DT);
        o[j] = DT == LLMC_BF16 ? f32_to_bf16_bits(d) : f32_to_f16_bits(d);
      }
      uint16_t* orow = (uint16_t*)out + r * ldo;
      if (vec && (ldo % 8 == 0) && (((uintptr_t)out & 15) == 0)) {
        *(uint4*)(orow + c) = make_uint4(o[0] | ((uint32_t)o[1] << 16), o[2] | ((uint32_t)o[3] << 16),
                                         o[4] | ((uint32_t)o[5] << 16), o[6] | ((uint32_t)o[7] << 16));
      } else {
        for (int j = 0; j < 8; ++j)
          if (c + j < K) orow[c + j] = o[j];
      }
    } else {
      uint8_t* orow = (uint8_t*)out + r * ldo;
      uint32_t w0 = 0, w1 = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        w0 |= code_bits(q[j], f, bits) << (8 * j);
        w1 |= code_bits(q[j + 4], f, bits) << (8 * j);
      }
      if (f.fmt == LLMC_FMT_INT) {
        w0 = w1 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w0 |= (uint32_t)(uint8_t)(int8_t)(int)q[j] << (8 * j);
          w1 |= (uint32_t)(uint8_t)(int8_t)(int)q[j + 4] << (8 * j);
        }
      }
      if (vec && (ldo % 8 == 0) && (((uintptr_t)out & 7) == 0)) {
        *(uint2*)(orow + c) = make_uint2(w0, w1);
      } else {
        for (int j = 0; j < 8; ++j)
          if (c + j < K) orow[c + j] = (uint8_t)((j < 4 ? w0 : w1) >> (8 * (j & 3)));
      }
    }
  }
}

// Per-token dynamic quantisation, rows of up to 8192 elements: one wavefront per row, the row
// held in registers between the absmax reduction and the quantisation (one HBM read, one write,
// no LDS, no workgroup barrier).  Lane l of the wave owns 16-byte chunks l, l+64, ...
template <int DT, int NC, int FMT, int OUT>
__global__ __launch_bounds__(256) void dynamic_token_wave_kernel(const void* __restrict__ x, int64_t ldx, int64_t N,
                                                                 int K, int bits, void* __restrict__ out,
                                                                 int64_t ldo, void* __restrict__ scale_out) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= N) return;
  const uint16_t* xr = (const uint16_t*)x + r * ldx;
  const int nchunk = K >> 3;
  uint4 raw[NC];
  u16x2_t m = {0, 0};  // packed max of 15-bit magnitudes (magnitude bits order like the values)
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = i * 64 + lane;
    raw[i] = c < nchunk ? *(const uint4*)(xr + (c << 3)) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = w[j] & 0x7fff7fffu;
      u16x2_t av;
      __builtin_memcpy(&av, &a, 4);
      m = __builtin_elementwise_max(m, av);
    }
  }
  uint32_t mm = max((uint32_t)m.x, (uint32_t)m.y);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mm = max(mm, (uint32_t)__shfl_xor((int)mm, o, 64));
  const float amax = DT == LLMC_BF16 ? bf16_bits_to_f32((uint16_t)mm) : f16_bits_to_f32((uint16_t)mm);
  const QFormat f = make_qformat(FMT, bits);
  float s = round_to<DT>(amax / ((f.qmax - f.qmin) * 0.5f));
  if (s == 0.f) s = dtype_eps(DT);
  if (lane == 0) store_from_f32<DT>(scale_out, r, s);
  const FastDiv d = make_fastdiv(s);
  // bf16 rows: the scale is a bf16 value too, so the rounded quotient is one multiply away (see qformat.h);
  // the row's largest magnitude is known, only values far below it need the guard
  const bool plain_scale = DT == LLMC_BF16 && bf16_scale_plain(s) && mm < ((127u + 96u) << 7);

#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = i * 64 + lane;
    if (c >= nchunk) break;
    float xv[8], v[8];
    unpack8<DT>(raw[i], xv);
    bool redo;
    if (DT == LLMC_BF16) {
      Bf16Range rg = bf16_range_init();
      bf16_range_add(rg, raw[i].x); bf16_range_add(rg, raw[i].y); bf16_range_add(rg, raw[i].z); bf16_range_add(rg, raw[i].w);
      redo = !(bf16_inputs_plain(rg) & plain_scale);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = xv[j] * d.y;
    } else {
      bool big = false, small = false;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[j] = fastdiv(xv[j], d);
        big = big | !fastdiv_big_ok(v[j]);
        small = small | fastdiv_small(v[j]);
      }
      redo = big | !d.ok;
      if (small) {
#pragma unroll
        for (int j = 0; j < 8; ++j) redo = redo | (fastdiv_small(v[j]) & (xv[j] != 0.f));
      }
    }
    if (redo) {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(round_to<DT>(xv[j] / s) + 0.0f, f.qmin), f.qmax);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        v[j] = __builtin_amdgcn_fmed3f(round16_finite<DT>(v[j]) + 0.0f, f.qmin, f.qmax);
    }
    uint32_t cw[2] = {0u, 0u};  // the eight element bytes
    if (FMT == LLMC_FMT_FP8) {
#pragma unroll
      for (int j = 0; j < 4; ++j) cw[j >> 1] |= hw_e4m3_pair(v[2 * j], v[2 * j + 1]) << (16 * (j & 1));
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        cw[j >> 2] = __builtin_amdgcn_alignbit(__float_as_uint(v[j] + 12582912.0f), cw[j >> 2], 8);
    }
    if (OUT == LLMC_OUT_CODES) {
      *(uint2*)((uint8_t*)out + r * ldo + (c << 3)) = make_uint2(cw[0], cw[1]);
    } else {
      if (FMT == LLMC_FMT_FP8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x2_t t = hw_e4m3_pair_decode(cw[j >> 1] >> (16 * (j & 1)));
          v[2 * j] = t.x;
          v[2 * j + 1] = t.y;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = rintf(v[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] *= s;
      *(uint4*)((uint16_t*)out + r * ldo + (c << 3)) =
          make_uint4(pack16<DT>(v[0], v[1]), pack16<DT>(v[2], v[3]), pack16<DT>(v[4], v[5]), pack16<DT>(v[6], v[7]));
    }
  }
}

template <int DT, int NC>
void launch_token_wave(const void* x, int64_t ldx, int64_t N, int K, int fmt, int bits, int out_mode, void* out,
                       int64_t ldo, void* scale_out, hipStream_t st) {
  const dim3 grid((unsigned)((N + 3) / 4)), block(256);
#define LLMC_TOK(F, O) \
  hipLaunchKernelGGL((dynamic_token_wave_kernel<DT, NC, F, O>), grid, block, 0, st, x, ldx, N, K, bits, out, ldo, scale_out)
  if (fmt == LLMC_FMT_FP8) {
    if (out_mode == LLMC_OUT_CODES) LLMC_TOK(LLMC_FMT_FP8, LLMC_OUT_CODES);
    else LLMC_TOK(LLMC_FMT_FP8, LLMC_OUT_FAKEQUANT);
  } else {
    if (out_mode == LLMC_OUT_CODES) LLMC_TOK(LLMC_FMT_INT, LLMC_OUT_CODES);
    else LLMC_TOK(LLMC_FMT_INT, LLMC_OUT_FAKEQUANT);
  }
#undef LLMC_TOK
}

template <int DT>
void launch_token_wave_nc(const void* x, int64_t ldx, int64_t N, int K, int fmt, int bits, int out_mode,
                          void* out, int64_t ldo, void* scale_out, hipStream_t st) {
  const int nc = (K / 8 + 63) / 64;
  if (nc <= 2) launch_token_wave<DT, 2>(x, ldx, N, K, fmt, bits, out_mode, out, ldo, scale_out, st);
  else if (nc <= 8) launch_token_wave<DT, 8>(x, ldx, N, K, fmt, bits, out_mode, out, ldo, scale_out, st);
  else launch_token_wave<DT, 16>(x, ldx, N, K, fmt, bits, out_mode, out, ldo, scale_out, st);
}

__global__ void fill_u32_kernel(uint32_t* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

int promote(int a, int b) {
  if (a == LLMC_F32 || b == LLMC_F32) return LLMC_F32;
  return a == b ? a : LLMC_F32;
}

}  // namespace

extern "C" int llmc_quantize(const void* x, int32_t x_dtype, int64_t R, int64_t K, int64_t ldx,
                             const void* scale, int32_t scale_dtype, const int8_t* zero_point,
                             const int32_t* g_idx, const float* global_scale, int32_t fmt, int32_t num_bits,
                             int64_t row_div, int64_t scale_row_stride, int64_t col_div, int32_t out_mode,
                             void* out, int32_t out_dtype, int64_t ldo, void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  LLMC_CHECK_ARG(x_dtype >= 0 && x_dtype <= 2, 2);
  LLMC_CHECK_ARG(ldx >= K, 5);
  LLMC_CHECK_ARG(scale, 6);
  LLMC_CHECK_ARG(scale_dtype >= 0 && scale_dtype <= 2, 7);
  LLMC_CHECK_ARG(fmt >= 0 && fmt <= 2, 11);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || (num_bits >= 2 && num_bits <= 8), 12);
  LLMC_CHECK_ARG(row_div > 0 && col_div > 0 && scale_row_stride >= 0, 13);
  LLMC_CHECK_ARG(out_mode >= 0 && out_mode <= 2, 16);
  LLMC_CHECK_ARG(out, 17);
  hipStream_t st = (hipStream_t)stream;
  QuantParams p;
  p.x = x; p.x_dt = x_dtype; p.R = R; p.K = K; p.ldx = ldx;
  p.scale = scale; p.scale_dt = scale_dtype; p.zp = zero_point; p.g_idx = g_idx; p.gscale = global_scale;
  p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.rdiv = row_div; p.srow = scale_row_stride; p.cdiv = col_div;
  const int eff_scale_dt = global_scale ? LLMC_F32 : scale_dtype;
  p.pd = promote(x_dtype, eff_scale_dt);
  p.sd = eff_scale_dt;
  p.out_mode = out_mode; p.out = out; p.out_dt = out_dtype; p.ldo = ldo;

  if (try_launch_rows(p, st)) {
    LLMC_LAUNCH_STATUS();
    return 0;
  }
  bool vec = (K % 8 == 0) && (col_div % 8 == 0) && g_idx == nullptr && (((uintptr_t)x & 15) == 0) &&
             (x_dtype == LLMC_F32 || ldx % 8 == 0);
  if (out_mode == LLMC_OUT_FAKEQUANT)
    vec = vec && (out_dtype == LLMC_F32 || ((ldo % 8 == 0) && (((uintptr_t)out & 15) == 0)));
  else if (out_mode == LLMC_OUT_CODES)
    vec = vec && (ldo % 8 == 0) && (((uintptr_t)out & 7) == 0);
  else if (fmt == LLMC_FMT_FP4)
    vec = vec && (ldo % 4 == 0) && (((uintptr_t)out & 3) == 0);
  if (out_mode == LLMC_OUT_PACKED && fmt == LLMC_FMT_INT) {
    const int pf = 32 / p.bits;
    if (pf != 8 && pf != 4) {
      // fields are OR-ed into place: clear the destination first (a fill kernel, not a memset
      // node, so the call stays safe to capture in a HIP graph)
      const int64_t nw = R * ldo;
      hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((nw + 255) / 256)), dim3(256), 0, st, (uint32_t*)out, nw);
      LLMC_LAUNCH_STATUS();
    }
  }
  const int64_t threads = R * ((K + 7) / 8);
  const unsigned grid = (unsigned)((threads + 255) / 256);
  if (vec)
    hipLaunchKernelGGL((quantize_kernel<true>), dim3(grid), dim3(256), 0, st, p);
  else
    hipLaunchKernelGGL((quantize_kernel<false>), dim3(grid), dim3(256), 0, st, p);
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_dynamic_per_token_quantize(const void* x, int32_t x_dtype, int64_t N, int64_t K,
                                               int64_t ldx, int32_t fmt, int32_t num_bits, int32_t out_mode,
                                               void* out, int64_t ldo, void* scale_out, void* stream) {
  LLMC_CHECK_ARG(x && N > 0 && K > 0, 1);
  LLMC_CHECK_ARG(x_dtype == LLMC_BF16 || x_dtype == LLMC_F16, 2);
  LLMC_CHECK_ARG(K <= 65536, 4);
  LLMC_CHECK_ARG(ldx >= K, 5);
  LLMC_CHECK_ARG(fmt == LLMC_FMT_INT || fmt == LLMC_FMT_FP8, 6);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || num_bits == 8, 7);
  LLMC_CHECK_ARG(out_mode == LLMC_OUT_FAKEQUANT || out_mode == LLMC_OUT_CODES, 8);
  LLMC_CHECK_ARG(out && scale_out, 9);
  hipStream_t st = (hipStream_t)stream;
  const bool wave_ok = K % 8 == 0 && K <= 8192 && ldx % 8 == 0 && (((uintptr_t)x) & 15) == 0 &&
                       (out_mode == LLMC_OUT_CODES ? (ldo % 8 == 0 && (((uintptr_t)out) & 7) == 0)
                                                   : (ldo % 8 == 0 && (((uintptr_t)out) & 15) == 0));
  if (wave_ok) {
    const int nb = fmt == LLMC_FMT_INT ? num_bits : 8;
    if (x_dtype == LLMC_BF16)
      launch_token_wave_nc<LLMC_BF16>(x, ldx, N, (int)K, fmt, nb, out_mode, out, ldo, scale_out, st);
    else
      launch_token_wave_nc<LLMC_F16>(x, ldx, N, (int)K, fmt, nb, out_mode, out, ldo, scale_out, st);
    LLMC_LAUNCH_STATUS();
    return 0;
  }
  const size_t smem = (size_t)((K + 7) / 8 * 8) * 2;
  auto kern = x_dtype == LLMC_BF16 ? dynamic_token_kernel<LLMC_BF16> : dynamic_token_kernel<LLMC_F16>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return 1000 + (int)e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)N), dim3(256), smem, st, x, ldx, (int)K, fmt,
                     fmt == LLMC_FMT_INT ? num_bits : 8, out_mode, out, ldo, scale_out);
  LLMC_LAUNCH_STATUS();
  return 0;
}
