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
