// Min/max observers and scale/zero-point generation (bandwidth-bound, no MFMA).
//
// A weight [R,K] is observed in groups of g consecutive columns (g = K for
// per-channel, g = R*K for per-tensor on a contiguous weight).  Each group's
// min and max come out in the observed dtype, exactly as torch.amin/amax give
// them.  Loads are 16 bytes per lane and fully coalesced; a group narrower than
// a wavefront is reduced with xor-shuffles inside its lane segment.
#include "qformat.h"

namespace {

template <int DT>
struct Vec;  // 16-byte vector of DT elements
template <>
struct Vec<LLMC_BF16> {
  static constexpr int N = 8;
};
template <>
struct Vec<LLMC_F16> {
  static constexpr int N = 8;
};
template <>
struct Vec<LLMC_F32> {
  static constexpr int N = 4;
};

template <int DT>
__device__ __forceinline__ void minmax16(const void* p, float& mn, float& mx) {
  const uint4 v = *(const uint4*)p;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (DT == LLMC_F32) {
      const float f = __uint_as_float(w[j]);
      mn = fminf(mn, f);
      mx = fmaxf(mx, f);
    } else if (DT == LLMC_BF16) {
      const float lo = __uint_as_float(w[j] << 16), hi = __uint_as_float(w[j] & 0xffff0000u);
      mn = fminf(mn, fminf(lo, hi));
      mx = fmaxf(mx, fmaxf(lo, hi));
    } else {
      const float lo = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu)), hi = f16_bits_to_f32((uint16_t)(w[j] >> 16));
      mn = fminf(mn, fminf(lo, hi));
      mx = fmaxf(mx, fmaxf(lo, hi));
    }
  }
}

// Groups of g = L * VPL * N elements: one workgroup walks one row, L (power of two <= 64)
// neighbouring lanes share a group and each lane loads VPL consecutive 16-byte vectors.
template <int DT, int VPL>
__global__ __launch_bounds__(256) void minmax_rows_kernel(const void* __restrict__ x, int64_t ldw, int upr,
                                                          int ng, int lshift, void* __restrict__ mn_out,
                                                          void* __restrict__ mx_out) {
  constexpr int N = Vec<DT>::N;
  const int64_t r = blockIdx.x;
  const char* row = (const char*)x + r * ldw * (DT == LLMC_F32 ? 4 : 2);
  const int L = 1 << lshift;
  for (int u = threadIdx.x; u < upr; u += 256) {
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < VPL; ++k) minmax16<DT>(row + ((int64_t)u * VPL + k) * 16, mn, mx);
    for (int o = L >> 1; o > 0; o >>= 1) {
      mn = fminf(mn, __shfl_xor(mn, o, 64));
      mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    }
    if ((u & (L - 1)) == 0) {
      const int64_t grp = r * ng + (u >> lshift);
      store_from_f32<DT>(mn_out, grp, mn);
      store_from_f32<DT>(mx_out, grp, mx);
    }
  }
  (void)N;
}

// One wave per (group, split): strided 16-byte loads when VEC, element loads otherwise.
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void minmax_wave_kernel(const void* __restrict__ x, int64_t ldw,
                                                          int64_t ngroups_total, int ng, int64_t g,
                                                          int splits, float* __restrict__ part_mn,
                                                          float* __restrict__ part_mx,
                                                          void* __restrict__ mn_out,
                                                          void* __restrict__ mx_out) {
  constexpr int N = Vec<DT>::N;
  const int lane = threadIdx.x & 63;
  const int64_t wid = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wid >= ngroups_total * splits) return;
  const int64_t grp = wid / splits;
  const int sp = (int)(wid % splits);
  const int64_t r = grp / ng, gi = grp % ng;
  const int64_t base = r * ldw + gi * g;
  // this split covers [lo, hi) of the group, chunk boundaries on multiples of 64*N
  const int64_t chunk = (((g + splits - 1) / splits + 64 * N - 1) / (64 * N)) * (64 * N);
  const int64_t lo = sp * chunk;
  const int64_t hi = lo + chunk < g ? lo + chunk : g;
  float mn = INFINITY, mx = -INFINITY;
  if (VEC) {
    for (int64_t j = lo + (int64_t)lane * N; j < hi; j += 64 * N)
      minmax16<DT>((const char*)x + (base + j) * (DT == LLMC_F32 ? 4 : 2), mn, mx);
  } else {
    for (int64_t j = lo + lane; j < hi; j += 64) {
      const float f = load_as_f32<DT>(x, base + j);
      mn = fminf(mn, f);
      mx = fmaxf(mx, f);
    }
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (lane == 0) {
    if (splits == 1) {
      store_from_f32<DT>(mn_out, grp, mn);
      store_from_f32<DT>(mx_out, grp, mx);
    } else {
      part_mn[wid] = mn;
      part_mx[wid] = mx;
    }
  }
}

template <int DT>
__global__ void minmax_finish_kernel(const float* part_mn, const float* part_mx, int64_t ngroups,
                                     int splits, void* mn_out, void* mx_out) {
  const int64_t grp = blockIdx.x;
  float mn = INFINITY, mx = -INFINITY;
  for (int s = threadIdx.x; s < splits; s += 64) {
    mn = fminf(mn, part_mn[grp * splits + s]);
    mx = fmaxf(mx, part_mx[grp * splits + s]);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (threadIdx.x == 0) {
    store_from_f32<DT>(mn_out, grp, mn);
    store_from_f32<DT>(mx_out, grp, mx);
  }
}

// bh x bw blocks of a [R,K] weight (zero padded past the edges, as the reference pads)
template <int DT>
__global__ __launch_bounds__(64) void minmax_block_kernel(const void* __restrict__ x, int64_t ldw, int R,
                                                          int K, int bh, int bw, int nbc,
                                                          void* __restrict__ mn_out,
                                                          void* __restrict__ mx_out) {
  const int64_t blk = blockIdx.x;
  const int br = (int)(blk / nbc), bc = (int)(blk % nbc);
  float mn = INFINITY, mx = -INFINITY;
  const int n = bh * bw;
  for (int e = threadIdx.x; e < n; e += 64) {
    const int rr = br * bh + e / bw, cc = bc * bw + e % bw;
    const float f = (rr < R && cc < K) ? load_as_f32<DT>(x, (int64_t)rr * ldw + cc) : 0.f;
    mn = fminf(mn, f);
    mx = fmaxf(mx, f);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (threadIdx.x == 0) {
    store_from_f32<DT>(mn_out, blk, mn);
    store_from_f32<DT>(mx_out, blk, mx);
  }
}

// x viewed as [N0, N1, G] with element strides (s0, s1, 1); reduce over N0 and G -> [N1]
template <int DT>
__global__ __launch_bounds__(256) void minmax_strided_kernel(const void* __restrict__ x, int64_t N0,
                                                             int64_t G, int64_t s0, int64_t s1,
                                                             void* __restrict__ mn_out,
                                                             void* __restrict__ mx_out) {
  __shared__ float smn[4], smx[4];
  const int64_t n1 = blockIdx.x;
  float mn = INFINITY, mx = -INFINITY;
  const int64_t total = N0 * G;
  for (int64_t e = threadIdx.x; e < total; e += 256) {
    const float f = load_as_f32<DT>(x, (e / G) * s0 + n1 * s1 + (e % G));
    mn = fminf(mn, f);
    mx = fmaxf(mx, f);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) {
    smn[threadIdx.x >> 6] = mn;
    smx[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      mn = fminf(mn, smn[w]);
      mx = fmaxf(mx, smx[w]);
    }
    store_from_f32<DT>(mn_out, n1, mn);
    store_from_f32<DT>(mx_out, n1, mx);
  }
}

template <int DT>
__global__ __launch_bounds__(256) void absmax_kernel(const void* __restrict__ mn, const void* __restrict__ mx,
                                                     int64_t n, uint32_t* __restrict__ out_bits) {
  float a = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    a = fmaxf(a, fmaxf(-load_as_f32<DT>(mn, i), load_as_f32<DT>(mx, i)));
  }
  a = wave_max(a);
  // non-negative floats order like their bit patterns
  if ((threadIdx.x & 63) == 0) atomicMax(out_bits, __float_as_uint(fmaxf(a, 0.f)));
}

__global__ void gparam_kernel(const float* absmax, int sd, float* out) {
  // The reference forms `448 * 6 / absmax` with a Python float on the left, which torch evaluates as
  // absmax.reciprocal() * 2688: the reciprocal is rounded to the statistics' dtype before the product, and
  // the product is rounded again (2688/40 gives 67.5 in bf16 this way, not the 67.0 of a single division).
  const float r = round_rt(__fdiv_rn(1.0f, round_rt(absmax[0], sd)), sd);
  out[0] = round_rt(__fmul_rn(r, 2688.0f), sd);
}

__global__ __launch_bounds__(256) void qparams_kernel(const void* __restrict__ mn, const void* __restrict__ mx,
                                                      int64_t n, int sd, int fmt, int bits, int symmetric,
                                                      int scale_mode, const float* __restrict__ gscale,
                                                      void* __restrict__ scale_out, int scale_out_dt,
                                                      int8_t* __restrict__ zp_out,
                                                      uint8_t* __restrict__ scale_code_out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const QFormat f = make_qformat(fmt, bits);
  float s, zp;
  int e;
  qparams_from_minmax(load_rt(mn, i, sd), load_rt(mx, i, sd), sd, f, symmetric != 0, scale_mode,
                      gscale ? gscale[0] : 1.f, &s, &zp, &e);
  store_rt(scale_out, i, s, scale_out_dt);
  if (zp_out) zp_out[i] = (int8_t)zp;
  if (scale_code_out) scale_code_out[i] = scale_mode == LLMC_SCALE_MXFP4 ? (uint8_t)e : e4m3_encode(s);
}

template <int DT>
int observe_groups(const void* x, int64_t R, int64_t K, int64_t ldw, int64_t g, void* mn, void* mx,
                   float* ws, int64_t ws_bytes, hipStream_t st) {
  constexpr int N = Vec<DT>::N;
  const int esz = DT == LLMC_F32 ? 4 : 2;
  const int64_t ng = K / g;
  const int64_t total = R * ng;
  const bool aligned = (((uintptr_t)x) & 15) == 0 && (ldw % N) == 0 && (g % N) == 0;
  const int64_t L = g / N;  // 16-byte vectors per group
  if (aligned && L >= 1 && L <= 128 && (L & (L - 1)) == 0 && R <= 0x7fffffffLL && K <= (1LL << 30)) {
    const int vpl = L >= 2 ? 2 : 1;
    const int lanes = (int)(L / vpl);
    int lshift = 0;
    while ((1 << lshift) < lanes) ++lshift;
    const int upr = (int)(K / (N * vpl));
    if (vpl == 2)
      hipLaunchKernelGGL((minmax_rows_kernel<DT, 2>), dim3((unsigned)R), dim3(256), 0, st, x, ldw, upr, (int)ng,
                         lshift, mn, mx);
    else
      hipLaunchKernelGGL((minmax_rows_kernel<DT, 1>), dim3((unsigned)R), dim3(256), 0, st, x, ldw, upr, (int)ng,
                         lshift, mn, mx);
    LLMC_LAUNCH_STATUS();
    return 0;
  }
  // split long groups when there are too few of them to fill the chip
  int splits = 1;
  if (total < 2048 && g >= 64 * N * 8) {
    int64_t want = 4096 / (total > 0 ? total : 1);
    int64_t maxs = g / (64 * N * 4);
    splits = (int)(want < maxs ? want : maxs);
    if (splits < 1) splits = 1;
    if ((int64_t)splits * total * 8 > ws_bytes) splits = 1;
  }
  float* pmn = ws;
  float* pmx = ws ? ws + total * splits : nullptr;
  const int64_t waves = total * splits;
  const unsigned grid = (unsigned)((waves * 64 + 255) / 256);
  if (aligned)
    hipLaunchKernelGGL((minmax_wave_kernel<DT, true>), dim3(grid), dim3(256), 0, st, x, ldw, total, (int)ng,
                       g, splits, pmn, pmx, mn, mx);
  else
    hipLaunchKernelGGL((minmax_wave_kernel<DT, false>), dim3(grid), dim3(256), 0, st, x, ldw, total, (int)ng,
                       g, splits, pmn, pmx, mn, mx);
  LLMC_LAUNCH_STATUS();
  if (splits > 1) {
    hipLaunchKernelGGL((minmax_finish_kernel<DT>), dim3((unsigned)total), dim3(64), 0, st, pmn, pmx, total,
                       splits, mn, mx);
    LLMC_LAUNCH_STATUS();
  }
  (void)esz;
  return 0;
}

}  // namespace

extern "C" int64_t llmc_minmax_workspace_bytes(void) { return 64 * 1024; }

extern "C" int llmc_minmax_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                  int64_t group, void* min_out, void* max_out, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  LLMC_CHECK_ARG(ldw >= K, 5);
  LLMC_CHECK_ARG(group > 0 && K % group == 0, 6);
  LLMC_CHECK_ARG(min_out && max_out, 7);
  hipStream_t st = (hipStream_t)stream;
  float* ws = (float*)workspace;
  if (dtype == LLMC_BF16) return observe_groups<LLMC_BF16>(x, R, K, ldw, group, min_out, max_out, ws, workspace_bytes, st);
  if (dtype == LLMC_F16) return observe_groups<LLMC_F16>(x, R, K, ldw, group, min_out, max_out, ws, workspace_bytes, st);
  return observe_groups<LLMC_F32>(x, R, K, ldw, group, min_out, max_out, ws, workspace_bytes, st);
}

extern "C" int llmc_minmax_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                  int32_t block_h, int32_t block_w, void* min_out, void* max_out,
                                  void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  LLMC_CHECK_ARG(block_h > 0 && block_w > 0, 6);
  hipStream_t st = (hipStream_t)stream;
  const int nbr = (int)((R + block_h - 1) / block_h), nbc = (int)((K + block_w - 1) / block_w);
  dim3 grid((unsigned)(nbr * (int64_t)nbc));
#define LLMC_BLK(DT)                                                                                   \
  hipLaunchKernelGGL((minmax_block_kernel<DT>), grid, dim3(64), 0, st, x, ldw, (int)R, (int)K, block_h, \
                     block_w, nbc, min_out, max_out)
  if (dtype == LLMC_BF16) LLMC_BLK(LLMC_BF16);
  else if (dtype == LLMC_F16) LLMC_BLK(LLMC_F16);
  else LLMC_BLK(LLMC_F32);
#undef LLMC_BLK
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_minmax_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                                   int64_t stride0, int64_t stride1, void* min_out, void* max_out,
                                   void* stream) {
  LLMC_CHECK_ARG(x && n0 > 0 && n1 > 0 && group > 0, 1);
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  hipStream_t st = (hipStream_t)stream;
#define LLMC_STR(DT)                                                                                 \
  hipLaunchKernelGGL((minmax_strided_kernel<DT>), dim3((unsigned)n1), dim3(256), 0, st, x, n0, group, \
                     stride0, stride1, min_out, max_out)
  if (dtype == LLMC_BF16) LLMC_STR(LLMC_BF16);
  else if (dtype == LLMC_F16) LLMC_STR(LLMC_F16);
  else LLMC_STR(LLMC_F32);
#undef LLMC_STR
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_absmax_accumulate(const void* min_vals, const void* max_vals, int64_t n, int32_t dtype,
                                      float* absmax_inout, void* stream) {
  LLMC_CHECK_ARG(min_vals && max_vals && n > 0, 1);
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 4);
  LLMC_CHECK_ARG(absmax_inout, 5);
  hipStream_t st = (hipStream_t)stream;
  unsigned grid = (unsigned)((n + 255) / 256);
  if (grid > 1024) grid = 1024;
#define LLMC_ABS(DT) \
  hipLaunchKernelGGL((absmax_kernel<DT>), dim3(grid), dim3(256), 0, st, min_vals, max_vals, n, (uint32_t*)absmax_inout)
  if (dtype == LLMC_BF16) LLMC_ABS(LLMC_BF16);
  else if (dtype == LLMC_F16) LLMC_ABS(LLMC_F16);
  else LLMC_ABS(LLMC_F32);
#undef LLMC_ABS
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_generate_gparam(const float* absmax, int32_t stats_dtype, float* global_scale_out,
                                    void* stream) {
  LLMC_CHECK_ARG(absmax, 1);
  LLMC_CHECK_ARG(stats_dtype >= 0 && stats_dtype <= 2, 2);
  LLMC_CHECK_ARG(global_scale_out, 3);
  hipLaunchKernelGGL(gparam_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, absmax, stats_dtype, global_scale_out);
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_calculate_qparams(const void* min_vals, const void* max_vals, int64_t n,
                                      int32_t stats_dtype, int32_t fmt, int32_t num_bits, int32_t symmetric,
                                      int32_t scale_mode, const float* global_scale, void* scale_out,
                                      int32_t scale_out_dtype, int8_t* zero_point_out,
                                      uint8_t* scale_code_out, void* stream) {
  LLMC_CHECK_ARG(min_vals && max_vals && n > 0, 1);
  LLMC_CHECK_ARG(stats_dtype >= 0 && stats_dtype <= 2, 4);
  LLMC_CHECK_ARG(fmt >= 0 && fmt <= 2, 5);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || (num_bits >= 2 && num_bits <= 8), 6);
  LLMC_CHECK_ARG(symmetric || fmt == LLMC_FMT_INT || fmt == LLMC_FMT_FP8, 7);
  LLMC_CHECK_ARG(scale_mode >= 0 && scale_mode <= 2, 8);
  LLMC_CHECK_ARG(scale_mode != LLMC_SCALE_NVFP4 || global_scale, 9);
  LLMC_CHECK_ARG(scale_out, 10);
  hipLaunchKernelGGL(qparams_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     min_vals, max_vals, n, stats_dtype, fmt, num_bits, symmetric, scale_mode, global_scale,
                     scale_out, scale_out_dtype, zero_point_out, scale_code_out);
  LLMC_LAUNCH_STATUS();
  return 0;
}
