// MSE observer: grid search over shrink factors p_i = 1 - i/grid of each group's (min,max).
//
// The reference walks the steps on the host and stops GLOBALLY after `patience`
// consecutive steps in which no group improved.  Here every group walks all steps in
// one launch with its running best in registers and records the steps at which it
// improved in a bit mask; the masks are OR-ed into a global per-step flag word.  A
// one-thread kernel replays the patience rule on the flags to get the stop step, and
// a last kernel picks, per group, its latest improvement at or before that step --
// the same selection as the host loop, without a host round trip per step.
// The inner loop is VALU/transcendental bound (powf per element per step); the
// weight is read from HBM once.
#include <string.h>

#include <mutex>

#include "qformat.h"

namespace {

constexpr int MAX_STEPS = 256;
constexpr int MASK_WORDS = MAX_STEPS / 64;

struct MseParams {
  const void* x;
  int dt;            // dtype of the observed values (and of every intermediate)
  int fmt, bits, symmetric, scale_mode;
  int steps;
  double grid;       // step i shrinks the range by p_i = (float)(1.0 - i/grid), as the host loop does
  float norm;
  float expand;
  void* min0;        // [N] expanded observed min (dtype dt)
  void* max0;        // [N]
  uint64_t* masks;   // [N][MASK_WORDS]
  uint64_t* flags;   // [MASK_WORDS] zero-initialised
  const uint16_t* powtab;  // a^norm rounded to dt for every non-negative 16-bit a (see mse_powtab_kernel), or NULL
  // importance-weighted variant (observers/imatrix.py:255-328): the error |fq(x) - x|^norm is formed and
  // summed in fp32 (values are quantised in dt as before) and weighted per input channel
  int err32;
  const float* imp;  // [K] weights, or NULL for uniform
};

__device__ __forceinline__ float step_factor(int i, double grid) { return (float)(1.0 - (double)i / grid); }

// a^norm (a >= 0) as the eager pow forms it in dtype dt: exponents 2, 3 and 0.5 have closed forms (a*a,
// (a*a)*a with the inner product rounded to dt as well, sqrt), anything else is one pow rounded to dt
__device__ __forceinline__ float pow_eager(float a, float norm, int dt) {
  if (norm == 2.0f) return round_rt(__fmul_rn(a, a), dt);
  if (norm == 3.0f) return round_rt(__fmul_rn(round_rt(__fmul_rn(a, a), dt), a), dt);
  if (norm == 0.5f) return round_rt(__fsqrt_rn(a), dt);
  return round_rt(powf(a, norm), dt);
}

// |fq(x) - x|^norm with every intermediate rounded to dt
__device__ __forceinline__ float elem_error(float x, float s, float zp, bool has_zp, int dt, const QFormat& f,
                                            float norm) {
  const float q = quantize_value(x, s, zp, has_zp, dt, f);
  const float dq = dequantize_value(q, s, zp, has_zp, dt);
  const float a = fabsf(round_rt(dq - x, dt));
  // `norm` arrives already rounded to dt: the eager pow converts its scalar exponent to the tensor dtype
  return pow_eager(a, norm, dt);
}

// fp32 error of the importance-weighted search: fq(x) in dt, then (fq - x), abs, pow in fp32; the
// eager pow multiplies for exponents 2 and 3
__device__ __forceinline__ float elem_error32(float x, float s, float zp, bool has_zp, int dt, const QFormat& f,
                                              float norm) {
  const float q = quantize_value(x, s, zp, has_zp, dt, f);
  const float dq = dequantize_value(q, s, zp, has_zp, dt);
  const float a = fabsf(__fsub_rn(dq, x));
  if (norm == 2.0f) return __fmul_rn(a, a);
  if (norm == 3.0f) return __fmul_rn(__fmul_rn(a, a), a);
  if (norm == 0.5f) return __fsqrt_rn(a);
  return powf(a, norm);
}

__device__ __forceinline__ void unpack8(uint4 v, int dt, float* o) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (dt == LLMC_BF16) {
      o[2 * j] = __uint_as_float(w[j] << 16);
      o[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    } else {
      o[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
      o[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
    }
  }
}

__device__ __forceinline__ void or_flags(uint64_t* flags, const uint64_t* m) {
  // OR over the workgroup first, then one atomic per word and workgroup
  __shared__ unsigned long long sflags[MASK_WORDS];
  if (threadIdx.x < MASK_WORDS) sflags[threadIdx.x] = 0ull;
  __syncthreads();
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) {
    unsigned long long v = m[wd];
    for (int o = 32; o > 0; o >>= 1) v |= __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0 && v) atomicOr(&sflags[wd], v);
  }
  __syncthreads();
  if (threadIdx.x < MASK_WORDS && sflags[threadIdx.x]) atomicOr((unsigned long long*)&flags[threadIdx.x], sflags[threadIdx.x]);
}

// 16-bit inputs, groups of g = 8*L consecutive elements (L a power of two <= 64 lanes per group)
__global__ __launch_bounds__(256) void mse_team_kernel(MseParams p, int64_t ngroups, int ng, int g, int L,
                                                       int64_t ldw) {
  const int64_t gtid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t grp = gtid / L;
  const int sub = (int)(gtid % L);
  const bool live = grp < ngroups;
  const QFormat f = make_qformat(p.fmt, p.bits);
  float xv[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) xv[j] = 0.f;
  float mn = INFINITY, mx = -INFINITY;
  if (live) {
    const int64_t r = grp / ng, gi = grp % ng;
    const uint4 v = *(const uint4*)((const uint16_t*)p.x + r * ldw + gi * g + (int64_t)sub * 8);
    unpack8(v, p.dt, xv);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      mn = fminf(mn, xv[j]);
      mx = fmaxf(mx, xv[j]);
    }
  }
  for (int o = L >> 1; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  mn = round_rt(mn * p.expand, p.dt);
  mx = round_rt(mx * p.expand, p.dt);
  float best = p.dt == LLMC_BF16 ? 3.3895313892515355e38f : p.dt == LLMC_F16 ? 65504.0f : 3.4028234663852886e38f;
  if (p.err32) best = 3.4028234663852886e38f;
  float wt[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) wt[j] = 1.f;
  if (p.err32 && p.imp && live) {
    const int64_t gi = grp % ng;
#pragma unroll
    for (int j = 0; j < 8; ++j) wt[j] = p.imp[gi * g + (int64_t)sub * 8 + j];
  }
  uint64_t mask[MASK_WORDS];
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) mask[wd] = 0ull;
  for (int i = 0; i < p.steps; ++i) {
    const float pi = step_factor(i, p.grid);
    const float smin = round_rt(mn * pi, p.dt), smax = round_rt(mx * pi, p.dt);
    float s, zp;
    int e;
    qparams_from_minmax(smin, smax, p.dt, f, p.symmetric != 0, p.scale_mode, 1.f, &s, &zp, &e);
    float err = 0.f;
    if (p.err32) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float ej = elem_error32(xv[j], s, zp, !p.symmetric, p.dt, f, p.norm);
        err += p.imp ? __fmul_rn(ej, wt[j]) : ej;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) err += elem_error(xv[j], s, zp, !p.symmetric, p.dt, f, p.norm);
    }
    for (int o = L >> 1; o > 0; o >>= 1) err += __shfl_xor(err, o, 64);
    if (!p.err32) err = round_rt(err, p.dt);
    if (err < best) {
      best = err;
#pragma unroll
      for (int wd = 0; wd < MASK_WORDS; ++wd)
        if (wd == (i >> 6)) mask[wd] |= 1ull << (i & 63);
    }
  }
  if (!live) {
#pragma unroll
    for (int wd = 0; wd < MASK_WORDS; ++wd) mask[wd] = 0ull;
  }
  if (live && sub == 0) {
    store_rt(p.min0, grp, mn, p.dt);
    store_rt(p.max0, grp, mx, p.dt);
#pragma unroll
    for (int wd = 0; wd < MASK_WORDS; ++wd) p.masks[grp * MASK_WORDS + wd] = mask[wd];
  }
  or_flags(p.flags, mask);
}

// ---- 16-bit inputs: the same arithmetic with everything the format decides fixed at compile time,
// the division by the step's scale done with the shared-divisor sequence (exact, see qformat.h), the
// e4m3 / e2m1 rounding done by the conversion instructions, and the power evaluated as
// 2^(norm*log2 a) in extended precision.

// a^norm (a >= 0) rounded to DT.  a = m*2^E; norm*E is exact in fp32 (norm has at most 11
// significant bits, E at most 8) and splits into an integer I and a fraction r, so
// a^norm = 2^I * 2^(r + norm*log2 m) with the second exponent small: the hardware log2/exp2 (1 ulp
// each) leave a few ulps of error in total.  If rounding to DT could fall either way within 16 ulps
// the library powf decides, so the rounded value matches the reference's pow-then-round.
template <int DT>
__device__ __forceinline__ float pow_round16(float a, float norm) {
  const float m = __builtin_amdgcn_frexp_mantf(a);
  const int E = __builtin_amdgcn_frexp_expf(a);
  const float y = norm * (float)E;
  const float I = rintf(y);
  const float t = fmaf(norm, __builtin_amdgcn_logf(m), y - I);
  const float pf = ldexpf(__builtin_amdgcn_exp2f(t), (int)I);
  const uint32_t w = pack16<DT>(pf * 0.99999809265136719f, pf * 1.0000019073486328f);  // 1 -+ 2^-19
  if ((w & 0xffffu) != (w >> 16)) return round_rt(powf(a, norm), DT);
  return DT == LLMC_BF16 ? __uint_as_float(w << 16) : f16_bits_to_f32((uint16_t)(w & 0xffffu));
}

template <int DT>
__device__ __forceinline__ void unpack8t(const uint4& v, float* x) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (DT == LLMC_BF16) {
      x[2 * j] = __uint_as_float(w[j] << 16);
      x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    } else {
      x[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
      x[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
    }
  }
}

// sum over 8 elements of |fq(x) - x|^norm, every intermediate rounded to DT
template <int DT, int FMT, bool HAS_ZP, bool TAB>
__device__ __forceinline__ float chunk_error(const float (&x)[8], float s, float zp, const QFormat& f, float norm,
                                             const uint16_t* __restrict__ tab) {
  float v[8];
  const FastDiv d = make_fastdiv(s);
  bool big = false, small = false;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    v[j] = fastdiv(x[j], d);
    big = big | !fastdiv_big_ok(v[j]);
    small = small | fastdiv_small(v[j]);
  }
  bool redo = big | !d.ok;
  if (small) {
#pragma unroll
    for (int j = 0; j < 8; ++j) redo = redo | (fastdiv_small(v[j]) & (x[j] != 0.f));
  }
  if (redo) {
    float err = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float q = quantize_value(x[j], s, zp, HAS_ZP, DT, f);
      const float dq = dequantize_value(q, s, zp, HAS_ZP, DT);
      const float a = fabsf(round_rt(dq - x[j], DT));
      err += pow_eager(a, norm, DT);
    }
    return err;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    v[j] = round16_finite<DT>(v[j]);
    v[j] = HAS_ZP ? round16_finite<DT>(v[j] + zp) : v[j] + 0.0f;
    v[j] = __builtin_amdgcn_fmed3f(v[j], f.qmin, f.qmax);
    if (FMT == LLMC_FMT_INT) v[j] = rintf(v[j]);
  }
  if (FMT == LLMC_FMT_FP8) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x2_t t = hw_e4m3_pair_decode(hw_e4m3_pair(v[2 * j], v[2 * j + 1]));
      v[2 * j] = t.x;
      v[2 * j + 1] = t.y;
    }
  } else if (FMT == LLMC_FMT_FP4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x2_t t = hw_e2m1_pair_decode(hw_e2m1_pair(v[2 * j], v[2 * j + 1]));
      v[2 * j] = t.x;
      v[2 * j + 1] = t.y;
    }
  }
  float err = 0.f;
  if (TAB) {
    // a is a non-negative value of the 16-bit dtype: its power, already rounded, sits in the table at a's bits
    uint32_t at[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float dq = v[j];
      if (HAS_ZP) dq = round16_finite<DT>(dq - zp);
      dq = round16_finite<DT>(dq * s);
      const float a = fabsf(round16_finite<DT>(dq - x[j]));
      at[j] = DT == LLMC_BF16 ? (__float_as_uint(a) >> 16) : (uint32_t)f32_to_f16_bits(a);
    }
    uint32_t pw[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) pw[j] = tab[at[j] & 0x7fffu];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      err += DT == LLMC_BF16 ? __uint_as_float(pw[j] << 16) : f16_bits_to_f32((uint16_t)pw[j]);
    return err;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float dq = v[j];
    if (HAS_ZP) dq = round16_finite<DT>(dq - zp);
    dq = round16_finite<DT>(dq * s);
    const float a = fabsf(round16_finite<DT>(dq - x[j]));
    if (norm == 2.0f)
      err += round16_finite<DT>(a * a);
    else if (norm == 3.0f)
      err += round16_finite<DT>(round16_finite<DT>(a * a) * a);
    else if (norm == 0.5f)
      err += round16_finite<DT>(__fsqrt_rn(a));
    else
      err += pow_round16<DT>(a, norm);
  }
  return err;
}

// 16-bit inputs, groups of g = 8*L consecutive elements (L a power of two <= 64 lanes per group)
// TAB: the power comes from p.powtab, copied into LDS (64 KiB) when the workgroup starts: a lookup instead of the
// two dozen issue slots of exp2(norm * log2 a) with its exactness guard.  Workgroups of 1024 threads then (the two
// that fit a CU's LDS put eight waves on every SIMD), and a workgroup walks over the groups in strides of the
// grid, so that the table is fetched a few hundred times per call and not once per 1024 threads of work.
template <int DT, int FMT, bool SYM, bool TAB>
__global__ __launch_bounds__(TAB ? 512 : 256) void mse_team_fast_kernel(MseParams p, int64_t ngroups, int ng, int g,
                                                                         int lshift, int64_t ldw) {
  constexpr int BLOCK = TAB ? 512 : 256;
  extern __shared__ __attribute__((aligned(16))) uint16_t powlds[];
  if (TAB) {
    const uint4* src = (const uint4*)p.powtab;
    uint4* dst = (uint4*)powlds;
#pragma unroll
    for (int k = 0; k < 65536 / 16 / BLOCK; ++k) dst[k * BLOCK + threadIdx.x] = src[k * BLOCK + threadIdx.x];
    __syncthreads();
  }
  const int L = 1 << lshift;
  uint64_t any[MASK_WORDS];  // OR of this thread's masks over its groups
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) any[wd] = 0ull;
  const int64_t threads = ngroups << lshift;
  // the bound is uniform over the workgroup, so every lane of a group's team takes part in every shuffle
  for (int64_t base = (int64_t)blockIdx.x * BLOCK; base < threads; base += (int64_t)gridDim.x * BLOCK) {
  const int64_t gtid = base + threadIdx.x;
  const int64_t grp = gtid >> lshift;
  const int sub = (int)(gtid & (L - 1));
  const bool live = grp < ngroups;
  const QFormat f = make_qformat(FMT, p.bits);
  float xv[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) xv[j] = 0.f;
  float mn = INFINITY, mx = -INFINITY;
  if (live) {
    const int64_t r = grp / ng, gi = grp % ng;
    const uint4 v = *(const uint4*)((const uint16_t*)p.x + r * ldw + gi * g + (int64_t)sub * 8);
    unpack8t<DT>(v, xv);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      mn = fminf(mn, xv[j]);
      mx = fmaxf(mx, xv[j]);
    }
  }
  for (int o = L >> 1; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  mn = round_to<DT>(mn * p.expand);
  mx = round_to<DT>(mx * p.expand);
  float best = DT == LLMC_BF16 ? 3.3895313892515355e38f : 65504.0f;
  uint64_t mask[MASK_WORDS];
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) mask[wd] = 0ull;
  for (int i = 0; i < p.steps; ++i) {
    const float pi = step_factor(i, p.grid);
    const float smin = round_to<DT>(mn * pi), smax = round_to<DT>(mx * pi);
    float s, zp;
    int e;
    qparams_from_minmax(smin, smax, DT, f, SYM, p.scale_mode, 1.f, &s, &zp, &e);
    float err = chunk_error<DT, FMT, !SYM, TAB>(xv, s, zp, f, p.norm, powlds);
    for (int o = L >> 1; o > 0; o >>= 1) err += __shfl_xor(err, o, 64);
    err = round_to<DT>(err);
    if (err < best) {
      best = err;
#pragma unroll
      for (int wd = 0; wd < MASK_WORDS; ++wd)
        if (wd == (i >> 6)) mask[wd] |= 1ull << (i & 63);
    }
  }
  if (!live) {
#pragma unroll
    for (int wd = 0; wd < MASK_WORDS; ++wd) mask[wd] = 0ull;
  }
  if (live && sub == 0) {
    store_from_f32<DT>(p.min0, grp, mn);
    store_from_f32<DT>(p.max0, grp, mx);
#pragma unroll
    for (int wd = 0; wd < MASK_WORDS; ++wd) p.masks[grp * MASK_WORDS + wd] = mask[wd];
  }
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) any[wd] |= mask[wd];
  }
  or_flags(p.flags, any);
}

// a^norm rounded to dt for each of the 32768 non-negative 16-bit values a, as 16-bit patterns: exactly what the
// eager pow gives element by element, evaluated once per call instead of once per element and candidate
__global__ __launch_bounds__(256) void mse_powtab_kernel(uint16_t* __restrict__ tab, float norm, int dt) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const float a = dt == LLMC_BF16 ? bf16_bits_to_f32((uint16_t)i) : f16_bits_to_f32((uint16_t)i);
  const float r = pow_eager(a, norm, dt);
  tab[i] = dt == LLMC_BF16 ? f32_to_bf16_bits(r) : f32_to_f16_bits(r);
}

template <int DT, int FMT, bool SYM>
int launch_team_fast_one(const MseParams& p, int64_t n, int ng, int g, int lshift, int64_t ldw, hipStream_t st) {
  const int64_t threads = n << lshift;
  if (p.powtab != nullptr) {
    auto kern = mse_team_fast_kernel<DT, FMT, SYM, true>;
    static const hipError_t configured =
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    if (configured != hipSuccess) return 1000 + (int)configured;
    const int64_t wgs = (threads + 511) / 512;
    hipLaunchKernelGGL(kern, dim3((unsigned)(wgs < 4096 ? wgs : 4096)), dim3(512), 65536, st, p, n, ng, g, lshift, ldw);
  } else {
    hipLaunchKernelGGL((mse_team_fast_kernel<DT, FMT, SYM, false>), dim3((unsigned)((threads + 255) / 256)),
                       dim3(256), 0, st, p, n, ng, g, lshift, ldw);
  }
  return 0;
}

template <int DT>
int launch_team_fast(const MseParams& p, int64_t n, int ng, int g, int lshift, int64_t ldw, hipStream_t st) {
  if (p.fmt == LLMC_FMT_INT)
    return p.symmetric ? launch_team_fast_one<DT, LLMC_FMT_INT, true>(p, n, ng, g, lshift, ldw, st)
                       : launch_team_fast_one<DT, LLMC_FMT_INT, false>(p, n, ng, g, lshift, ldw, st);
  if (p.fmt == LLMC_FMT_FP8)
    return p.symmetric ? launch_team_fast_one<DT, LLMC_FMT_FP8, true>(p, n, ng, g, lshift, ldw, st)
                       : launch_team_fast_one<DT, LLMC_FMT_FP8, false>(p, n, ng, g, lshift, ldw, st);
  return launch_team_fast_one<DT, LLMC_FMT_FP4, true>(p, n, ng, g, lshift, ldw, st);
}

struct GenericLayout {
  int mode;  // 0: (n0, n1, G) view with element strides (s0, s1, 1); 1: bh x bw blocks of an [R,K] matrix
  int64_t n0, G, s0, s1;
  int R, K, bh, bw, nbc;
  int64_t ldw;
  int64_t ng;  // mode 0, weighted search: groups per row (column of element e of group n1 = (n1 % ng)*G + e % G)
};

__device__ __forceinline__ float generic_load(const void* x, int dt, const GenericLayout& l, int64_t n1, int64_t e) {
  if (l.mode == 0) return load_rt(x, (e / l.G) * l.s0 + n1 * l.s1 + (e % l.G), dt);
  const int br = (int)(n1 / l.nbc), bc = (int)(n1 % l.nbc);
  const int rr = br * l.bh + (int)(e / l.bw), cc = bc * l.bw + (int)(e % l.bw);
  return (rr < l.R && cc < l.K) ? load_rt(x, (int64_t)rr * l.ldw + cc, dt) : 0.f;
}

__device__ __forceinline__ float block_sum(float v, float* sh) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  return sh[0] + sh[1] + sh[2] + sh[3];
}

// any layout / dtype: one workgroup per group, values re-read (from L2) at every step
__global__ __launch_bounds__(256) void mse_generic_kernel(MseParams p, GenericLayout l) {
  __shared__ float sh[4];
  __shared__ float shm[8];
  const int64_t n1 = blockIdx.x;
  const int64_t total = l.mode == 0 ? l.n0 * l.G : (int64_t)l.bh * l.bw;
  const QFormat f = make_qformat(p.fmt, p.bits);
  float mn = INFINITY, mx = -INFINITY;
  for (int64_t e = threadIdx.x; e < total; e += 256) {
    const float v = generic_load(p.x, p.dt, l, n1, e);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) {
    shm[threadIdx.x >> 6] = mn;
    shm[4 + (threadIdx.x >> 6)] = mx;
  }
  __syncthreads();
  mn = fminf(fminf(shm[0], shm[1]), fminf(shm[2], shm[3]));
  mx = fmaxf(fmaxf(shm[4], shm[5]), fmaxf(shm[6], shm[7]));
  mn = round_rt(mn * p.expand, p.dt);
  mx = round_rt(mx * p.expand, p.dt);
  float best = p.dt == LLMC_BF16 ? 3.3895313892515355e38f : p.dt == LLMC_F16 ? 65504.0f : 3.4028234663852886e38f;
  if (p.err32) best = 3.4028234663852886e38f;
  uint64_t mask[MASK_WORDS];
#pragma unroll
  for (int wd = 0; wd < MASK_WORDS; ++wd) mask[wd] = 0ull;
  for (int i = 0; i < p.steps; ++i) {
    const float pi = step_factor(i, p.grid);
    const float smin = round_rt(mn * pi, p.dt), smax = round_rt(mx * pi, p.dt);
    float s, zp;
    int e_;
    qparams_from_minmax(smin, smax, p.dt, f, p.symmetric != 0, p.scale_mode, 1.f, &s, &zp, &e_);
    float err = 0.f;
    if (p.err32) {
      for (int64_t e = threadIdx.x; e < total; e += 256) {
        const float ej = elem_error32(generic_load(p.x, p.dt, l, n1, e), s, zp, !p.symmetric, p.dt, f, p.norm);
        err += p.imp ? __fmul_rn(ej, p.imp[(n1 % l.ng) * l.G + e % l.G]) : ej;
      }
      err = block_sum(err, sh);
    } else {
      for (int64_t e = threadIdx.x; e < total; e += 256)
        err += elem_error(generic_load(p.x, p.dt, l, n1, e), s, zp, !p.symmetric, p.dt, f, p.norm);
      err = round_rt(block_sum(err, sh), p.dt);
    }
    if (err < best) {
      best = err;
#pragma unroll
      for (int wd = 0; wd < MASK_WORDS; ++wd)
        if (wd == (i >> 6)) mask[wd] |= 1ull << (i & 63);
    }
  }
  if (threadIdx.x == 0) {
    store_rt(p.min0, n1, mn, p.dt);
    store_rt(p.max0, n1, mx, p.dt);
#pragma unroll
    for (int wd = 0; wd < MASK_WORDS; ++wd) {
      p.masks[n1 * MASK_WORDS + wd] = mask[wd];
      if (mask[wd]) atomicOr((unsigned long long*)&p.flags[wd], (unsigned long long)mask[wd]);
    }
  }
}

// replay of the host loop's patience rule on the per-step "any group improved" flags
__global__ void mse_stop_kernel(const uint64_t* flags, int steps, int patience, int* last_step) {
  int no_improve = 0, last = steps - 1;
  for (int i = 0; i < steps; ++i) {
    if ((flags[i >> 6] >> (i & 63)) & 1ull) {
      no_improve = 0;
    } else if (++no_improve >= patience) {
      last = i;
      break;
    }
  }
  *last_step = last;
}

__global__ __launch_bounds__(256) void mse_select_kernel(const uint64_t* __restrict__ masks, int64_t n,
                                                         const int* __restrict__ last_step,
                                                         double grid, int dt,
                                                         const void* __restrict__ min0,
                                                         const void* __restrict__ max0,
                                                         void* __restrict__ min_out, void* __restrict__ max_out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int last = *last_step;
  int best = -1;
  for (int wd = MASK_WORDS - 1; wd >= 0 && best < 0; --wd) {
    uint64_t m = masks[i * MASK_WORDS + wd];
    const int lo = wd * 64;
    if (last < lo) continue;
    if (last - lo < 63) m &= (2ull << (last - lo)) - 1ull;
    if (m) best = lo + 63 - __clzll((long long)m);
  }
  const float mn = load_rt(min0, i, dt), mx = load_rt(max0, i, dt);
  // no recorded improvement (e.g. non-finite errors): the reference keeps the un-shrunk range
  const float pb = best < 0 ? 1.0f : step_factor(best, grid);
  store_rt(min_out, i, best < 0 ? mn : round_rt(mn * pb, dt), dt);
  store_rt(max_out, i, best < 0 ? mx : round_rt(mx * pb, dt), dt);
}

__global__ void mse_zero_flags_kernel(uint64_t* flags) {
  if (threadIdx.x < MASK_WORDS) flags[threadIdx.x] = 0ull;
}

inline int64_t align256(int64_t b) { return (b + 255) / 256 * 256; }

// host-side round-to-nearest-even of a scalar to bf16 / f16
float round_host(float v, int dt) {
  if (dt == LLMC_BF16) {
    uint32_t u;
    memcpy(&u, &v, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&v, &u, 4);
    return v;
  }
  if (dt == LLMC_F16) return (float)(_Float16)v;
  return v;
}

struct Workspace {
  uint64_t* flags;
  int* last;
  uint16_t* powtab;
  void* min0;
  void* max0;
  uint64_t* masks;
};

Workspace carve(void* ws, int64_t n) {
  char* c = (char*)ws;
  Workspace w;
  w.flags = (uint64_t*)c; c += 256;
  w.last = (int*)c; c += 256;
  w.powtab = (uint16_t*)c; c += 65536;
  w.min0 = c; c += align256(n * 4);
  w.max0 = c; c += align256(n * 4);
  w.masks = (uint64_t*)c;
  return w;
}

int finish(const MseParams& p, const Workspace& w, int64_t n, int patience, void* min_out, void* max_out,
           hipStream_t st) {
  hipLaunchKernelGGL(mse_stop_kernel, dim3(1), dim3(1), 0, st, w.flags, p.steps, patience, w.last);
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(mse_select_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w.masks, n, w.last,
                     p.grid, p.dt, w.min0, w.max0, min_out, max_out);
  LLMC_LAUNCH_STATUS();
  return 0;
}

int setup(MseParams& p, Workspace& w, void* workspace, int64_t n, hipStream_t st) {
  w = carve(workspace, n);
  hipLaunchKernelGGL(mse_zero_flags_kernel, dim3(1), dim3(64), 0, st, w.flags);
  LLMC_LAUNCH_STATUS();
  p.min0 = w.min0;
  p.max0 = w.max0;
  p.masks = w.masks;
  p.flags = w.flags;
  return 0;
}

}  // namespace

extern "C" int64_t llmc_mse_workspace_bytes(int64_t n_groups) {
  return 512 + 65536 + 2 * align256(n_groups * 4) + align256(n_groups * MASK_WORDS * 8);
}

static int check_common(int32_t dtype, int32_t fmt, int32_t num_bits, int32_t scale_mode, int32_t steps,
                        double grid, float norm, float expand, int32_t patience) {
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  LLMC_CHECK_ARG(fmt >= 0 && fmt <= 2, 100);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || (num_bits >= 2 && num_bits <= 8), 101);
  LLMC_CHECK_ARG(scale_mode == LLMC_SCALE_PLAIN || scale_mode == LLMC_SCALE_MXFP4, 102);
  LLMC_CHECK_ARG(steps >= 0 && steps <= MAX_STEPS, 103);
  LLMC_CHECK_ARG(grid > 0.0, 104);
  LLMC_CHECK_ARG(norm > 0.f && expand > 0.f && patience > 0, 105);
  return 0;
}

extern "C" int llmc_mse_observe_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                       int64_t group, int32_t fmt, int32_t num_bits, int32_t symmetric,
                                       int32_t scale_mode, int32_t steps, double grid, int32_t patience,
                                       float norm, float expand, void* min_out, void* max_out, void* workspace,
                                       int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  int rc = check_common(dtype, fmt, num_bits, scale_mode, steps, grid, norm, expand, patience);
  if (rc) return rc;
  LLMC_CHECK_ARG(ldw >= K, 5);
  LLMC_CHECK_ARG(group > 0 && K % group == 0, 6);
  LLMC_CHECK_ARG(min_out && max_out, 16);
  const int64_t n = R * (K / group);
  LLMC_CHECK_ARG(workspace && (((uintptr_t)workspace) & 255) == 0 && workspace_bytes >= llmc_mse_workspace_bytes(n), 18);
  hipStream_t st = (hipStream_t)stream;
  MseParams p = {};
  p.x = x; p.dt = dtype; p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.symmetric = symmetric; p.scale_mode = scale_mode; p.steps = steps; p.grid = grid; p.norm = round_host(norm, dtype); p.expand = expand;
  Workspace w;
  rc = setup(p, w, workspace, n, st);
  if (rc) return rc;
  const int64_t L = group / 8;
  const bool team = dtype != LLMC_F32 && group % 8 == 0 && L <= 64 && (L & (L - 1)) == 0 && ldw % 8 == 0 &&
                    (((uintptr_t)x) & 15) == 0;
  if (team && (fmt != LLMC_FMT_FP4 || symmetric)) {
    int lshift = 0;
    while ((1 << lshift) < L) ++lshift;
    if (p.norm != 2.0f && p.norm != 3.0f && p.norm != 0.5f) {  // the other exponents have closed forms
      hipLaunchKernelGGL(mse_powtab_kernel, dim3(128), dim3(256), 0, st, w.powtab, p.norm, dtype);
      LLMC_LAUNCH_STATUS();
      p.powtab = w.powtab;
    }
    const int lrc = dtype == LLMC_BF16
                        ? launch_team_fast<LLMC_BF16>(p, n, (int)(K / group), (int)group, lshift, ldw, st)
                        : launch_team_fast<LLMC_F16>(p, n, (int)(K / group), (int)group, lshift, ldw, st);
    if (lrc) return lrc;
  } else if (team) {
    const int64_t threads = n * L;
    hipLaunchKernelGGL(mse_team_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, p, n,
                       (int)(K / group), (int)group, (int)L, ldw);
  } else {
    GenericLayout l = {};
    l.mode = 0; l.n0 = 1; l.G = group; l.s0 = 0; l.s1 = group; l.ldw = ldw;
    if (ldw != K) {
      // rows are not contiguous: one row at a time keeps the strided view valid
      LLMC_CHECK_ARG(group == K, 5);
      l.s1 = ldw;
    }
    hipLaunchKernelGGL(mse_generic_kernel, dim3((unsigned)n), dim3(256), 0, st, p, l);
  }
  LLMC_LAUNCH_STATUS();
  return finish(p, w, n, patience, min_out, max_out, st);
}

static int observe_strided_impl(int err32, const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                                        int64_t stride0, int64_t stride1, int32_t fmt, int32_t num_bits,
                                        int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                        int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(x && n0 > 0 && n1 > 0 && group > 0, 1);
  int rc = check_common(dtype, fmt, num_bits, scale_mode, steps, grid, norm, expand, patience);
  if (rc) return rc;
  LLMC_CHECK_ARG(min_out && max_out, 17);
  LLMC_CHECK_ARG(workspace && (((uintptr_t)workspace) & 255) == 0 && workspace_bytes >= llmc_mse_workspace_bytes(n1), 19);
  hipStream_t st = (hipStream_t)stream;
  MseParams p = {};
  p.x = x; p.dt = dtype; p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.symmetric = symmetric; p.scale_mode = scale_mode; p.steps = steps; p.grid = grid;
  p.norm = err32 ? norm : round_host(norm, dtype); p.expand = expand; p.err32 = err32;
  Workspace w;
  rc = setup(p, w, workspace, n1, st);
  if (rc) return rc;
  GenericLayout l = {};
  l.mode = 0; l.n0 = n0; l.G = group; l.s0 = stride0; l.s1 = stride1;
  hipLaunchKernelGGL(mse_generic_kernel, dim3((unsigned)n1), dim3(256), 0, st, p, l);
  LLMC_LAUNCH_STATUS();
  return finish(p, w, n1, patience, min_out, max_out, st);
}

extern "C" int llmc_mse_observe_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                                        int64_t stride0, int64_t stride1, int32_t fmt, int32_t num_bits,
                                        int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                        int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
  return observe_strided_impl(0, x, dtype, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode, steps,
                              grid, patience, norm, expand, min_out, max_out, workspace, workspace_bytes, stream);
}

static int observe_blocks_impl(int err32, const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                       int32_t block_h, int32_t block_w, int32_t fmt, int32_t num_bits,
                                       int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                       int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                       void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  int rc = check_common(dtype, fmt, num_bits, scale_mode, steps, grid, norm, expand, patience);
  if (rc) return rc;
  LLMC_CHECK_ARG(block_h > 0 && block_w > 0, 6);
  const int nbr = (int)((R + block_h - 1) / block_h), nbc = (int)((K + block_w - 1) / block_w);
  const int64_t n = (int64_t)nbr * nbc;
  LLMC_CHECK_ARG(min_out && max_out, 17);
  LLMC_CHECK_ARG(workspace && (((uintptr_t)workspace) & 255) == 0 && workspace_bytes >= llmc_mse_workspace_bytes(n), 19);
  hipStream_t st = (hipStream_t)stream;
  MseParams p = {};
  p.x = x; p.dt = dtype; p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.symmetric = symmetric; p.scale_mode = scale_mode; p.steps = steps; p.grid = grid;
  p.norm = err32 ? norm : round_host(norm, dtype); p.expand = expand; p.err32 = err32;
  Workspace w;
  rc = setup(p, w, workspace, n, st);
  if (rc) return rc;
  GenericLayout l = {};
  l.mode = 1; l.R = (int)R; l.K = (int)K; l.bh = block_h; l.bw = block_w; l.nbc = nbc; l.ldw = ldw;
  hipLaunchKernelGGL(mse_generic_kernel, dim3((unsigned)n), dim3(256), 0, st, p, l);
  LLMC_LAUNCH_STATUS();
  return finish(p, w, n, patience, min_out, max_out, st);
}

extern "C" int llmc_mse_observe_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                       int32_t block_h, int32_t block_w, int32_t fmt, int32_t num_bits,
                                       int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                       int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                       void* workspace, int64_t workspace_bytes, void* stream) {
  return observe_blocks_impl(0, x, dtype, R, K, ldw, block_h, block_w, fmt, num_bits, symmetric, scale_mode, steps, grid,
                             patience, norm, expand, min_out, max_out, workspace, workspace_bytes, stream);
}

// ---- importance-weighted search (observers/imatrix.py) -------------------------------------------

namespace {

// partial[s][c] = sum over the s-th slice of the token rows of x[t][c]^2 (fp32, fixed order)
__global__ __launch_bounds__(256) void sumsq_partial_kernel(const void* __restrict__ x, int dt, int64_t T, int64_t K,
                                                            int64_t ldx, int slices, float* __restrict__ partial) {
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= K) return;
  const int s = blockIdx.y;
  const int64_t per = (T + slices - 1) / slices;
  const int64_t t0 = s * per, t1 = (t0 + per) < T ? t0 + per : T;
  float acc = 0.f;
  for (int64_t t = t0; t < t1; ++t) {
    const float v = load_rt(x, t * ldx + c, dt);
    acc += v * v;
  }
  partial[(int64_t)s * K + c] = acc;
}

__global__ __launch_bounds__(64) void sumsq_finish_kernel(const float* __restrict__ partial, int64_t K, int slices,
                                                          float* __restrict__ sum) {
  const int64_t c = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (c >= K) return;
  // the loads of 16 slices are issued together (one memory round trip per batch); the additions keep
  // the order s = 0, 1, 2, ...
  float acc = 0.f;
  int s = 0;
  for (; s + 16 <= slices; s += 16) {
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = partial[(int64_t)(s + j) * K + c];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc += v[j];
  }
  for (; s < slices; ++s) acc += partial[(int64_t)s * K + c];
  sum[c] += acc;
}

constexpr int SUMSQ_SLICES = 64;

// 16-bit input with 16-byte aligned rows: a workgroup covers 256 columns of one token slice as 32 column
// groups (16-byte loads) x 8 token lanes, folds the token lanes through LDS and writes one partial row
__global__ __launch_bounds__(256) void sumsq_partial16_kernel(const uint16_t* __restrict__ x, int dt, int64_t T,
                                                              int64_t K, int64_t ldx, int slices,
                                                              float* __restrict__ partial) {
  __shared__ float red[8][256 + 8];
  const int cg = threadIdx.x & 31, tl = threadIdx.x >> 5;
  const int64_t c0 = (int64_t)blockIdx.x * 256 + cg * 8;
  const int s = blockIdx.y;
  const int64_t per = (T + slices - 1) / slices;
  const int64_t t0 = s * per, t1 = (t0 + per) < T ? t0 + per : T;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  if (c0 < K) {
    for (int64_t t = t0 + tl; t < t1; t += 8) {
      const uint4 v = *(const uint4*)(x + t * ldx + c0);
      float f[8];
      unpack8(v, dt, f);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] += f[j] * f[j];
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) red[tl][cg * 8 + j] = acc[j];
  __syncthreads();
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c < K) {
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) sum += red[r][threadIdx.x];
    partial[(int64_t)s * K + c] = sum;
  }
}

}  // namespace

extern "C" int64_t llmc_sumsq_workspace_bytes(int64_t K) { return align256(K * SUMSQ_SLICES * 4); }

// both entry points: partial sums of the token slices into `partial` ([slices, K] fp32), then sum += their total
static int sumsq_launch(const void* x, int32_t dtype, int64_t T, int64_t K, int64_t ldx, float* sum, float* partial,
                        hipStream_t st) {
  const int slices = T < SUMSQ_SLICES ? (int)T : SUMSQ_SLICES;
  const bool wide = dtype != LLMC_F32 && K % 8 == 0 && ldx % 8 == 0 && (((uintptr_t)x) & 15) == 0;
  if (wide)
    hipLaunchKernelGGL(sumsq_partial16_kernel, dim3((unsigned)((K + 255) / 256), (unsigned)slices), dim3(256), 0, st,
                       (const uint16_t*)x, dtype, T, K, ldx, slices, partial);
  else
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3((unsigned)((K + 255) / 256), (unsigned)slices), dim3(256), 0, st, x,
                       dtype, T, K, ldx, slices, partial);
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(sumsq_finish_kernel, dim3((unsigned)((K + 63) / 64)), dim3(64), 0, st,
                     (const float*)partial, K, slices, sum);
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_sumsq_accumulate(const void* x, int32_t dtype, int64_t T, int64_t K, int64_t ldx, float* sum,
                                     void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  LLMC_CHECK_ARG(T >= 0 && K > 0 && ldx >= K, 3);
  if (T == 0) return 0;
  LLMC_CHECK_ARG(x != nullptr && sum != nullptr, 1);
  LLMC_CHECK_ARG(workspace && (((uintptr_t)workspace) & 255) == 0 && workspace_bytes >= llmc_sumsq_workspace_bytes(K), 7);
  return sumsq_launch(x, dtype, T, K, ldx, sum, (float*)workspace, (hipStream_t)stream);
}

// ---- the same accumulation for callers that cannot allocate ---------------------------------------
// The partial sums live in a device array of this library instead of a caller's workspace.  Every GPU
// that loads the library holds its own copy of the array (4 MiB) at its own address until the process
// ends; host code never uses the array's name as an address, only the pointer hipGetSymbolAddress
// returned for the device that is current.
constexpr int64_t SUMSQ_NOALLOC_MAX_K = LLMC_SUMSQ_NOALLOC_MAX_K;
static __device__ __align__(256) float scratch[SUMSQ_SLICES * SUMSQ_NOALLOC_MAX_K];

namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

// the address of `scratch` on the current device, looked up once per device
int scratch_for_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return 1000 + (int)e;
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return 2000;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return 1000 + (int)e;
    if (!p) return 2001;
    g_scratch_ptr[dev] = (float*)p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace

extern "C" int llmc_sumsq_accumulate_noalloc(const void* x, int32_t dtype, int64_t T, int64_t K, int64_t ldx,
                                             float* sum, void* stream) {
  LLMC_CHECK_ARG(dtype >= 0 && dtype <= 2, 2);
  LLMC_CHECK_ARG(T >= 0 && ldx >= K, 3);
  // widths beyond the array's capacity are refused, never truncated
  LLMC_CHECK_ARG(K > 0 && K <= SUMSQ_NOALLOC_MAX_K, 4);
  if (T == 0) return 0;
  LLMC_CHECK_ARG(x != nullptr && sum != nullptr, 1);
  float* partial = nullptr;
  const int rc = scratch_for_current_device(&partial);
  if (rc) return rc;
  // every partial row that the finishing kernel reads is written by this call's first kernel, so the
  // contents that an earlier (possibly wider or longer) call left behind need no clearing
  return sumsq_launch(x, dtype, T, K, ldx, sum, partial, (hipStream_t)stream);
}

extern "C" int llmc_imatrix_observe_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                           int64_t group, int32_t fmt, int32_t num_bits, int32_t symmetric,
                                           int32_t scale_mode, int32_t steps, double grid, int32_t patience,
                                           float norm, float expand, const float* importance, void* min_out,
                                           void* max_out, void* workspace, int64_t workspace_bytes,
                                           void* stream) {
  LLMC_CHECK_ARG(x && R > 0 && K > 0, 1);
  // patience 0 = never stop early (imatrix.py:321-325)
  const int pat = patience > 0 ? patience : 0x7fffffff;
  int rc = check_common(dtype, fmt, num_bits, scale_mode, steps, grid, norm, expand, pat);
  if (rc) return rc;
  LLMC_CHECK_ARG(patience >= 0, 13);
  LLMC_CHECK_ARG(ldw >= K, 5);
  LLMC_CHECK_ARG(group > 0 && K % group == 0, 6);
  LLMC_CHECK_ARG(min_out && max_out, 17);
  const int64_t n = R * (K / group);
  LLMC_CHECK_ARG(workspace && (((uintptr_t)workspace) & 255) == 0 && workspace_bytes >= llmc_mse_workspace_bytes(n), 19);
  hipStream_t st = (hipStream_t)stream;
  MseParams p = {};
  p.x = x; p.dt = dtype; p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.symmetric = symmetric; p.scale_mode = scale_mode; p.steps = steps; p.grid = grid; p.norm = norm; p.expand = expand;
  p.err32 = 1; p.imp = importance;
  Workspace w;
  rc = setup(p, w, workspace, n, st);
  if (rc) return rc;
  const int64_t L = group / 8;
  const bool team = dtype != LLMC_F32 && group % 8 == 0 && L <= 64 && (L & (L - 1)) == 0 && ldw % 8 == 0 &&
                    (((uintptr_t)x) & 15) == 0;
  if (team) {
    const int64_t threads = n * L;
    hipLaunchKernelGGL(mse_team_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, p, n,
                       (int)(K / group), (int)group, (int)L, ldw);
  } else {
    GenericLayout l = {};
    l.mode = 0; l.n0 = 1; l.G = group; l.s0 = 0; l.s1 = group; l.ldw = ldw; l.ng = K / group;
    if (ldw != K) {
      LLMC_CHECK_ARG(group == K, 5);
      l.s1 = ldw;
    }
    hipLaunchKernelGGL(mse_generic_kernel, dim3((unsigned)n), dim3(256), 0, st, p, l);
  }
  LLMC_LAUNCH_STATUS();
  return finish(p, w, n, pat, min_out, max_out, st);
}

// the uniform fall-back of the importance-weighted observer on the other layouts (imatrix.py:141-245 route
// block-wise weights and non-weight observers to the same search without weights): fp32 error, patience 0 = never stop
extern "C" int llmc_imatrix_observe_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                                            int64_t stride0, int64_t stride1, int32_t fmt, int32_t num_bits,
                                            int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                            int32_t patience, float norm, float expand, void* min_out,
                                            void* max_out, void* workspace, int64_t workspace_bytes,
                                            void* stream) {
  LLMC_CHECK_ARG(patience >= 0, 14);
  return observe_strided_impl(1, x, dtype, n0, n1, group, stride0, stride1, fmt, num_bits, symmetric, scale_mode, steps,
                              grid, patience > 0 ? patience : 0x7fffffff, norm, expand, min_out, max_out, workspace,
                              workspace_bytes, stream);
}

extern "C" int llmc_imatrix_observe_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                           int32_t block_h, int32_t block_w, int32_t fmt, int32_t num_bits,
                                           int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                           int32_t patience, float norm, float expand, void* min_out,
                                           void* max_out, void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(patience >= 0, 14);
  return observe_blocks_impl(1, x, dtype, R, K, ldw, block_h, block_w, fmt, num_bits, symmetric, scale_mode, steps, grid,
                             patience > 0 ? patience : 0x7fffffff, norm, expand, min_out, max_out, workspace,
                             workspace_bytes, stream);
}
