// Workgroup-level pieces of the blocked Cholesky chain (256 threads = four 64-wide waves):
//
//   factor_invert_64 : Cholesky factor L of one 64 x 64 block held in LDS and X = L^-1, both left in LDS
//   mm64_nt          : C(64x64, registers) += / -= A(64x64, LDS) * B(64x64, LDS)^T on v_mfma_f32_32x32x2_f32
//
// factor_invert_64.  A row of the block lives in a lane (lane r = row r) and each wave owns a slab of 16
// columns in 16 registers, so the pivot row's entries reach every row as scalars (v_readlane) and nothing
// crosses waves inside a slab.  Right-looking over the four slabs: wave k factors slab k (16 pivot steps,
// each a readlane + rsqrt chain followed by the slab-internal rank-1 update), publishes it through LDS, and
// the waves to its right apply its rank-16 update to their slabs with the multipliers read as LDS broadcasts.
// The inverse follows by recursive doubling over 16-wide blocks (four diagonal inverses, then
// X21 = -X22 L21 X11 at widths 16 and 32), every product row-times-broadcast on the vector ALU.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cholblk {

constexpr int NB = 64;
constexpr int LDD = 68;  // LDS row stride (floats) of a 64-wide block: 16-byte aligned rows, staggered banks
constexpr int LDP = 20;  // LDS row stride of a 16-wide slab

struct FactorScratch {
  float P[4][NB][LDP];   // factored slabs: P[k][r][t] = L[r][16k+t], 0 above the diagonal
  float Xd[4][16][LDP];  // inverses of the four diagonal 16 x 16 blocks
  float T[32][LDD];      // first product of a doubling step
  float rs[NB];          // reciprocals of L's diagonal
  int bad;               // smallest column whose pivot was not positive and finite, NB if none
  int pad[3];
};

__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// slab K of the factor, in the wave that owns it: a[c] = column 16K+c of the partly updated block, row r
template <int K>
__device__ __forceinline__ void factor_slab(float (&a)[16], int r, FactorScratch& s) {
  int bad = NB;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int jr = 16 * K + j;
    float d = lane_value(a[j], jr);
    if (!(d > 0.f) || d > 3.0e38f) {  // uniform: d is the same in every lane
      bad = bad < jr ? bad : jr;
      d = 1.f;
    }
    // 1/sqrt(d): hardware estimate plus one Newton step (the pivots form a dependent chain, so the
    // full-precision sqrt and divide sequences would dominate it)
    float rs = __builtin_amdgcn_rsqf(d);
    rs = rs * (1.5f - 0.5f * d * rs * rs);
    const float ljj = d * rs;
    a[j] = r > jr ? a[j] * rs : (r == jr ? ljj : 0.f);
    if (r == jr) s.rs[jr] = rs;
#pragma unroll
    for (int c = j + 1; c < 16; ++c) {
      const float lc = lane_value(a[j], 16 * K + c);
      a[c] = fmaf(-a[j], lc, a[c]);
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
    *(float4*)&s.P[K][r][4 * q] = make_float4(a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]);
  if (bad < NB && r == 0 && s.bad == NB) s.bad = bad;  // slabs run in ascending order: the first one found is the smallest
}

// rank-16 update of the slab of wave w (> k) by slab k:  a[c] -= sum_t L[r][16k+t] * L[16w+c][16k+t]
__device__ __forceinline__ void update_slab(float (&a)[16], int r, int w, int k, const FactorScratch& s) {
  float p[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 v = *(const float4*)&s.P[k][r][4 * q];
    p[4 * q] = v.x; p[4 * q + 1] = v.y; p[4 * q + 2] = v.z; p[4 * q + 3] = v.w;
  }
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const float* row = &s.P[k][16 * w + c][0];  // the same address in every lane: a broadcast read
    float acc = a[c];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = *(const float4*)(row + 4 * q);
      acc = fmaf(-p[4 * q], v.x, acc);
      acc = fmaf(-p[4 * q + 1], v.y, acc);
      acc = fmaf(-p[4 * q + 2], v.z, acc);
      acc = fmaf(-p[4 * q + 3], v.w, acc);
    }
    a[c] = acc;
  }
}

// a[c] = D[r][16w + c] for thread (wave w, lane r): the 64 x 64 block to factor (its lower triangle incl. the
// diagonal is used) -> X = inverse of its lower Cholesky factor (LDS, [64][LDD], exact zeros above the
// diagonal).  Every thread of the 256 calls it.  Returns, in every thread, the smallest column whose pivot
// failed (NB if none); that pivot is replaced by 1 and the factorisation carries on.  Ends with a barrier: X is
// readable by all on return.
__device__ __forceinline__ int factor_invert_64(float (&a)[16], float* __restrict__ X, FactorScratch& s) {
  const int tid = threadIdx.x, w = tid >> 6, r = tid & 63;
  if (tid == 0) s.bad = NB;
  for (int i = tid; i < NB * LDD / 4; i += 256) ((float4*)X)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();

  if (w == 0) factor_slab<0>(a, r, s);
  __syncthreads();
  if (w > 0) update_slab(a, r, w, 0, s);
  if (w == 1) factor_slab<1>(a, r, s);
  __syncthreads();
  if (w > 1) update_slab(a, r, w, 1, s);
  if (w == 2) factor_slab<2>(a, r, s);
  __syncthreads();
  if (w > 2) update_slab(a, r, w, 2, s);
  if (w == 3) factor_slab<3>(a, r, s);
  __syncthreads();

  // ---- inverse, level 0: wave w inverts the diagonal block w, one column per lane (lanes 0..15) by forward
  // substitution, the factor's entries read as broadcasts
  if (r < 16) {
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float acc = (i == r) ? 1.f : 0.f;
      const float* lrow = &s.P[w][16 * w + i][0];
#pragma unroll
      for (int t = 0; t < i; ++t) acc = fmaf(-lrow[t], x[t], acc);
      x[i] = acc * s.rs[16 * w + i];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s.Xd[w][i][r] = x[i];
      X[(16 * w + i) * LDD + 16 * w + r] = x[i];
    }
  }
  __syncthreads();

  // ---- level 1 (waves 0 and 1): X[16(2p+1).., 16(2p)..] = -Xd[2p+1] * (L[2p+1][2p] * Xd[2p]); lane (i, q) owns
  // row i, columns 4q..4q+3 of the 16 x 16 result
  if (w < 2) {
    const int p = w, i = r & 15, q = r >> 4;
    const int lo = 2 * p, hi = 2 * p + 1;
    float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float l = s.P[lo][16 * hi + i][k];
      const float4 xv = *(const float4*)&s.Xd[lo][k][4 * q];
      t[0] = fmaf(l, xv.x, t[0]); t[1] = fmaf(l, xv.y, t[1]); t[2] = fmaf(l, xv.z, t[2]); t[3] = fmaf(l, xv.w, t[3]);
    }
    *(float4*)&s.T[16 * p + i][4 * q] = make_float4(t[0], t[1], t[2], t[3]);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's own LDS writes have landed (one wave per product)
    __builtin_amdgcn_wave_barrier();
    float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float xh = s.Xd[hi][i][k];
      const float4 tv = *(const float4*)&s.T[16 * p + k][4 * q];
      o[0] = fmaf(-xh, tv.x, o[0]); o[1] = fmaf(-xh, tv.y, o[1]); o[2] = fmaf(-xh, tv.z, o[2]); o[3] = fmaf(-xh, tv.w, o[3]);
    }
    *(float4*)(X + (16 * hi + i) * LDD + 16 * lo + 4 * q) = make_float4(o[0], o[1], o[2], o[3]);
  }
  __syncthreads();

  // ---- level 2 (all waves): X[32.., 0..32) = -X22 * (L21 * X11) with 32 x 32 blocks; thread (i, q) owns row i,
  // columns 4q..4q+3 of the 32 x 32 result
  {
    const int i = tid >> 3, q = tid & 7;
    float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      const float l = s.P[k >> 4][32 + i][k & 15];
      const float4 xv = *(const float4*)(X + k * LDD + 4 * q);
      t[0] = fmaf(l, xv.x, t[0]); t[1] = fmaf(l, xv.y, t[1]); t[2] = fmaf(l, xv.z, t[2]); t[3] = fmaf(l, xv.w, t[3]);
    }
    *(float4*)&s.T[i][4 * q] = make_float4(t[0], t[1], t[2], t[3]);
    __syncthreads();
    float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      const float xh = X[(32 + i) * LDD + 32 + k];
      const float4 tv = *(const float4*)&s.T[k][4 * q];
      o[0] = fmaf(-xh, tv.x, o[0]); o[1] = fmaf(-xh, tv.y, o[1]); o[2] = fmaf(-xh, tv.z, o[2]); o[3] = fmaf(-xh, tv.w, o[3]);
    }
    *(float4*)(X + (32 + i) * LDD + 4 * q) = make_float4(o[0], o[1], o[2], o[3]);
  }
  __syncthreads();
  return s.bad;
}

}  // namespace cholblk
