// Workgroup-level pieces of the blocked Cholesky chain (512 threads = eight 64-wide waves, two per SIMD).
//
// factor_invert_64: Cholesky factor L of one 64 x 64 block and X = L^-1, left in LDS.
//
// The block lives in LDS column-major; a column slab of 16 is factored by one wave with a row of the block in
// each lane (lane r = row r, the slab's 16 entries of that row in 16 registers), so a pivot row's entries reach
// every row as scalars (v_readlane) and nothing crosses waves inside a slab.  A lone wave issues one vector
// instruction every eight cycles on this part, so the slab loop is trimmed to what the chain needs:
//
//   * the columns stay unscaled (the L D L^T form): the rank-1 update of column c by pivot column j is
//     a[c] -= a[j] * (a_c[j] / d_j); the serial chain from one pivot to the next is readlane -> reciprocal ->
//     multiply -> readlane -> fma, and no square root sits on it;
//   * a pivot that is not positive and finite is only recorded (one ballot per slab): what follows it is
//     discarded by the caller, so no fix-up sits on the chain either;
//   * what the other phases need goes to LDS once per slab: V (the unscaled columns), T (V D^-1, the unit-lower
//     factor) and 1/sqrt(d) per row.
//
// Between two slabs all eight waves apply the rank-16 update to the columns still to come
// (A[r][c] -= sum_t V[r][t] T[c][t], T read as LDS broadcasts), and while wave k+1 factors its slab, waves 4-7
// invert slab k: the elimination on an identity with the unit-lower factor needs no row scaling and, run over all
// 64 rows, leaves X_kk = L_kk^-1 in the rows of the diagonal block and W_k = -L[below, k] X_kk in the rows below.
// The off-diagonal blocks of X follow by doubling, X21 = X22 (-L21 X11) at widths 16 and 32, as 16 x 16 tiles on
// v_mfma_f32_16x16x4_f32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cholblk {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int NB = 64;
constexpr int NT = 512;  // threads per workgroup
constexpr int LDD = 68;  // LDS row stride (floats) of a 64-wide block: 16-byte aligned rows, staggered banks
constexpr int LDP = 20;  // LDS row stride of a 16-wide slab

struct FactorScratch {
  float X[NB][LDD];      // the result: inverse of the factor, zeros above the diagonal
  float AT[NB][LDD];     // the block, column-major: AT[c][r] = A[r][c]; the doubling reuses it for -L21 X11
  float V[4][NB][LDP];   // V[k][r][t]: unscaled factored columns of slab k (L = V D^-1/2)
  float T[4][NB][LDP];   // T[k][r][t] = V[k][r][t] / d: the unit-lower factor
  float W[3][NB][LDP];   // W[k][r][c] = -(L[r, slab k] X_kk)[c] for the rows r below slab k's diagonal block
  float rs[NB];          // 1 / L[r][r]
  int bad;               // smallest column whose pivot was not positive and finite, NB if none
  int pad[3];
};

__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Slab K, in one wave, lane r = row r.
template <int K>
__device__ __forceinline__ void factor_slab(int r, FactorScratch& s) {
  float a[16], t[16], myd = 1.f;
#pragma unroll
  for (int c = 0; c < 16; ++c) a[c] = s.AT[16 * K + c][r];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int jr = 16 * K + j;
    const float d = lane_value(a[j], jr);
    t[j] = a[j] * __builtin_amdgcn_rcpf(d);
    // the multipliers are read into distinct scalar registers first and applied afterwards: a scalar register
    // written by a readlane cannot feed the very next vector instruction, and one register reused for every
    // pair serialises them
    float m[16];
#pragma unroll
    for (int c = j + 1; c < 16; ++c) m[c] = lane_value(t[j], 16 * K + c);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = j + 1; c < 16; ++c) a[c] = fmaf(-a[j], m[c], a[c]);
    myd = r == jr ? a[j] : myd;
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    *(float4*)&s.V[K][r][4 * q] = make_float4(a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]);
    *(float4*)&s.T[K][r][4 * q] = make_float4(t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]);
  }
  // per row of the diagonal block: 1/sqrt(d) (hardware estimate plus one Newton step) and the pivot check.  A
  // pivot that is zero, negative, infinite or NaN gives an estimate that is infinite, zero or NaN, and the
  // Newton step turns each of those into NaN.
  const bool diag = r >= 16 * K && r < 16 * K + 16;
  float rs = __builtin_amdgcn_rsqf(myd);
  rs = rs * (1.5f - 0.5f * myd * rs * rs);
  if (diag) s.rs[r] = rs;
  const unsigned long long failed = __ballot(diag && !(rs > 0.f && rs < 3.0e38f && myd <= 3.0e38f));
  if (failed != 0ull && r == 0 && s.bad == NB) s.bad = __builtin_ctzll(failed);  // slabs run in ascending order
}

// Rank-16 update by slab k of the columns still to come, shared by the eight waves: wave v takes NC / 8 columns.
template <int K>
__device__ __forceinline__ void update_trailing(int r, int v, FactorScratch& s) {
  constexpr int NC = (48 - 16 * K) / 8;  // 6, 4, 2
  float p[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 x = *(const float4*)&s.V[K][r][4 * q];
    p[4 * q] = x.x; p[4 * q + 1] = x.y; p[4 * q + 2] = x.z; p[4 * q + 3] = x.w;
  }
  const int c0 = 16 * (K + 1) + v * NC;
  float acc[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) acc[i] = s.AT[c0 + i][r];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float4 tv[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) tv[i] = *(const float4*)&s.T[K][c0 + i][4 * q];  // one address per wave: broadcast
#pragma unroll
    for (int i = 0; i < NC; ++i) acc[i] = fmaf(-p[4 * q], tv[i].x, acc[i]);
#pragma unroll
    for (int i = 0; i < NC; ++i) acc[i] = fmaf(-p[4 * q + 1], tv[i].y, acc[i]);
#pragma unroll
    for (int i = 0; i < NC; ++i) acc[i] = fmaf(-p[4 * q + 2], tv[i].z, acc[i]);
#pragma unroll
    for (int i = 0; i < NC; ++i) acc[i] = fmaf(-p[4 * q + 3], tv[i].w, acc[i]);
  }
#pragma unroll
  for (int i = 0; i < NC; ++i) s.AT[c0 + i][r] = acc[i];
}

// Elimination on an identity with the unit-lower form of slab K, one of four helper waves (h = 0..3): the wave
// owns the columns h, h+4, h+8, h+12 of the slab's 16.  Rows of the diagonal block end up holding X_kk (after the
// row scaling by 1/L[r][r]), rows below it W_k.
template <int K>
__device__ __forceinline__ void invert_slab(int r, int h, FactorScratch& s) {
  float tl[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 x = *(const float4*)&s.T[K][r][4 * q];
    tl[4 * q] = x.x; tl[4 * q + 1] = x.y; tl[4 * q + 2] = x.z; tl[4 * q + 3] = x.w;
  }
  float y[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = (r == 16 * K + h + 4 * i) ? 1.f : 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int jr = 16 * K + j;
    const float vm = r > jr ? tl[j] : 0.f;  // column j of the unit-lower factor, below its diagonal
    float m[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) m[i] = lane_value(y[i], jr);  // row jr of the columns h + 4i: 1 on its own diagonal
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) y[i] = fmaf(-vm, m[i], y[i]);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (r >= 16 * K && r < 16 * K + 16) {
    const float rs = s.rs[r];
#pragma unroll
    for (int i = 0; i < 4; ++i) s.X[r][16 * K + h + 4 * i] = y[i] * rs;
  } else if (K < 3 && r >= 16 * K + 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) s.W[K < 3 ? K : 0][r][h + 4 * i] = y[i];
  }
}

// one 16 x 16 tile on the matrix cores: acc += A(16 x 4n) * B(4n x 16), A[i][k] at A + i * lda + k scaled by
// ascale[k] when given and negated when NEG, B[k][c] at B + k * ldb + c, all in LDS.  Result layout: lane l holds
// column l % 16, rows 4 * (l / 16) + v.
template <int N4, bool NEG>
__device__ __forceinline__ v4f tile16(v4f acc, const float* A, int lda, const float* B, int ldb, int lane,
                                      const float* ascale = nullptr) {
  const int i = lane & 15, g = lane >> 4;
#pragma unroll
  for (int kk = 0; kk < N4; ++kk) {
    float av = A[i * lda + 4 * kk + g];
    if (ascale) av *= ascale[4 * kk + g];
    const float bv = B[(4 * kk + g) * ldb + i];
    if (NEG) av = -av;
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc, 0, 0, 0);
  }
  return acc;
}

// s.AT holds the 64 x 64 block to factor, column-major (its lower triangle incl. the diagonal is used; the caller
// passes a barrier after writing it)  ->  s.X = inverse of its lower Cholesky factor, exact zeros above the
// diagonal.  Every thread of the 512 calls it.  Returns, in every thread, the smallest column whose pivot was not
// positive and finite (NB if none; the numbers computed after such a pivot are meaningless).  Ends with a
// barrier: s.X is readable by all on return.
__device__ __forceinline__ int factor_invert_64(FactorScratch& s) {
  const int tid = threadIdx.x, w = tid >> 6, r = tid & 63;
  if (tid == 0) s.bad = NB;
  for (int i = tid; i < NB * LDD / 4; i += NT) ((float4*)&s.X[0][0])[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();

  if (w == 0) factor_slab<0>(r, s);
  __syncthreads();
  update_trailing<0>(r, w, s);
  __syncthreads();
  if (w == 1) factor_slab<1>(r, s);
  if (w >= 4) invert_slab<0>(r, w - 4, s);
  __syncthreads();
  update_trailing<1>(r, w, s);
  __syncthreads();
  if (w == 2) factor_slab<2>(r, s);
  if (w >= 4) invert_slab<1>(r, w - 4, s);
  __syncthreads();
  update_trailing<2>(r, w, s);
  __syncthreads();
  if (w == 3) factor_slab<3>(r, s);
  if (w >= 4) invert_slab<2>(r, w - 4, s);
  __syncthreads();
  if (w >= 4) invert_slab<3>(r, w - 4, s);
  __syncthreads();

  float (*Z)[LDD] = s.AT;  // the block itself is no longer needed: rows 0..31 take -L21 X11 of the 32-wide step
  // ---- doubling, width 16: X[16.., 0..16) = X_11 W_0[16..32) (wave 0), X[48.., 32..48) = X_33 W_2[48..64) (wave 1)
  if (w < 2) {
    const int lo = 2 * w, hi = 2 * w + 1;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    acc = tile16<4, false>(acc, &s.X[16 * hi][16 * hi], LDD, &s.W[lo][16 * hi][0], LDP, r);
    const int c = r & 15, g = r >> 4;
#pragma unroll
    for (int v = 0; v < 4; ++v) s.X[16 * hi + 4 * g + v][16 * lo + c] = acc[v];
  }
  __syncthreads();
  // ---- width 32, first half: Z = -L21 X11 for rows 32..63: columns 16..31 are W_1 as it stands (waves 2, 3 copy
  // it), columns 0..15 are W_0 - L[32.., 16..32) X_10 (waves 0, 1: one 16-row tile each; L = V scaled by 1/sqrt(d)
  // of its column)
  if (w < 2) {
    const int c = r & 15, g = r >> 4;
    v4f acc;
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[v] = s.W[0][32 + 16 * w + 4 * g + v][c];
    acc = tile16<4, true>(acc, &s.V[1][32 + 16 * w][0], LDP, &s.X[16][0], LDD, r, &s.rs[16]);
#pragma unroll
    for (int v = 0; v < 4; ++v) Z[16 * w + 4 * g + v][c] = acc[v];
  } else if (w < 4) {
    const int row = (w - 2) * 16 + (r >> 2), q = r & 3;
    *(float4*)&Z[row][16 + 4 * q] = *(const float4*)&s.W[1][32 + row][4 * q];
  }
  __syncthreads();
  // ---- width 32, second half: X[32.., 0..32) = X22 Z, one 16 x 16 tile per wave 0..3 (X22 is lower triangular: the
  // upper tile row stops at 16)
  if (w < 4) {
    const int ti = w >> 1, tj = w & 1;
    const int c = r & 15, g = r >> 4;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    acc = tile16<4, false>(acc, &s.X[32 + 16 * ti][32], LDD, &Z[0][16 * tj], LDD, r);
    if (ti == 1) acc = tile16<4, false>(acc, &s.X[48][48], LDD, &Z[16][16 * tj], LDD, r);
#pragma unroll
    for (int v = 0; v < 4; ++v) s.X[32 + 16 * ti + 4 * g + v][16 * tj + c] = acc[v];
  }
  __syncthreads();
  return s.bad;
}

}  // namespace cholblk

// ---- 64 x 64 products on the matrix cores, for the kernels that keep a block row of the factorisation in one
// workgroup.  A 64 x 64 result is 16 tiles of 16 x 16; wave w of the eight owns the tiles (w / 2, 2 * (w % 2) + e),
// e = 0, 1.  Tile layout of v_mfma_f32_16x16x4_f32: lane l holds column l % 16, rows 4 * (l / 16) + v.
namespace cholblk {

struct Acc64 {
  v4f t[2];
};

// acc (+/-)= A * B^T with A and B row-major 64 x 64 blocks in LDS (row stride LDD).  The k index a lane group
// feeds into a matrix instruction is free as long as both operands agree, so lane group g takes k = 16 g .. 16 g + 15
// and reads its 16 values as four 16-byte loads.
template <bool NEG>
__device__ __forceinline__ void mm64_nt(Acc64& acc, const float (*A)[LDD], const float (*B)[LDD], int w, int lane) {
  const int i = lane & 15, g = lane >> 4, ti = w >> 1;
  float a[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 x = *(const float4*)&A[16 * ti + i][16 * g + 4 * q];
    a[4 * q] = NEG ? -x.x : x.x; a[4 * q + 1] = NEG ? -x.y : x.y; a[4 * q + 2] = NEG ? -x.z : x.z; a[4 * q + 3] = NEG ? -x.w : x.w;
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int tj = 2 * (w & 1) + e;
    float b[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 x = *(const float4*)&B[16 * tj + i][16 * g + 4 * q];
      b[4 * q] = x.x; b[4 * q + 1] = x.y; b[4 * q + 2] = x.z; b[4 * q + 3] = x.w;
    }
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) acc.t[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[kk], b[kk], acc.t[e], 0, 0, 0);
  }
}

// the wave's two tiles of a 64 x 64 block at `p` (row stride ld, global or LDS)
__device__ __forceinline__ void acc_load(Acc64& acc, const float* p, int64_t ld, int w, int lane) {
  const int i = lane & 15, g = lane >> 4, ti = w >> 1;
#pragma unroll
  for (int e = 0; e < 2; ++e)
#pragma unroll
    for (int v = 0; v < 4; ++v) acc.t[e][v] = p[(int64_t)(16 * ti + 4 * g + v) * ld + 16 * (2 * (w & 1) + e) + i];
}
__device__ __forceinline__ void acc_store(const Acc64& acc, float* p, int64_t ld, int w, int lane) {
  const int i = lane & 15, g = lane >> 4, ti = w >> 1;
#pragma unroll
  for (int e = 0; e < 2; ++e)
#pragma unroll
    for (int v = 0; v < 4; ++v) p[(int64_t)(16 * ti + 4 * g + v) * ld + 16 * (2 * (w & 1) + e) + i] = acc.t[e][v];
}

// a 64 x 64 block of a row-major global matrix through registers into a row-major LDS block: fetch() issues the
// loads (two 16-byte loads per thread), put() stores them, so that a product can run in between
struct BlockFetch {
  float4 v[2];
  __device__ __forceinline__ void fetch(const float* src, int64_t ld, int tid) {
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int idx = tid + NT * n;
      v[n] = *(const float4*)(src + (int64_t)(idx >> 4) * ld + (idx & 15) * 4);
    }
  }
  __device__ __forceinline__ void put(float (*dst)[LDD], int tid) const {
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int idx = tid + NT * n;
      *(float4*)&dst[idx >> 4][(idx & 15) * 4] = v[n];
    }
  }
};

}  // namespace cholblk
