// Damped Cholesky chain of GPTQ:  H -> U upper triangular with U^T U = (H + damp I)^-1.
//
// The reference factors H, inverts, and factors the inverse again.  U is the unique
// upper factor of H^-1 with positive diagonal, and it equals the inverse of the
// "reverse" Cholesky factor R of H (H = R R^T, R upper).  With J the exchange
// matrix, R = J L J for the ordinary lower factor L of J H J, so
//     U[i][j] = (L^-1)[K-1-i][K-1-j].
// This file therefore (1) copies J (P^T H P / n + damp I) J into a work matrix
// (P = optional activation-order permutation), (2) runs a blocked
// lower Cholesky (regions of 256 columns: 64-wide steps that factor and invert the
// diagonal block and solve the region's rows in one launch, one more launch for the
// rows below the region; the trailing update is a GEMM on the matrix cores),
// (3) inverts L by recursive doubling with batched triangular GEMMs and
// (4) writes the index-reversed result over H.  A non-positive pivot sets
// *info and the output becomes the identity (the reference's round-to-nearest
// fallback) without a host round trip.
#include <vector>

#include "chol_block.h"
#include "common.h"
#include "gemm_f32.h"

namespace {

constexpr int NB = 64;

struct HinvScalars {
  float damp;
  int info;
};

// One problem of a grouped call (llmc_gptq_hinv_grouped): the kernels below take an optional array of
// these and pick theirs by the workgroup index; the work matrices and scalars of problem b then sit at
// a fixed stride behind those of problem 0.
struct HinvItem {
  const float* H;
  const int32_t* perm;
  uint8_t* dead;
  float* U;
  float div;
  int pad;
};

// damp = percdamp * mean(diag(H')) where H' = H/div with zero diagonal entries replaced by 1;
// dead[c] = 1 where the (permuted) diagonal was zero
__global__ __launch_bounds__(256) void hinv_stats_kernel(const float* __restrict__ H, int64_t ldh, int K,
                                                         const int32_t* __restrict__ perm, float div,
                                                         float percdamp, uint8_t* __restrict__ dead,
                                                         HinvScalars* sc, const HinvItem* __restrict__ items) {
  if (items) {
    const HinvItem it = items[blockIdx.x];
    H = it.H; perm = it.perm; dead = it.dead; div = it.div;
    sc += blockIdx.x;
  }
  __shared__ double red[4];
  double sum = 0.0;
  for (int c = threadIdx.x; c < K; c += 256) {
    const int pc = perm ? perm[c] : c;
    float d = H[(int64_t)pc * ldh + pc] / div;
    const bool is_dead = d == 0.f;
    if (is_dead) d = 1.f;
    if (dead) dead[c] = is_dead ? 1 : 0;
    sum += (double)d;
  }
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float mean = (float)((red[0] + red[1] + red[2] + red[3]) / (double)K);
    sc->damp = percdamp * mean;
    sc->info = 0;
  }
}

// A[i][j] (Kp x Kp, lower incl. diagonal; zeros above) = H'[pi][pj], pi = perm[K-1-i]; identity padding
__global__ __launch_bounds__(256) void hinv_copyin_kernel(const float* __restrict__ H, int64_t ldh, int K,
                                                          int Kp, const int32_t* __restrict__ perm,
                                                          float div, const HinvScalars* __restrict__ sc,
                                                          float* __restrict__ A, const HinvItem* __restrict__ items) {
  if (items) {
    const HinvItem it = items[blockIdx.z];
    H = it.H; perm = it.perm; div = it.div;
    sc += blockIdx.z;
    A += (int64_t)blockIdx.z * Kp * Kp;
  }
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int i = blockIdx.y;
  if (j >= Kp) return;
  float v = 0.f;
  if (j <= i) {
    if (i >= K) {
      v = (i == j) ? 1.f : 0.f;
    } else {
      const int ri = K - 1 - i, rj = K - 1 - j;
      const int pi = perm ? perm[ri] : ri, pj = perm ? perm[rj] : rj;
      v = H[(int64_t)pi * ldh + pj] / div;
      if (i == j) {
        if (v == 0.f) v = 1.f;
        v += sc->damp;
      }
    }
  }
  A[(int64_t)i * Kp + j] = v;
}

// hinv_copyin_kernel for a permuted order, one workgroup per row of A: row perm[K-1-i] of H is read whole and
// coalesced into LDS and the permuted columns are picked there (element-wise the gather costs one cache line
// per value).  Rows of up to COPYIN_STAGE_MAX values.
constexpr int COPYIN_STAGE_MAX = 16384;
// Launched with 256 threads per row, or with 1024 for rows of more than 8192 values: a row of 14336 floats takes
// 56 KB of LDS, two workgroups fit a CU, and with 256 threads each the CU would hold 8 waves' worth of loads.
__global__ __launch_bounds__(1024) void hinv_copyin_rows_kernel(const float* __restrict__ H, int64_t ldh, int K,
                                                               int Kp, const int32_t* __restrict__ perm, float div,
                                                               const HinvScalars* __restrict__ sc,
                                                               float* __restrict__ A,
                                                               const HinvItem* __restrict__ items) {
  extern __shared__ float rowbuf[];
  if (items) {
    const HinvItem it = items[blockIdx.y];
    H = it.H; perm = it.perm; div = it.div;
    sc += blockIdx.y;
    A += (int64_t)blockIdx.y * Kp * Kp;
  }
  const int i = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  float* out = A + (int64_t)i * Kp;
  if (i >= K) {  // identity padding
    for (int j = tid; j < Kp; j += nt) out[j] = (i == j) ? 1.f : 0.f;
    return;
  }
  const float* src = H + (int64_t)perm[K - 1 - i] * ldh;
  constexpr int BATCH = 8;
  for (int c0 = 0; c0 < K; c0 += nt * BATCH) {
    float v[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      v[b] = src[c < K ? c : K - 1];
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      if (c < K) rowbuf[c] = v[b];
    }
  }
  __syncthreads();
  const float damp = sc->damp;
  for (int j = tid; j < Kp; j += nt) {
    float v = 0.f;
    if (j <= i) {
      v = rowbuf[perm[K - 1 - j]] / div;
      if (i == j) {
        if (v == 0.f) v = 1.f;
        v += damp;
      }
    }
    out[j] = v;
  }
}

// ---- a 256-wide region of the factorisation in two kinds of launches -------------------------------------------
// The serial spine of the blocked factorisation is one 64 x 64 diagonal block after the other.  Inside a region
// of up to four such blocks, step m is ONE launch (chol_region_step_kernel): every workgroup factors and inverts
// the diagonal block m itself (the same arithmetic in each, so nothing has to cross workgroups), and workgroup
// b > 0 then solves its own 64 rows of block column m against it, after bringing them up to date with the
// region's earlier steps, and takes the new columns' contribution off its own diagonal block -- so that block
// is complete when its turn comes.  The rows below the region are not on the spine: they are solved against
// the whole region afterwards, one launch (chol_region_rows_kernel), 64 rows per workgroup, the block row kept
// in LDS from one block column to the next.
//
// The inverses of the diagonal blocks' factors go to a side array Xs (block c0 / 64 at Xs + (c0 / 64) * 4096, dense
// 64 x 64) and not over the diagonal block itself: within one launch every workgroup reads that block, whenever it
// happens to start, so nothing may overwrite it before the launch has ended.  chol_scatter_diag_kernel moves them
// into the diagonal blocks once the factorisation is complete (where the inversion expects them).
struct RegionStepLds {
  cholblk::FactorScratch fs;
  float Abuf[NB][cholblk::LDD];
  float Bbuf[NB][cholblk::LDD];
};

__global__ __launch_bounds__(cholblk::NT) void chol_region_step_kernel(float* __restrict__ A, int Kp, int r0, int m,
                                                                       int K, HinvScalars* sc, float* __restrict__ Xs,
                                                                       int64_t xs_stride) {
  using namespace cholblk;
  A += (int64_t)blockIdx.y * Kp * Kp;  // grouped call: blockIdx.y = problem
  Xs += (int64_t)blockIdx.y * xs_stride;
  sc += blockIdx.y;
  extern __shared__ __attribute__((aligned(16))) unsigned char region_smem[];
  RegionStepLds& L = *(RegionStepLds*)region_smem;
  const int tid = threadIdx.x, w = tid >> 6, r = tid & 63;
  const int b = blockIdx.x;                // 0: owner of the diagonal block; b > 0: row block m + b of the region
  const int c0 = r0 + NB * m;              // the step's block column
  const int64_t rows = c0 + (int64_t)NB * b;
  // the diagonal block's loads are issued first: their latency hides behind the products below
  const float* dsrc = A + (int64_t)(c0 + r) * Kp + c0 + 8 * w;
  const float4 d0 = *(const float4*)dsrc, d1 = *(const float4*)(dsrc + 4);
  Acc64 acc, dg;
  if (b > 0) {
    // own rows of block column m, brought up to date with the region's earlier steps:
    // acc = A[rows, c0..] - sum_{i<m} A[rows, cols_i] A[c0 rows, cols_i]^T
    acc_load(acc, A + rows * Kp + c0, Kp, w, r);
    acc_load(dg, A + rows * Kp + rows, Kp, w, r);  // this row block's own diagonal block, needed at the very end
    for (int i = 0; i < m; ++i) {
      BlockFetch fa, fb;
      fa.fetch(A + rows * Kp + r0 + NB * i, Kp, tid);
      fb.fetch(A + (int64_t)c0 * Kp + r0 + NB * i, Kp, tid);
      if (i > 0) __syncthreads();  // the previous product has read the buffers
      fa.put(L.Abuf, tid);
      fb.put(L.Bbuf, tid);
      __syncthreads();
      mm64_nt<true>(acc, L.Abuf, L.Bbuf, w, r);
    }
  }
  L.fs.AT[8 * w + 0][r] = d0.x; L.fs.AT[8 * w + 1][r] = d0.y; L.fs.AT[8 * w + 2][r] = d0.z; L.fs.AT[8 * w + 3][r] = d0.w;
  L.fs.AT[8 * w + 4][r] = d1.x; L.fs.AT[8 * w + 5][r] = d1.y; L.fs.AT[8 * w + 6][r] = d1.z; L.fs.AT[8 * w + 7][r] = d1.w;
  __syncthreads();
  const int bad = factor_invert_64(L.fs);
  if (b == 0) {
    // first failing pivot, 1-based index in the ORIGINAL (un-reversed) ordering
    if (tid == 0 && bad < NB && c0 + bad < K) atomicCAS(&sc->info, 0, K - (c0 + bad));
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int idx = tid + NT * n, row = idx >> 4, c4 = (idx & 15) * 4;
      *(float4*)(Xs + (int64_t)(c0 / NB) * NB * NB + row * NB + c4) = *(const float4*)&L.fs.X[row][c4];
    }
    return;
  }
  // solve: R = acc * inv(L_mm)^T  (the barriers inside the factorisation separate this from the last product)
  acc_store(acc, &L.Abuf[0][0], LDD, w, r);
  __syncthreads();
  Acc64 sol = {};
  mm64_nt<false>(sol, L.Abuf, L.fs.X, w, r);
  acc_store(sol, A + rows * Kp + c0, Kp, w, r);
  __syncthreads();  // every wave has read Abuf
  acc_store(sol, &L.Abuf[0][0], LDD, w, r);
  // the new columns' contribution to this row block's own diagonal block: D_b -= R R^T
  __syncthreads();
  mm64_nt<true>(dg, L.Abuf, L.Abuf, w, r);
  acc_store(dg, A + rows * Kp + rows, Kp, w, r);
}

struct RegionRowsLds {
  float R[4][NB][cholblk::LDD];  // the workgroup's solved blocks of the region's block columns
  float Abuf[NB][cholblk::LDD];
  float Bbuf[NB][cholblk::LDD];
};

// rows row_start + 64 * blockIdx.x .. of the nb block columns of the region at r0, whose diagonal region is done
__global__ __launch_bounds__(cholblk::NT) void chol_region_rows_kernel(float* __restrict__ A, int Kp, int r0, int nb,
                                                                       int row_start, const float* __restrict__ Xs,
                                                                       int64_t xs_stride) {
  using namespace cholblk;
  A += (int64_t)blockIdx.y * Kp * Kp;
  Xs += (int64_t)blockIdx.y * xs_stride;
  extern __shared__ __attribute__((aligned(16))) unsigned char rows_smem[];
  RegionRowsLds& L = *(RegionRowsLds*)rows_smem;
  const int tid = threadIdx.x, w = tid >> 6, r = tid & 63;
  const int64_t rows = row_start + (int64_t)NB * blockIdx.x;
  // schedule: for block column j the factor blocks (j, 0) .. (j, j-1) at A[r0 + 64 j rows, r0 + 64 i columns], then
  // the inverse of the diagonal block's factor from the side array.  One block ahead is in flight while the current
  // product runs.
  const float* xs0 = Xs + (int64_t)(r0 / NB) * NB * NB;
  BlockFetch next;
  next.fetch(xs0, NB, tid);
  Acc64 own[4];  // the workgroup's rows of the region's block columns: all loads in flight from the start
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (j < nb) acc_load(own[j], A + rows * Kp + r0 + NB * j, Kp, w, r);
  bool first = true;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (j >= nb) break;
    Acc64 acc = own[j];
    for (int i = 0; i <= j; ++i) {
      if (!first) __syncthreads();  // the previous product has read Bbuf (and Abuf)
      first = false;
      next.put(L.Bbuf, tid);
      {  // the block after this one
        int nj = j, ni = i + 1;
        if (ni > nj) { nj = j + 1; ni = 0; }
        if (nj < nb) {
          if (ni == nj)
            next.fetch(xs0 + (int64_t)nj * NB * NB, NB, tid);
          else
            next.fetch(A + (int64_t)(r0 + NB * nj) * Kp + r0 + NB * ni, Kp, tid);
        }
      }
      if (i == j) acc_store(acc, &L.Abuf[0][0], LDD, w, r);
      __syncthreads();
      if (i < j) {
        mm64_nt<true>(acc, L.R[i], L.Bbuf, w, r);
      } else {
        Acc64 sol = {};
        mm64_nt<false>(sol, L.Abuf, L.Bbuf, w, r);
        acc_store(sol, A + rows * Kp + r0 + NB * j, Kp, w, r);
        acc_store(sol, &L.R[j][0][0], LDD, w, r);  // read by later products, after the barriers in between
      }
    }
  }
}

// diagonal block c of the work matrix <- Xs block c (after the factorisation, before the inversion)
__global__ __launch_bounds__(256) void chol_scatter_diag_kernel(float* __restrict__ A, int Kp, const float* __restrict__ Xs,
                                                                int64_t xs_stride) {
  A += (int64_t)blockIdx.y * Kp * Kp;
  Xs += (int64_t)blockIdx.y * xs_stride + (int64_t)blockIdx.x * NB * NB;
  const int c0 = blockIdx.x * NB;
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const int idx = threadIdx.x + 256 * n, row = idx >> 4, c4 = (idx & 15) * 4;
    *(float4*)(A + (int64_t)(c0 + row) * Kp + c0 + c4) = *(const float4*)(Xs + row * NB + c4);
  }
}

template <typename KernelT>
inline int set_dynamic_lds(KernelT kernel, size_t bytes) {
  const hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  return e == hipSuccess ? 0 : 1000 + (int)e;
}

// U[i][j] = X[K-1-i][K-1-j] for j >= i, 0 below; identity when the factorisation failed.  Four columns per
// thread: a row of U is a row of X read backwards, so four neighbours of U are four neighbours of X.
__global__ __launch_bounds__(256) void hinv_copyout_kernel(const float* __restrict__ X, int Kp, int K,
                                                           const HinvScalars* __restrict__ sc,
                                                           float* __restrict__ U, int64_t ldu,
                                                           int32_t* __restrict__ info_out,
                                                           const HinvItem* __restrict__ items) {
  if (items) {
    U = items[blockIdx.z].U;
    sc += blockIdx.z;
    X += (int64_t)blockIdx.z * Kp * Kp;
    if (info_out) info_out += blockIdx.z;
  }
  const int j0 = (blockIdx.x * 256 + threadIdx.x) * 4;
  const int i = blockIdx.y;
  if (i == 0 && j0 == 0 && info_out) *info_out = sc->info;
  if (j0 >= K) return;
  const bool failed = sc->info != 0;
  const float* xrow = X + (int64_t)(K - 1 - i) * Kp;
  float* urow = U + (int64_t)i * ldu;
  const bool vec = j0 + 3 < K && (K & 3) == 0 && (ldu & 3) == 0 && (((uintptr_t)U | (uintptr_t)X) & 15) == 0;
  if (vec && !failed && j0 >= i) {  // four values of X at K-4-j0 .. K-1-j0, reversed
    const float4 x = *(const float4*)(xrow + (K - 4 - j0));
    *(float4*)(urow + j0) = make_float4(x.w, x.z, x.y, x.x);
    return;
  }
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int j = j0 + e;
    v[e] = 0.f;
    if (j < K) {
      if (failed)
        v[e] = (i == j) ? 1.f : 0.f;
      else if (j >= i)
        v[e] = xrow[K - 1 - j];
    }
  }
  if (vec) {
    *(float4*)(urow + j0) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (j0 + e < K) urow[j0 + e] = v[e];
  }
}

inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

// floats of the temporary behind a work matrix: the inversion's first products (Kp^2 / 4) and, before that, the
// side array of the diagonal blocks' inverses (64 Kp)
inline int64_t hinv_temp_floats(int64_t Kp) { return Kp * Kp / 4 > NB * Kp ? Kp * Kp / 4 : NB * Kp; }

// Blocked lower Cholesky of n work matrices (one every Kp^2 floats) in lock-step; Xs (one every xs_stride floats) takes
// the inverses of the diagonal blocks' factors and is moved into the diagonal blocks at the end.
//
// Two levels.  An outer panel (512 wide once the trailing matrix is big enough to pay for it, else 256) ends with one
// rank-256/512 update of the trailing matrix, which cuts that matrix's read-modify-write traffic 4-8x compared with
// rank-64 updates.  Inside it, regions of 256 columns: four single-launch steps on the diagonal region, one launch for
// the rows below it (see chol_region_step_kernel); the second region of a 512-wide panel first takes the first
// region's update as one product.
inline int chol_factor(float* A, int Kp, int K, HinvScalars* sc, float* Xs, int64_t xs_stride, int n, hipStream_t st) {
  static const int cfg_step = set_dynamic_lds(chol_region_step_kernel, sizeof(RegionStepLds));
  static const int cfg_rows = set_dynamic_lds(chol_region_rows_kernel, sizeof(RegionRowsLds));
  if (cfg_step) return cfg_step;
  if (cfg_rows) return cfg_rows;
  const int64_t mat = (int64_t)Kp * Kp;
  const int NBO = Kp >= 8192 ? 512 : 256;
  constexpr int RW = 256;
  for (int k0 = 0; k0 < Kp; k0 += NBO) {
    const int pw = (Kp - k0) < NBO ? (Kp - k0) : NBO;
    for (int r0 = k0; r0 < k0 + pw; r0 += RW) {
      const int rw = (k0 + pw - r0) < RW ? (k0 + pw - r0) : RW;
      const int nb = rw / NB;
      if (r0 > k0) {
        // columns r0 .. r0+rw of the rows from r0 down take the panel's first region in one product,
        // C[M, rw] -= L[rows, k0:r0] L[r0:r0+rw, k0:r0]^T, lower part only (C starts on the matrix diagonal)
        float* Lp = A + (int64_t)r0 * Kp + k0;
        GemmF32 u = {};
        u.A = Lp; u.lda = Kp; u.B = Lp; u.ldb = Kp; u.C = A + (int64_t)r0 * Kp + r0; u.ldc = Kp;
        u.M = Kp - r0; u.N = rw; u.Kc = r0 - k0; u.alpha = -1.f; u.beta = 1.f; u.trans_b = 1; u.c_lower = 1;
        u.batch = 1; u.batch2 = n; u.stride2_a = mat; u.stride2_b = mat; u.stride2_c = mat;
        const int rc = llmc_gemm_f32(u, st);
        if (rc) return rc;
      }
      for (int m = 0; m < nb; ++m) {
        hipLaunchKernelGGL(chol_region_step_kernel, dim3(nb - m, n), dim3(cholblk::NT), sizeof(RegionStepLds), st, A, Kp,
                           r0, m, K, sc, Xs, xs_stride);
        LLMC_LAUNCH_STATUS();
      }
      const int below = (Kp - (r0 + rw)) / NB;
      if (below > 0) {
        hipLaunchKernelGGL(chol_region_rows_kernel, dim3(below, n), dim3(cholblk::NT), sizeof(RegionRowsLds), st, A, Kp,
                           r0, nb, r0 + rw, (const float*)Xs, xs_stride);
        LLMC_LAUNCH_STATUS();
      }
    }
    const int M2 = Kp - (k0 + pw);
    if (M2 > 0) {
      float* P = A + (int64_t)(k0 + pw) * Kp + k0;
      GemmF32 t = {};
      t.A = P; t.lda = Kp; t.B = P; t.ldb = Kp; t.C = A + (int64_t)(k0 + pw) * ((int64_t)Kp + 1); t.ldc = Kp;
      t.M = M2; t.N = M2; t.Kc = pw; t.alpha = -1.f; t.beta = 1.f; t.trans_b = 1; t.c_lower = 1;
      t.batch = 1; t.batch2 = n; t.stride2_a = mat; t.stride2_b = mat; t.stride2_c = mat;
      const int rc = llmc_gemm_f32(t, st);
      if (rc) return rc;
    }
  }
  hipLaunchKernelGGL(chol_scatter_diag_kernel, dim3(Kp / NB, n), dim3(256), 0, st, A, Kp, (const float*)Xs, xs_stride);
  LLMC_LAUNCH_STATUS();
  return 0;
}

}  // namespace

namespace {
// ---- activation order: argsort of the Hessian's diagonal, descending, equal entries in index order -------------
// (gptq_quantize.py:131-140 sorts diag(H) with torch.argsort; a stable sort is what keeps equal entries in column
// order.)  One workgroup per Hessian: the diagonal and the column numbers sit in LDS, padded to a power of two
// with entries that sort last, and a bitonic network orders them by (value descending, index ascending) -- a total
// order, so the network's result is the stable sort's.  NaN sorts before every number, as in torch; the two zeros
// compare equal.
constexpr int ORDER_MAX_K = 16384;
constexpr int ORDER_MAX_PROBLEMS = 256;
struct OrderArgs {
  const float* H[ORDER_MAX_PROBLEMS];
};

// (value, index) as one 64-bit key whose ascending order is "value descending, index ascending": the float's bits
// are mapped to an unsigned that grows with the value (both zeros to one key, every NaN to one key above +inf),
// complemented, and the index goes into the low half.
__device__ __forceinline__ unsigned long long order_key(float v, int i) {
  uint32_t u = __float_as_uint(v);
  if (v != v) u = 0x7fc00000u;          // one NaN
  if ((u << 1) == 0u) u = 0u;           // -0 -> +0
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ((unsigned long long)(~u) << 32) | (unsigned)i;
}

__global__ __launch_bounds__(1024) void diag_order_kernel(OrderArgs args, int64_t ldh, int K, int N,
                                                          int64_t* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char order_smem[];
  unsigned long long* key = (unsigned long long*)order_smem;
  const float* H = args.H[blockIdx.x];
  const int tid = threadIdx.x;
  for (int i = tid; i < N; i += 1024) key[i] = i < K ? order_key(H[(int64_t)i * ldh + i], i) : ~0ull;
  __syncthreads();
  for (int k = 2; k <= N; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < N / 2; t += 1024) {
        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));  // the element of the pair with bit j clear
        const int p = i | j;
        const bool up = (i & k) == 0;  // this run ends up in order (first element first)
        const unsigned long long a = key[i], b = key[p];
        if ((a < b) != up) {
          key[i] = b;
          key[p] = a;
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < K; i += 1024) out[(int64_t)blockIdx.x * K + i] = (int64_t)(key[i] & 0xffffffffull);
}
}  // namespace

extern "C" int llmc_diag_argsort_desc(const float* const* H, int64_t ldh, int32_t n, int64_t K, int64_t* out,
                                      void* stream) {
  LLMC_CHECK_ARG(H != nullptr && out != nullptr, 1);
  LLMC_CHECK_ARG(n >= 0 && K > 0 && K <= ORDER_MAX_K && ldh >= K, 3);
  int N = 2;
  while (N < K) N <<= 1;
  const size_t smem = (size_t)N * 8;
  static const hipError_t configured = hipFuncSetAttribute(
      (const void*)diag_order_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ORDER_MAX_K * 8);
  if (configured != hipSuccess) return 1000 + (int)configured;
  for (int first = 0; first < n; first += ORDER_MAX_PROBLEMS) {
    const int m = n - first < ORDER_MAX_PROBLEMS ? n - first : ORDER_MAX_PROBLEMS;
    OrderArgs args;
    for (int b = 0; b < m; ++b) {
      LLMC_CHECK_ARG(H[first + b] != nullptr, 1);
      args.H[b] = H[first + b];
    }
    hipLaunchKernelGGL(diag_order_kernel, dim3((unsigned)m), dim3(1024), smem, (hipStream_t)stream, args, ldh, (int)K,
                       N, out + (int64_t)first * K);
    LLMC_LAUNCH_STATUS();
  }
  return 0;
}

extern "C" int64_t llmc_gptq_hinv_workspace_bytes(int64_t K) {
  const int64_t Kp = round_up(K, NB);
  // work matrix + temporary (recursive doubling, side array of the diagonal inverses) + scalars
  return (Kp * Kp + hinv_temp_floats(Kp) + 64) * 4 + 256;
}

// Width up to which the inverse of the factor is formed: everything for LLMC_FACTOR_INVERSE, 512-wide diagonal
// blocks for LLMC_FACTOR_GROUPS (the recursive doubling stops there, which leaves the Cholesky factor itself outside
// those blocks).  The work matrix is in reversed index order, so the blocks start at multiples of 512 counted from
// the LAST column: [K - 512, K), [K - 1024, K - 512), ... and a first block of the K % 512 columns that are left
// (K must be a multiple of 128, so that the work matrix has no padding and the column loop's 128-column blocks do
// not straddle two of them).
inline int64_t inverse_width(int32_t form, int64_t Kp) { return form == LLMC_FACTOR_GROUPS ? LLMC_FACTOR_GROUP_WIDTH : Kp; }

// The chain saves the part of the triangular inverse that crosses blocks (a third of its arithmetic, growing with
// K^3: 0.6 ms at K = 4096, 7.3 ms at 14336), the column loop pays three more launches and one 512-wide product per
// group (0.06 - 0.1 ms per group, growing with K): from 8192 columns on the first outweighs the second for every
// number of rows; at 4096 columns the two cancel.
constexpr int64_t FACTOR_GROUPS_MIN_K = 8192;

extern "C" int32_t llmc_gptq_factor_form(int64_t K, int32_t blocksize) {
  return (K % 128 == 0 && K >= FACTOR_GROUPS_MIN_K && blocksize >= 128) ? LLMC_FACTOR_GROUPS : LLMC_FACTOR_INVERSE;
}

extern "C" int llmc_gptq_hinv(float* H, int64_t ldh, int64_t K, const int32_t* perm, float divisor,
                              float percdamp, int32_t form, uint8_t* dead_out, void* workspace,
                              int64_t workspace_bytes, int32_t* info_out, void* stream) {
  LLMC_CHECK_ARG(H != nullptr, 1);
  LLMC_CHECK_ARG(form == LLMC_FACTOR_INVERSE || (form == LLMC_FACTOR_GROUPS && K % 128 == 0), 7);
  LLMC_CHECK_ARG(ldh >= K, 2);
  LLMC_CHECK_ARG(K > 0 && K <= 65536, 3);
  LLMC_CHECK_ARG(divisor != 0.f, 5);
  LLMC_CHECK_ARG(workspace != nullptr && (((uintptr_t)workspace) & 255) == 0, 8);
  LLMC_CHECK_ARG(workspace_bytes >= llmc_gptq_hinv_workspace_bytes(K), 9);
  hipStream_t st = (hipStream_t)stream;
  const int Kp = (int)round_up(K, NB);
  HinvScalars* sc = (HinvScalars*)workspace;
  float* A = (float*)((char*)workspace + 256);
  float* T = A + (int64_t)Kp * Kp;

  hipLaunchKernelGGL(hinv_stats_kernel, dim3(1), dim3(256), 0, st, H, ldh, (int)K, perm, divisor, percdamp,
                     dead_out, sc, (const HinvItem*)nullptr);
  LLMC_LAUNCH_STATUS();
  if (perm != nullptr && K <= COPYIN_STAGE_MAX) {
    if (K * 4 > 48 * 1024) {
      const hipError_t e = hipFuncSetAttribute((const void*)hinv_copyin_rows_kernel,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)K * 4);
      if (e != hipSuccess) return 1000 + (int)e;
    }
    hipLaunchKernelGGL(hinv_copyin_rows_kernel, dim3(Kp), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4, st, H, ldh, (int)K, Kp, perm,
                       divisor, sc, A, (const HinvItem*)nullptr);
  } else {
    hipLaunchKernelGGL(hinv_copyin_kernel, dim3((Kp + 255) / 256, Kp), dim3(256), 0, st, H, ldh, (int)K, Kp, perm,
                       divisor, sc, A, (const HinvItem*)nullptr);
  }
  LLMC_LAUNCH_STATUS();

  {
    const int frc = chol_factor(A, Kp, (int)K, sc, T, 0, 1, st);
    if (frc) return frc;
  }

  // inverse by recursive doubling: [[X11,0],[X21,X22]] with X21 = -X22 * L21 * X11
  for (int64_t s = NB; s < inverse_width(form, Kp); s *= 2) {
    const int64_t full = Kp / (2 * s);
    const int64_t rem = Kp % (2 * s);
    const int64_t step = 2 * s * ((int64_t)Kp + 1);
    for (int part = 0; part < 2; ++part) {
      int64_t base, s2, batch;
      if (part == 0) {
        base = 0; s2 = s; batch = full;
      } else {
        base = full * 2 * s; s2 = rem - s; batch = 1;
      }
      if (batch <= 0 || s2 <= 0) continue;
      float* X11 = A + base * ((int64_t)Kp + 1);
      float* X22 = X11 + s * ((int64_t)Kp + 1);
      float* L21 = X11 + s * (int64_t)Kp;
      GemmF32 g = {};
      g.A = L21; g.lda = Kp; g.B = X11; g.ldb = Kp; g.C = T; g.ldc = s;
      g.M = (int)s2; g.N = (int)s; g.Kc = (int)s; g.alpha = 1.f; g.beta = 0.f; g.b_lower_tri = 1;
      g.batch = (int)batch; g.stride_a = step; g.stride_b = step; g.stride_c = s * s;
      int rc = llmc_gemm_f32(g, st);
      if (rc) return rc;
      GemmF32 h = {};
      h.A = X22; h.lda = Kp; h.B = T; h.ldb = s; h.C = L21; h.ldc = Kp;
      h.M = (int)s2; h.N = (int)s; h.Kc = (int)s2; h.alpha = -1.f; h.beta = 0.f; h.a_lower_tri = 1;
      h.batch = (int)batch; h.stride_a = step; h.stride_b = s * s; h.stride_c = step;
      rc = llmc_gemm_f32(h, st);
      if (rc) return rc;
    }
  }

  hipLaunchKernelGGL(hinv_copyout_kernel, dim3((unsigned)((K + 1023) / 1024), (unsigned)K), dim3(256), 0, st, A, Kp,
                     (int)K, sc, H, ldh, info_out, (const HinvItem*)nullptr);
  LLMC_LAUNCH_STATUS();
  return 0;
}

// ---- grouped form: n independent problems of one width in lock-step ---------------------------------
// The chain of a small Hessian (an MoE expert's: K = 768 or 2048) is a run of tiny kernels that uses a few
// CUs for microseconds each; run for 128 experts one after the other, the chip idles.  Here every kernel of
// the chain is launched once for all problems (one more grid dimension / GEMM batch level), so the chain is
// as long as a single problem's while each launch carries n times the work.

extern "C" int64_t llmc_gptq_hinv_grouped_workspace_bytes(int64_t n, int64_t K) {
  const int64_t Kp = round_up(K, NB);
  return round_up(n * (int64_t)sizeof(HinvItem), 256) + round_up(n * (int64_t)sizeof(HinvScalars), 256) +
         n * (Kp * Kp + hinv_temp_floats(Kp)) * 4 + 256;
}

extern "C" int llmc_gptq_hinv_grouped(const float* const* H, int64_t ldh, int32_t n, int64_t K,
                                      const int32_t* const* perm, const float* divisors, float percdamp,
                                      int32_t form, uint8_t* dead_out, float* U_out, int64_t ldu, void* workspace,
                                      int64_t workspace_bytes, int32_t* info_out, void* stream) {
  LLMC_CHECK_ARG(H != nullptr && ldh >= K, 1);
  LLMC_CHECK_ARG(form == LLMC_FACTOR_INVERSE || (form == LLMC_FACTOR_GROUPS && K % 128 == 0), 8);
  LLMC_CHECK_ARG(n >= 0 && n <= 4096, 3);
  if (n == 0) return 0;
  LLMC_CHECK_ARG(K > 0 && K <= 65536, 4);
  LLMC_CHECK_ARG(divisors != nullptr, 6);
  LLMC_CHECK_ARG(U_out != nullptr && ldu >= K, 9);
  LLMC_CHECK_ARG(workspace != nullptr && (((uintptr_t)workspace) & 255) == 0, 11);
  LLMC_CHECK_ARG(workspace_bytes >= llmc_gptq_hinv_grouped_workspace_bytes(n, K), 12);
  hipStream_t st = (hipStream_t)stream;
  const int Kp = (int)round_up(K, NB);
  const int64_t mat = (int64_t)Kp * Kp;
  LLMC_CHECK_ARG((int64_t)n * (Kp / 128 + 1) < 65535, 3);  // deepest GEMM batch in one grid dimension

  char* wp = (char*)workspace;
  HinvItem* items = (HinvItem*)wp; wp += round_up(n * (int64_t)sizeof(HinvItem), 256);
  HinvScalars* sc = (HinvScalars*)wp; wp += round_up(n * (int64_t)sizeof(HinvScalars), 256);
  float* A = (float*)wp;
  float* T = A + (int64_t)n * mat;
  const int64_t tstride = hinv_temp_floats(Kp);
  std::vector<HinvItem> host(n);
  for (int b = 0; b < n; ++b) {
    LLMC_CHECK_ARG(H[b] != nullptr && divisors[b] != 0.f, 1);
    host[b].H = H[b];
    host[b].perm = perm ? perm[b] : nullptr;
    host[b].dead = dead_out ? dead_out + (int64_t)b * K : nullptr;
    host[b].U = U_out + (int64_t)b * K * ldu;
    host[b].div = divisors[b];
    host[b].pad = 0;
  }
  {
    const int urc = upload_items(host.data(), n, (HinvItem*)items, st);
    if (urc) return urc;
  }

  hipLaunchKernelGGL(hinv_stats_kernel, dim3(n), dim3(256), 0, st, (const float*)nullptr, ldh, (int)K,
                     (const int32_t*)nullptr, 1.f, percdamp, (uint8_t*)nullptr, sc, (const HinvItem*)items);
  LLMC_LAUNCH_STATUS();
  bool all_perm = perm != nullptr;
  for (int b = 0; b < n && all_perm; ++b) all_perm = perm[b] != nullptr;
  if (all_perm && K <= COPYIN_STAGE_MAX) {
    if (K * 4 > 48 * 1024) {
      const hipError_t e = hipFuncSetAttribute((const void*)hinv_copyin_rows_kernel,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)K * 4);
      if (e != hipSuccess) return 1000 + (int)e;
    }
    hipLaunchKernelGGL(hinv_copyin_rows_kernel, dim3(Kp, n), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4, st, (const float*)nullptr, ldh,
                       (int)K, Kp, (const int32_t*)nullptr, 1.f, sc, A, (const HinvItem*)items);
  } else {
    hipLaunchKernelGGL(hinv_copyin_kernel, dim3((Kp + 255) / 256, Kp, n), dim3(256), 0, st, (const float*)nullptr, ldh,
                       (int)K, Kp, (const int32_t*)nullptr, 1.f, sc, A, (const HinvItem*)items);
  }
  LLMC_LAUNCH_STATUS();

  {
    const int frc = chol_factor(A, Kp, (int)K, sc, T, tstride, n, st);
    if (frc) return frc;
  }

  for (int64_t s = NB; s < inverse_width(form, Kp); s *= 2) {
    const int64_t full = Kp / (2 * s);
    const int64_t rem = Kp % (2 * s);
    const int64_t step = 2 * s * ((int64_t)Kp + 1);
    for (int part = 0; part < 2; ++part) {
      int64_t base, s2, batch;
      if (part == 0) {
        base = 0; s2 = s; batch = full;
      } else {
        base = full * 2 * s; s2 = rem - s; batch = 1;
      }
      if (batch <= 0 || s2 <= 0) continue;
      float* X11 = A + base * ((int64_t)Kp + 1);
      float* X22 = X11 + s * ((int64_t)Kp + 1);
      float* L21 = X11 + s * (int64_t)Kp;
      GemmF32 g = {};
      g.A = L21; g.lda = Kp; g.B = X11; g.ldb = Kp; g.C = T; g.ldc = s;
      g.M = (int)s2; g.N = (int)s; g.Kc = (int)s; g.alpha = 1.f; g.beta = 0.f; g.b_lower_tri = 1;
      g.batch = (int)batch; g.stride_a = step; g.stride_b = step; g.stride_c = s * s;
      g.batch2 = n; g.stride2_a = mat; g.stride2_b = mat; g.stride2_c = tstride;
      int rc = llmc_gemm_f32(g, st);
      if (rc) return rc;
      GemmF32 h = {};
      h.A = X22; h.lda = Kp; h.B = T; h.ldb = s; h.C = L21; h.ldc = Kp;
      h.M = (int)s2; h.N = (int)s; h.Kc = (int)s2; h.alpha = -1.f; h.beta = 0.f; h.a_lower_tri = 1;
      h.batch = (int)batch; h.stride_a = step; h.stride_b = s * s; h.stride_c = step;
      h.batch2 = n; h.stride2_a = mat; h.stride2_b = tstride; h.stride2_c = mat;
      rc = llmc_gemm_f32(h, st);
      if (rc) return rc;
    }
  }

  hipLaunchKernelGGL(hinv_copyout_kernel, dim3((unsigned)((K + 1023) / 1024), (unsigned)K, (unsigned)n), dim3(256), 0, st,
                     A, Kp, (int)K, sc, (float*)nullptr, ldu, info_out, (const HinvItem*)items);
  LLMC_LAUNCH_STATUS();
  return 0;
}
