// Damped Cholesky chain of GPTQ:  H -> U upper triangular with U^T U = (H + damp I)^-1.
//
// The reference factors H, inverts, and factors the inverse again.  U is the unique
// upper factor of H^-1 with positive diagonal, and it equals the inverse of the
// "reverse" Cholesky factor R of H (H = R R^T, R upper).  With J the exchange
// matrix, R = J L J for the ordinary lower factor L of J H J, so
//     U[i][j] = (L^-1)[K-1-i][K-1-j].
// This file therefore (1) copies J (P^T H P / n + damp I) J into a work matrix
// (P = optional activation-order permutation), (2) runs a right-looking blocked
// lower Cholesky (64-wide panels: the diagonal block is factored and inverted in
// LDS by one workgroup, panel solve and trailing update are MFMA GEMMs),
// (3) inverts L by recursive doubling with batched triangular GEMMs and
// (4) writes the index-reversed result over H.  A non-positive pivot sets
// *info and the output becomes the identity (the reference's round-to-nearest
// fallback) without a host round trip.
#include "common.h"
#include "gemm_f32.h"

namespace {

constexpr int NB = 64;

struct HinvScalars {
  float damp;
  int info;
};

// damp = percdamp * mean(diag(H')) where H' = H/div with zero diagonal entries replaced by 1;
// dead[c] = 1 where the (permuted) diagonal was zero
__global__ __launch_bounds__(256) void hinv_stats_kernel(const float* __restrict__ H, int64_t ldh, int K,
                                                         const int32_t* __restrict__ perm, float div,
                                                         float percdamp, uint8_t* __restrict__ dead,
                                                         HinvScalars* sc) {
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
                                                          float* __restrict__ A) {
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

// Factor the 64x64 diagonal block at (k0,k0) in LDS and replace it by the inverse of its factor.
__global__ __launch_bounds__(256) void potf2_inv_kernel(float* __restrict__ A, int Kp, int k0, int K,
                                                        HinvScalars* sc) {
  __shared__ float L[NB][NB + 1];
  __shared__ float X[NB][NB + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < NB * NB; e += 256) {
    const int i = e / NB, j = e % NB;
    L[i][j] = (j <= i) ? A[(int64_t)(k0 + i) * Kp + k0 + j] : 0.f;
    X[i][j] = 0.f;
  }
  for (int j = 0; j < NB; ++j) {
    __syncthreads();
    if (tid == 0) {
      float d = L[j][j];
      if (!(d > 0.f) || d != d || d > 3.0e38f) {
        // first failing pivot, 1-based index in the ORIGINAL (un-reversed) ordering
        if (k0 + j < K) atomicCAS(&sc->info, 0, K - (k0 + j));
        d = 1.f;
      }
      L[j][j] = sqrtf(d);
    }
    __syncthreads();
    const float piv = L[j][j];
    for (int i = j + 1 + tid; i < NB; i += 256) L[i][j] = L[i][j] / piv;
    __syncthreads();
    const int n = NB - 1 - j;
    for (int e = tid; e < n * n; e += 256) {
      const int i = j + 1 + e / n, c = j + 1 + e % n;
      if (c <= i) L[i][c] -= L[i][j] * L[c][j];
    }
  }
  __syncthreads();
  // column tid of X = L^-1 by forward substitution; a thread only ever reads its own column of X
  if (tid < NB) {
    const int j = tid;
    for (int i = j; i < NB; ++i) {
      float s = (i == j) ? 1.f : 0.f;
      for (int k = j; k < i; ++k) s -= L[i][k] * X[k][j];
      X[i][j] = s / L[i][i];
    }
  }
  __syncthreads();
  for (int e = tid; e < NB * NB; e += 256) {
    const int i = e / NB, j = e % NB;
    A[(int64_t)(k0 + i) * Kp + k0 + j] = (j <= i) ? X[i][j] : 0.f;
  }
}

// U[i][j] = X[K-1-i][K-1-j] for j >= i, 0 below; identity when the factorisation failed
__global__ __launch_bounds__(256) void hinv_copyout_kernel(const float* __restrict__ X, int Kp, int K,
                                                           const HinvScalars* __restrict__ sc,
                                                           float* __restrict__ U, int64_t ldu,
                                                           int32_t* __restrict__ info_out) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int i = blockIdx.y;
  if (i == 0 && j == 0 && info_out) *info_out = sc->info;
  if (j >= K) return;
  float v = 0.f;
  if (sc->info != 0) {
    v = (i == j) ? 1.f : 0.f;
  } else if (j >= i) {
    v = X[(int64_t)(K - 1 - i) * Kp + (K - 1 - j)];
  }
  U[(int64_t)i * ldu + j] = v;
}

inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

}  // namespace

extern "C" int64_t llmc_gptq_hinv_workspace_bytes(int64_t K) {
  const int64_t Kp = round_up(K, NB);
  // work matrix + recursive-doubling temporary (at most Kp^2/4) + scalars
  return (Kp * Kp + Kp * Kp / 4 + 64) * 4 + 256;
}

extern "C" int llmc_gptq_hinv(float* H, int64_t ldh, int64_t K, const int32_t* perm, float divisor,
                              float percdamp, uint8_t* dead_out, void* workspace, int64_t workspace_bytes,
                              int32_t* info_out, void* stream) {
  LLMC_CHECK_ARG(H != nullptr, 1);
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
                     dead_out, sc);
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(hinv_copyin_kernel, dim3((Kp + 255) / 256, Kp), dim3(256), 0, st, H, ldh, (int)K, Kp, perm,
                     divisor, sc, A);
  LLMC_LAUNCH_STATUS();

  // right-looking blocked Cholesky; diagonal blocks end up holding inv(L_kk)
  for (int k0 = 0; k0 < Kp; k0 += NB) {
    hipLaunchKernelGGL(potf2_inv_kernel, dim3(1), dim3(256), 0, st, A, Kp, k0, (int)K, sc);
    LLMC_LAUNCH_STATUS();
    const int M = Kp - k0 - NB;
    if (M <= 0) break;
    float* A21 = A + (int64_t)(k0 + NB) * Kp + k0;
    GemmF32 g = {};
    // panel: A21 <- A21 * inv(L_kk)^T   (in place: one tile column, each workgroup owns its rows)
    g.A = A21; g.lda = Kp; g.B = A + (int64_t)k0 * Kp + k0; g.ldb = Kp; g.C = A21; g.ldc = Kp;
    g.M = M; g.N = NB; g.Kc = NB; g.alpha = 1.f; g.beta = 0.f; g.trans_b = 1; g.batch = 1;
    int rc = llmc_gemm_f32(g, st);
    if (rc) return rc;
    // trailing: A22 <- A22 - A21 A21^T   (lower triangle only)
    GemmF32 s = {};
    s.A = A21; s.lda = Kp; s.B = A21; s.ldb = Kp; s.C = A + (int64_t)(k0 + NB) * Kp + k0 + NB; s.ldc = Kp;
    s.M = M; s.N = M; s.Kc = NB; s.alpha = -1.f; s.beta = 1.f; s.trans_b = 1; s.c_lower = 1; s.batch = 1;
    rc = llmc_gemm_f32(s, st);
    if (rc) return rc;
  }

  // inverse by recursive doubling: [[X11,0],[X21,X22]] with X21 = -X22 * L21 * X11
  for (int64_t s = NB; s < Kp; s *= 2) {
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

  hipLaunchKernelGGL(hinv_copyout_kernel, dim3((unsigned)((K + 255) / 256), (unsigned)K), dim3(256), 0, st, A, Kp,
                     (int)K, sc, H, ldh, info_out);
  LLMC_LAUNCH_STATUS();
  return 0;
}
