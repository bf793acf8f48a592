// fp32 GEMM on v_mfma_f32_32x32x2_f32 for the trailing-matrix updates (Cholesky chain, GPTQ).
//
// 256 threads = 2x2 waves; a BM x BN tile of C per workgroup; the A and B slabs
// (BK = 16 deep) are staged k-major in LDS so the per-lane MFMA operands
// (one float each: row/col = lane&31, k = lane>>5) are conflict-free reads.
// The next slab is fetched into registers while the current one is multiplied.
#include "common.h"
#include "gemm_f32.h"

namespace {

constexpr int BK = 16;

__device__ __forceinline__ float4 ld4(const float* p, int valid, bool vec) {
  // `valid` = how many of the 4 elements are inside the matrix (<=0: none)
  if (valid >= 4 && vec) return *(const float4*)p;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (valid > 0) v.x = p[0];
  if (valid > 1) v.y = p[1];
  if (valid > 2) v.z = p[2];
  if (valid > 3) v.w = p[3];
  return v;
}

// FAST: the tile lies fully inside C, the contraction range is a multiple of BK and all rows are
// 16-byte aligned, so every load is an unconditional float4 and the main loop is one basic block.
template <int BM, int BN, bool TRANS_B, bool FAST, bool TRANS_A>
__device__ __forceinline__ void gemm_tile(const GemmF32& g, const float* A, const float* B, float* C, int m0,
                                          int n0, int k_begin, int k_end, float* As, float* Bs) {
  constexpr int LDA_S = BM + 4, LDB_S = BN + 4;
  constexpr int MI = BM / 64, NI = BN / 64;
  constexpr int A_LD = BM / 64;  // float4 loads per thread for the A slab
  constexpr int B_LD = BN / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  f32x16_t acc[MI][NI];
#pragma unroll
  for (int a = 0; a < MI; ++a)
#pragma unroll
    for (int b = 0; b < NI; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  float4 ra[A_LD], rb[B_LD];
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int f = tid + i * 256;
      if (TRANS_A) {
        const int k = k0 + f / (BM / 4), m = m0 + (f % (BM / 4)) * 4;
        if (FAST)
          ra[i] = *(const float4*)(A + (int64_t)k * g.lda + m);
        else
          ra[i] = (k < k_end) ? ld4(A + (int64_t)k * g.lda + m, g.M - m, false) : make_float4(0.f, 0.f, 0.f, 0.f);
        continue;
      }
      const int m = m0 + f / 4, k = k0 + (f % 4) * 4;
      if (FAST)
        ra[i] = *(const float4*)(A + (int64_t)m * g.lda + k);
      else
        ra[i] = (m < g.M) ? ld4(A + (int64_t)m * g.lda + k, k_end - k, false) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < B_LD; ++i) {
      const int f = tid + i * 256;
      if (TRANS_B) {
        const int n = n0 + f / 4, k = k0 + (f % 4) * 4;
        if (FAST)
          rb[i] = *(const float4*)(B + (int64_t)n * g.ldb + k);
        else
          rb[i] = (n < g.N) ? ld4(B + (int64_t)n * g.ldb + k, k_end - k, false) : make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        const int k = k0 + f / (BN / 4), n = n0 + (f % (BN / 4)) * 4;
        if (FAST)
          rb[i] = *(const float4*)(B + (int64_t)k * g.ldb + n);
        else
          rb[i] = (k < k_end) ? ld4(B + (int64_t)k * g.ldb + n, g.N - n, false) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  };
  auto store_slab = [&]() {
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int f = tid + i * 256;
      if (TRANS_A) {
        const int k = f / (BM / 4), m = (f % (BM / 4)) * 4;
        *(float4*)&As[k * LDA_S + m] = ra[i];
        continue;
      }
      const int m = f / 4, k = (f % 4) * 4;
      As[(k + 0) * LDA_S + m] = ra[i].x;
      As[(k + 1) * LDA_S + m] = ra[i].y;
      As[(k + 2) * LDA_S + m] = ra[i].z;
      As[(k + 3) * LDA_S + m] = ra[i].w;
    }
#pragma unroll
    for (int i = 0; i < B_LD; ++i) {
      const int f = tid + i * 256;
      if (TRANS_B) {
        const int n = f / 4, k = (f % 4) * 4;
        Bs[(k + 0) * LDB_S + n] = rb[i].x;
        Bs[(k + 1) * LDB_S + n] = rb[i].y;
        Bs[(k + 2) * LDB_S + n] = rb[i].z;
        Bs[(k + 3) * LDB_S + n] = rb[i].w;
      } else {
        const int k = f / (BN / 4), n = (f % (BN / 4)) * 4;
        *(float4*)&Bs[k * LDB_S + n] = rb[i];
      }
    }
  };
  auto multiply = [&]() {
#pragma unroll
    for (int kk = 0; kk < BK / 2; ++kk) {
      const int k = 2 * kk + (lane >> 5);
      float fa[MI], fb[NI];
#pragma unroll
      for (int a = 0; a < MI; ++a) fa[a] = As[k * LDA_S + wm * (BM / 2) + a * 32 + (lane & 31)];
#pragma unroll
      for (int b = 0; b < NI; ++b) fb[b] = Bs[k * LDB_S + wn * (BN / 2) + b * 32 + (lane & 31)];
#pragma unroll
      for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int b = 0; b < NI; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a], fb[b], acc[a][b], 0, 0, 0);
    }
  };

  if (k_begin < k_end) {
    // two LDS stages: slab k+1 is fetched into registers before slab k is multiplied and
    // written to the other stage after it, one barrier per slab
    constexpr int STAGE_A = BK * LDA_S, STAGE_B = BK * LDB_S;
    float* const As0 = As;
    float* const Bs0 = Bs;
    load_slab(k_begin);
    store_slab();
    __syncthreads();
    int cur = 0;
    for (int k0 = k_begin; k0 + BK < k_end; k0 += BK) {
      load_slab(k0 + BK);
      multiply();
      cur ^= 1;
      As = As0 + cur * STAGE_A;
      Bs = Bs0 + cur * STAGE_B;
      store_slab();
      __syncthreads();
    }
    multiply();
  }

  // Epilogue.  A tile wholly inside C (and, for a lower-triangular C, wholly below the diagonal) needs no
  // per-element tests.  It uses buffer addressing: one descriptor for the wave's strip of C, the row offset
  // in a scalar register and a single per-lane byte offset, so no 64-bit address is kept per element; the
  // 16 values of a 32x32 sub-tile are fetched together, then combined and stored -- one memory round trip
  // per sub-tile instead of one per element.
  if (FAST && !(g.c_lower && n0 + BN - 1 > m0)) {
    const int wm_u = __builtin_amdgcn_readfirstlane(wm), wn_u = __builtin_amdgcn_readfirstlane(wn);
    float* const c0 = C + (int64_t)(m0 + wm_u * (BM / 2)) * g.ldc + n0 + wn_u * (BN / 2);
    const int lane_bytes = ((lane >> 5) * 4 * (int)g.ldc + (lane & 31)) * 4;
    const int row_bytes = (int)g.ldc * 4;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(c0, 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
      for (int b = 0; b < NI; ++b) {
        float cv[16];
        if (g.beta != 0.f) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            cv[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                rsrc, lane_bytes, (a * 32 + (v / 4) * 8 + (v & 3)) * row_bytes + b * 128, 0));
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float r = g.alpha * acc[a][b][v];
          if (g.beta != 0.f) r += g.beta * cv[v];
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, r), rsrc, lane_bytes,
                                                (a * 32 + (v / 4) * 8 + (v & 3)) * row_bytes + b * 128, 0);
        }
      }
    return;
  }

  // edge and diagonal tiles: element by element
#pragma unroll
  for (int a = 0; a < MI; ++a)
#pragma unroll
    for (int b = 0; b < NI; ++b) {
      const int col = n0 + wn * (BN / 2) + b * 32 + (lane & 31);
      if (!FAST && col >= g.N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * (BM / 2) + a * 32 + (v / 4) * 8 + (lane >> 5) * 4 + (v & 3);
        if ((!FAST && row >= g.M) || (g.c_lower && col > row)) continue;
        float* cp = C + (int64_t)row * g.ldc + col;
        float r = g.alpha * acc[a][b][v];
        if (g.beta != 0.f) r += g.beta * *cp;
        *cp = r;
      }
    }
}

// ALL_FAST: the host has checked that every tile of the launch takes the unconditional path
// (M, N multiples of the tile, contraction ranges multiples of BK, 16-byte aligned rows), so the
// bounds-checked variant is not even instantiated: fewer registers, more waves per SIMD.
template <int BM, int BN, bool TRANS_B, bool ALL_FAST, bool TRANS_A = false>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmF32 g, int vec) {
  __shared__ float As[2 * BK * (BM + 4)];
  __shared__ float Bs[2 * BK * (BN + 4)];
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (g.c_lower && n0 > m0 + BM - 1) return;
  const int b1 = (int)blockIdx.z % g.batch, b2 = (int)blockIdx.z / g.batch;
  const float* A = g.A + (int64_t)b1 * g.stride_a + (int64_t)b2 * g.stride2_a;
  const float* B = g.B + (int64_t)b1 * g.stride_b + (int64_t)b2 * g.stride2_b;
  float* C = g.C + (int64_t)b1 * g.stride_c + (int64_t)b2 * g.stride2_c;
  const int k_begin = g.b_lower_tri ? (n0 / BK) * BK : 0;
  int k_end = (g.kc_last > 0 && b1 == g.batch - 1) ? g.kc_last : g.Kc;
  if (g.a_lower_tri && m0 + BM < k_end) k_end = m0 + BM;
  if (ALL_FAST) {
    gemm_tile<BM, BN, TRANS_B, true, TRANS_A>(g, A, B, C, m0, n0, k_begin, k_end, As, Bs);
  } else {
    const bool fast = vec && m0 + BM <= g.M && n0 + BN <= g.N && ((k_end - k_begin) % BK) == 0 && g.ldc < (1 << 22);
    if (fast)
      gemm_tile<BM, BN, TRANS_B, true, TRANS_A>(g, A, B, C, m0, n0, k_begin, k_end, As, Bs);
    else
      gemm_tile<BM, BN, TRANS_B, false, TRANS_A>(g, A, B, C, m0, n0, k_begin, k_end, As, Bs);
  }
}

}  // namespace

static int gemm_f32_mfma(const GemmF32& g, hipStream_t st);

int llmc_gemm_f32(const GemmF32& g, hipStream_t st) {
  if (g.M <= 0 || g.N <= 0 || g.batch <= 0) return 0;
  if (g.trans_a && (g.trans_b || g.a_lower_tri)) return 1000 + (int)hipErrorInvalidValue;
  const int rc = llmc_gemm_x3(g, st);
  if (rc >= 0) return rc;
  return gemm_f32_mfma(g, st);
}

// C[M,N] = alpha * A * B' + beta * C for callers outside the library (the product of the lazy trailing
// update, W[:, i2:] -= Err1 @ Hinv[i1:i2, i2:]); flags: 1 = only the lower triangle of C, 2 = A lower
// triangular, 4 = B' zero above... (see include/llmc_amd.h), 8 = force the fp32 matrix instruction
extern "C" int llmc_sgemm(const float* A, int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc, int64_t M,
                          int64_t N, int64_t Kc, float alpha, float beta, int32_t trans_b, int32_t flags,
                          void* stream) {
  LLMC_CHECK_ARG(A != nullptr && lda > 0, 1);
  LLMC_CHECK_ARG(B != nullptr && ldb > 0, 3);
  LLMC_CHECK_ARG(C != nullptr && ldc >= N, 5);
  LLMC_CHECK_ARG(M >= 0 && N >= 0 && Kc >= 0 && M < (1 << 30) && N < (1 << 30) && Kc < (1 << 30), 7);
  LLMC_CHECK_ARG(lda >= Kc && ldb >= (trans_b ? Kc : N), 2);
  LLMC_CHECK_ARG(flags >= 0 && flags < 16, 13);
  GemmF32 g = {};
  g.A = A; g.lda = lda; g.B = B; g.ldb = ldb; g.C = C; g.ldc = ldc;
  g.M = (int)M; g.N = (int)N; g.Kc = (int)Kc; g.alpha = alpha; g.beta = beta; g.trans_b = trans_b ? 1 : 0;
  g.c_lower = flags & 1; g.a_lower_tri = (flags >> 1) & 1; g.b_lower_tri = (flags >> 2) & 1; g.batch = 1;
  if (g.M == 0 || g.N == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (flags & 8) return gemm_f32_mfma(g, st);
  return llmc_gemm_f32(g, st);
}

static int gemm_f32_mfma(const GemmF32& g, hipStream_t st) {
  const int nb2 = g.batch2 > 1 ? g.batch2 : 1;
  const int vec = ((g.lda & 3) == 0 && (g.ldb & 3) == 0 && (((uintptr_t)g.A | (uintptr_t)g.B) & 15) == 0 &&
                   (g.stride_a & 3) == 0 && (g.stride_b & 3) == 0 && (g.Kc & 3) == 0 &&
                   (nb2 == 1 || ((g.stride2_a & 3) == 0 && (g.stride2_b & 3) == 0)))
                      ? 1
                      : 0;
  // 128x128 tiles when they still give the chip enough workgroups, 64x64 otherwise
  const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * g.batch * nb2;
  const bool big = t128 >= 256 && g.M >= 128 && g.N >= 128;
  const int bt = big ? 128 : 64;
  // every tile unconditional?  (a_lower_tri / b_lower_tri cut the contraction at tile edges, which
  // are multiples of BK for both tile sizes)
  // (and the unconditional epilogue addresses a wave's strip of C with 32-bit byte offsets, up to 132 rows of ldc
  // floats from the strip's origin: rows of 4M floats and more take the per-element path with 64-bit addresses)
  const bool all_fast = vec && g.M % bt == 0 && g.N % bt == 0 && g.Kc % BK == 0 && g.kc_last % BK == 0 &&
                        g.ldc < (1 << 22);
  dim3 grid((g.N + bt - 1) / bt, (g.M + bt - 1) / bt, g.batch * nb2);
#define LLMC_GEMM(BT, TB, AF) hipLaunchKernelGGL((gemm_f32_kernel<BT, BT, TB, AF>), grid, dim3(256), 0, st, g, vec)
  if (g.trans_a) {
#define LLMC_GEMM_TA(BT, AF) hipLaunchKernelGGL((gemm_f32_kernel<BT, BT, false, AF, true>), grid, dim3(256), 0, st, g, vec)
    if (big) { if (all_fast) LLMC_GEMM_TA(128, true); else LLMC_GEMM_TA(128, false); }
    else { if (all_fast) LLMC_GEMM_TA(64, true); else LLMC_GEMM_TA(64, false); }
#undef LLMC_GEMM_TA
  } else if (big) {
    if (g.trans_b) { if (all_fast) LLMC_GEMM(128, true, true); else LLMC_GEMM(128, true, false); }
    else { if (all_fast) LLMC_GEMM(128, false, true); else LLMC_GEMM(128, false, false); }
  } else {
    if (g.trans_b) { if (all_fast) LLMC_GEMM(64, true, true); else LLMC_GEMM(64, true, false); }
    else { if (all_fast) LLMC_GEMM(64, false, true); else LLMC_GEMM(64, false, false); }
  }
#undef LLMC_GEMM
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : 1000 + (int)e;
}
