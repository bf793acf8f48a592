// GPTQ Hessian accumulation  H[K,K] += alpha * X^T X  on the gfx950 matrix cores.
//
// X is [T,K] row-major (tokens x features), so the contraction index t is the
// strided one.  Each workgroup owns one BT x BT tile of the upper triangle of
// H.  Per 64-token slab it loads the two [64 x BT] panels of X that the tile
// needs with 16-byte row-contiguous loads, transposes 8x8 (or 4x8) sub-blocks
// in registers and writes them to LDS feature-major, so every lane can fetch
// its 8 consecutive tokens of one feature with a single 128-bit LDS read --
// the operand shape of v_mfma_f32_32x32x16_{bf16,f16}.  bf16 x bf16 products
// are exact in fp32 and the accumulation is fp32, so the result differs from
// an fp32 GEMM on the upcast inputs only by summation order.
#include "common.h"

namespace {

constexpr int BK = 64;                  // tokens per slab
constexpr int ROW_BYTES = BK * 2 + 16;  // LDS bytes per feature row (padded: 36 dwords)

template <int DT>
struct Mfma;
template <>
struct Mfma<LLMC_BF16> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<LLMC_F16> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

// 8 consecutive 16-bit features of token row t starting at feature c (zero outside [T,K))
template <bool ALIGNED>
__device__ __forceinline__ uint4 load8(const uint16_t* X, int64_t ldx, int t, int c, int T, int K) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (t >= T || c >= K) return v;
  const uint16_t* p = X + (int64_t)t * ldx + c;
  if (ALIGNED) {
    v = *(const uint4*)p;
  } else {
    uint16_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = (c + j < K) ? p[j] : (uint16_t)0;
    v.x = e[0] | ((uint32_t)e[1] << 16);
    v.y = e[2] | ((uint32_t)e[3] << 16);
    v.z = e[4] | ((uint32_t)e[5] << 16);
    v.w = e[6] | ((uint32_t)e[7] << 16);
  }
  return v;
}

__device__ __forceinline__ uint32_t dword_of(const uint4& v, int j) {
  return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w;
}

// BT x BT output tile, 256 threads = 2x2 waves, each wave (BT/2)x(BT/2) = MI x MI MFMA tiles
template <int BT, int DT, bool ALIGNED>
__global__ __launch_bounds__(256) void hessian_syrk_kernel(float* __restrict__ H, int64_t ldh,
                                                            const uint16_t* __restrict__ X, int64_t ldx,
                                                            int T, int K, float alpha, int assume_sym,
                                                            int vec_ok, int nb, int ntiles) {
  constexpr int RT = BT / 32;  // token rows per thread per panel
  constexpr int GI = BT / 8;   // 8-feature groups per panel
  constexpr int MI = BT / 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* sA = smem;
  unsigned char* sB = smem + BT * ROW_BYTES;

  // consecutive tile ids land on the same XCD (workgroups are dealt round-robin to the 8 XCDs)
  const int per_xcd = (ntiles + 7) / 8;
  const int p = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (p >= ntiles) return;
  // p -> (I, J), J >= I, row-major over the upper triangle
  int I = 0, rem = p;
  while (rem >= nb - I) {
    rem -= nb - I;
    ++I;
  }
  const int J = I + rem;
  const int i0 = I * BT, j0 = J * BT;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int g_i = tid % GI, g_t = tid / GI;

  f32x16_t acc[MI][MI];
#pragma unroll
  for (int a = 0; a < MI; ++a)
#pragma unroll
    for (int b = 0; b < MI; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  uint4 ra[RT], rb[RT];
  auto load_slab = [&](int t0) {
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const int t = t0 + g_t * RT + r;
      ra[r] = load8<ALIGNED>(X, ldx, t, i0 + g_i * 8, T, K);
      rb[r] = load8<ALIGNED>(X, ldx, t, j0 + g_i * 8, T, K);
    }
  };
  // registers hold RT token rows x 8 features; LDS wants, per feature, RT consecutive tokens
  auto store_slab = [&]() {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      uint32_t oa[RT / 2], ob[RT / 2];
      const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int q = 0; q < RT / 2; ++q) {
        oa[q] = __builtin_amdgcn_perm(dword_of(ra[2 * q + 1], c >> 1), dword_of(ra[2 * q], c >> 1), sel);
        ob[q] = __builtin_amdgcn_perm(dword_of(rb[2 * q + 1], c >> 1), dword_of(rb[2 * q], c >> 1), sel);
      }
      const int off = (g_i * 8 + c) * ROW_BYTES + g_t * RT * 2;
      if (RT == 8) {
        *(uint4*)(sA + off) = make_uint4(oa[0], oa[1], oa[2 % (RT / 2)], oa[3 % (RT / 2)]);
        *(uint4*)(sB + off) = make_uint4(ob[0], ob[1], ob[2 % (RT / 2)], ob[3 % (RT / 2)]);
      } else {
        *(uint2*)(sA + off) = make_uint2(oa[0], oa[1 % (RT / 2)]);
        *(uint2*)(sB + off) = make_uint2(ob[0], ob[1 % (RT / 2)]);
      }
    }
  };

  const int nslab = (T + BK - 1) / BK;
  load_slab(0);
  store_slab();
  __syncthreads();
  for (int s = 0; s < nslab; ++s) {
    if (s + 1 < nslab) load_slab((s + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      uint4 fa[MI], fb[MI];
      const int koff = ks * 32 + (lane >> 5) * 16;
#pragma unroll
      for (int a = 0; a < MI; ++a)
        fa[a] = *(const uint4*)(sA + (wm * (BT / 2) + a * 32 + (lane & 31)) * ROW_BYTES + koff);
#pragma unroll
      for (int b = 0; b < MI; ++b)
        fb[b] = *(const uint4*)(sB + (wn * (BT / 2) + b * 32 + (lane & 31)) * ROW_BYTES + koff);
#pragma unroll
      for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int b = 0; b < MI; ++b) acc[a][b] = Mfma<DT>::run(fa[a], fb[b], acc[a][b]);
    }
    __syncthreads();
    if (s + 1 < nslab) {
      store_slab();
      __syncthreads();
    }
  }

  // 32x32 accumulator layout: lane holds column (lane&31); register v holds row
  // (v/4)*8 + (lane>>5)*4 + (v&3)
  const bool diag = (I == J);
#pragma unroll
  for (int a = 0; a < MI; ++a) {
#pragma unroll
    for (int b = 0; b < MI; ++b) {
      const int col = j0 + wn * (BT / 2) + b * 32 + (lane & 31);
      const int rbase = i0 + wm * (BT / 2) + a * 32 + (lane >> 5) * 4;
      if (col >= K) continue;
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        float out[4];
        const int r0 = rbase + vq * 8;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = r0 + e;
          out[e] = 0.f;
          if (row < K) {
            float* hp = H + (int64_t)row * ldh + col;
            out[e] = *hp + alpha * acc[a][b][vq * 4 + e];
            *hp = out[e];
          }
        }
        if (!diag) {
          float* mp = H + (int64_t)col * ldh + r0;
          if (assume_sym) {
            if (r0 + 3 < K && vec_ok) {
              *(float4*)mp = make_float4(out[0], out[1], out[2], out[3]);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (r0 + e < K) mp[e] = out[e];
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (r0 + e < K) mp[e] += alpha * acc[a][b][vq * 4 + e];
          }
        }
      }
    }
  }
}

template <int BT, int DT>
int launch(float* H, int64_t ldh, const void* X, int64_t ldx, int64_t T, int64_t K, float alpha,
           int flags, hipStream_t st) {
  const int nb = (int)((K + BT - 1) / BT);
  const int ntiles = nb * (nb + 1) / 2;
  const int grid = ((ntiles + 7) / 8) * 8;
  const bool aligned = (K % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)X & 15) == 0);
  const int sym = (flags & LLMC_HESSIAN_ASSUME_SYMMETRIC) ? 1 : 0;
  const int vec_ok = ((ldh & 3) == 0 && ((uintptr_t)H & 15) == 0) ? 1 : 0;
  constexpr int smem = 2 * BT * ROW_BYTES;
  auto kern = aligned ? hessian_syrk_kernel<BT, DT, true> : hessian_syrk_kernel<BT, DT, false>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return 1000 + (int)e;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, st, H, ldh, (const uint16_t*)X, ldx, (int)T,
                     (int)K, alpha, sym, vec_ok, nb, ntiles);
  LLMC_LAUNCH_STATUS();
  return 0;
}

}  // namespace

extern "C" int llmc_hessian_accumulate(float* H, int64_t ldh, const void* X, int64_t ldx, int64_t T,
                                       int64_t K, int32_t x_dtype, float alpha, int32_t flags,
                                       void* stream) {
  LLMC_CHECK_ARG(H != nullptr, 1);
  LLMC_CHECK_ARG(K > 0 && K < (1 << 30) && ldh >= K, 2);
  LLMC_CHECK_ARG(T >= 0 && T < (1ll << 31), 5);
  if (T == 0) return 0;
  LLMC_CHECK_ARG(X != nullptr, 3);
  LLMC_CHECK_ARG(ldx >= K, 4);
  LLMC_CHECK_ARG(x_dtype == LLMC_BF16 || x_dtype == LLMC_F16, 7);
  hipStream_t st = (hipStream_t)stream;
  // 256-wide tiles once there are enough of them to fill 256 CUs; 128-wide below that
  const int64_t nb256 = (K + 255) / 256;
  const bool big = nb256 * (nb256 + 1) / 2 >= 512;
  if (x_dtype == LLMC_BF16)
    return big ? launch<256, LLMC_BF16>(H, ldh, X, ldx, T, K, alpha, flags, st)
               : launch<128, LLMC_BF16>(H, ldh, X, ldx, T, K, alpha, flags, st);
  return big ? launch<256, LLMC_F16>(H, ldh, X, ldx, T, K, alpha, flags, st)
             : launch<128, LLMC_F16>(H, ldh, X, ldx, T, K, alpha, flags, st);
}

extern "C" int llmc_version(void) { return 1; }
