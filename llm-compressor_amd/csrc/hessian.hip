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
#include <type_traits>

#include "common.h"

namespace {

constexpr int BK = 64;          // tokens per slab
constexpr int ROW_BYTES = BK * 2;  // LDS bytes per feature row: 8 chunks of 8 tokens, XOR-swizzled

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

// 8 consecutive 16-bit features of token row t starting at feature c (zero outside [T,K)).
// The aligned form is branch-free (clamped address) so the main loop stays one basic block.
template <bool ALIGNED>
__device__ __forceinline__ uint4 load8(const uint16_t* X, int64_t ldx, int t, int c, int T, int K) {
  if (ALIGNED) {
    const int tt = t < T ? t : T - 1;
    const int cc = c < K ? c : K - 8;
    // rows past T are zeroed by the caller before use (last slab only); columns past K only
    // feed outputs that are never stored, so their (in-bounds) garbage is harmless
    return *(const uint4*)(X + (int64_t)tt * ldx + cc);
  }
  uint4 v = make_uint4(0, 0, 0, 0);
  if (t >= T || c >= K) return v;
  const uint16_t* p = X + (int64_t)t * ldx + c;
  uint16_t e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) e[j] = (c + j < K) ? p[j] : (uint16_t)0;
  v.x = e[0] | ((uint32_t)e[1] << 16);
  v.y = e[2] | ((uint32_t)e[3] << 16);
  v.z = e[4] | ((uint32_t)e[5] << 16);
  v.w = e[6] | ((uint32_t)e[7] << 16);
  return v;
}

__device__ __forceinline__ uint32_t dword_of(const uint4& v, int j) {
  return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w;
}

// byte offset of 16-byte chunk q (tokens 8q..8q+7) of feature row i.  The XOR keeps both access
// patterns conflict-free: MFMA operand reads touch 8+ consecutive rows at one q, the transposing
// writes touch rows 8 apart at one q.
__device__ __forceinline__ int chunk_off(int i, int q) {
  return i * ROW_BYTES + ((q ^ (i & 7) ^ ((i >> 3) & 7)) << 4);
}

// BT x BT output tile, 256 threads = 2x2 waves, each wave (BT/2)x(BT/2) = MI x MI MFMA tiles.
// LDS holds two stages of the two feature-major panels; global loads for slab s+2 are in
// flight while slab s is multiplied and slab s+1 is transposed into the other stage.
template <int BT, int DT, bool ALIGNED, bool FAST_EPI>
__global__ __launch_bounds__(256) void hessian_syrk_kernel(float* __restrict__ H, int64_t ldh,
                                                            const uint16_t* __restrict__ X, int64_t ldx,
                                                            int T, int K, float alpha, int assume_sym,
                                                            int vec_ok, int nb, int nslots) {
  constexpr int RT = BT / 32;  // token rows per thread per panel
  constexpr int GI = BT / 8;   // 8-feature groups per panel
  constexpr int MI = BT / 64;
  constexpr int PANEL = BT * ROW_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [2 stages][A,B][BT][128 B]

  // Tile order.  Workgroups are dealt round-robin to the 8 XCDs (each with a private L2), so
  // block b runs on XCD b%8; p makes every XCD walk a contiguous range of tile slots.  Slots are
  // grouped into SH x SW super-tiles (as many tiles as run concurrently on one XCD), so the
  // workgroups sharing an L2 touch only SH + SW feature panels of X per slab instead of one each.
  constexpr int SH = BT == 256 ? 4 : 8, SW = 8;
  const int per_xcd = (nslots + 7) / 8;
  const int p = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (p >= nslots) return;
  const int nsj = (nb + SW - 1) / SW;
  int su = p / (SH * SW), SI = 0;
  // super-row SI holds super-columns (SH*SI)/SW .. nsj-1 (those that reach the upper triangle)
  while (su >= nsj - (SH * SI) / SW) {
    su -= nsj - (SH * SI) / SW;
    ++SI;
  }
  const int SJ = (SH * SI) / SW + su;
  const int I = SI * SH + (p % (SH * SW)) / SW;
  const int J = SJ * SW + p % SW;
  if (I >= nb || J >= nb || J < I) return;
  const int i0 = I * BT, j0 = J * BT;
  const bool diag = (I == J);

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
  // RT token rows x 8 features of one panel (features col0 + g_i*8 ..) of the slab starting at t0
  auto load_panel = [&](uint4* rg, int t0, int col0) {
#pragma unroll
    for (int r = 0; r < RT; ++r) rg[r] = load8<ALIGNED>(X, ldx, t0 + g_t * RT + r, col0 + g_i * 8, T, K);
  };
  // registers hold RT token rows x 8 features; LDS wants, per feature, RT consecutive tokens:
  // column c of the thread's 8 features goes out as one 16-byte (RT == 8) or 8-byte LDS write
  auto store_col = [&](unsigned char* st, const uint4* rg, int c) {
    uint32_t o[RT / 2];
    const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
    for (int q = 0; q < RT / 2; ++q)
      o[q] = __builtin_amdgcn_perm(dword_of(rg[2 * q + 1], c >> 1), dword_of(rg[2 * q], c >> 1), sel);
    const int row = g_i * 8 + c;
    if constexpr (RT == 8) {
      *(uint4*)(st + chunk_off(row, g_t)) = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
      *(uint2*)(st + chunk_off(row, g_t >> 1) + (g_t & 1) * 8) = make_uint2(o[0], o[1]);
    }
  };
  auto store_panel = [&](unsigned char* st, const uint4* rg) {
#pragma unroll
    for (int c = 0; c < 8; ++c) store_col(st, rg, c);
  };
  // zero the token rows of a register-held panel that lie past T (only the last slab has any)
  auto mask_tail = [&](uint4* rg, int t0) {
    if (!ALIGNED) return;  // the element-wise loader already zero-fills
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const bool ok = t0 + g_t * RT + r < T;
      rg[r].x = ok ? rg[r].x : 0u; rg[r].y = ok ? rg[r].y : 0u; rg[r].z = ok ? rg[r].z : 0u; rg[r].w = ok ? rg[r].w : 0u;
    }
  };
  // One slab of matrix ops from stage `cur`, written out as an explicit software pipeline: the
  // slab is four groups of 16 tokens, each group NSTEP steps of two MFMAs, and every step also
  // issues its share of (1) the LDS reads of the next group's operand fragments (double-buffered
  // in registers), (2) when STORE, the transposing LDS writes of the next slab -- first panel
  // during group 0, second during group 2 -- and (3) the global loads that refill each register
  // set during the following group (slab after next, starting at token t2).  A scheduling fence
  // after every step keeps the compiler from regrouping them; with one wave per SIMD nothing
  // else would cover a stall.
  auto compute = [&](unsigned char* curA, unsigned char* nxtA, int t2, auto store_tag, auto mask_tag) {
    constexpr bool STORE = decltype(store_tag)::value;
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr int MPS = 2, NSTEP = MI * MI / MPS;  // matrix ops per step, steps per 16-token group
    constexpr int FPS = 2 * MI / NSTEP, CPS = 8 / NSTEP, LPS = RT / NSTEP;
    unsigned char* curB = curA + PANEL;
    uint4 fa[2][MI], fb[2][MI];
    // fragment number n of group ks, in the order the matrix ops first need them:
    // A rows 0, then all B rows, then the remaining A rows
    auto read_frag = [&](int ks, int n) {
      const int f = n == 0 ? 0 : (n <= MI ? MI + n - 1 : n - MI);  // f < MI -> A rows, else B rows
      const int q = ks * 2 + (lane >> 5);
      if (f < MI)
        fa[ks & 1][f] = *(const uint4*)(curA + chunk_off(wm * (BT / 2) + f * 32 + (lane & 31), q));
      else
        fb[ks & 1][f - MI] = *(const uint4*)(curB + chunk_off(wn * (BT / 2) + (f - MI) * 32 + (lane & 31), q));
    };
#pragma unroll
    for (int f = 0; f < 2 * MI; ++f) read_frag(0, f);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (STORE && MASK && ks == 0) mask_tail(ra, t2 - BK);
      if (STORE && MASK && ks == 2) mask_tail(rb, t2 - BK);
#pragma unroll
      for (int st = 0; st < NSTEP; ++st) {
        if (ks + 1 < BK / 16) {
#pragma unroll
          for (int f = st * FPS; f < (st + 1) * FPS; ++f) read_frag(ks + 1, f);
        }
        if (STORE) {
#pragma unroll
          for (int c = st * CPS; c < (st + 1) * CPS; ++c) {
            if (ks == 0) store_col(nxtA, ra, c);
            if (ks == 2) store_col(nxtA + PANEL, rb, c);
          }
#pragma unroll
          for (int r = st * LPS; r < (st + 1) * LPS; ++r) {
            if (ks == 1) ra[r] = load8<ALIGNED>(X, ldx, t2 + g_t * RT + r, i0 + g_i * 8, T, K);
            if (ks == 3) rb[r] = load8<ALIGNED>(X, ldx, t2 + g_t * RT + r, j0 + g_i * 8, T, K);
          }
        }
#pragma unroll
        for (int m = st * MPS; m < (st + 1) * MPS; ++m)
          acc[m / MI][m % MI] = Mfma<DT>::run(fa[ks & 1][m / MI], fb[ks & 1][m % MI], acc[m / MI][m % MI]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  const int nslab = (T + BK - 1) / BK;
  load_panel(ra, 0, i0);
  load_panel(rb, 0, j0);
  mask_tail(ra, 0);
  mask_tail(rb, 0);
  store_panel(smem, ra);
  store_panel(smem + PANEL, rb);
  load_panel(ra, BK, i0);  // (clamped in-bounds when there is no second slab)
  load_panel(rb, BK, j0);
  __syncthreads();
  // steady state: slab s multiplied, slab s+1 transposed into the other stage, slab s+2 in flight
  for (int s = 0; s + 2 < nslab; ++s) {
    compute(smem + (s & 1) * 2 * PANEL, smem + ((s + 1) & 1) * 2 * PANEL, (s + 2) * BK, std::true_type{},
            std::false_type{});
    __syncthreads();
  }
  if (nslab >= 2) {
    const int s = nslab - 2;
    compute(smem + (s & 1) * 2 * PANEL, smem + ((s + 1) & 1) * 2 * PANEL, (s + 2) * BK, std::true_type{},
            std::true_type{});
    __syncthreads();
  }
  compute(smem + ((nslab - 1) & 1) * 2 * PANEL, smem, 0, std::false_type{}, std::false_type{});

  // 32x32 accumulator layout: lane holds column n = lane&31; register v holds row
  // (v/4)*8 + (lane>>5)*4 + (v&3), i.e. 4 consecutive rows per register quad.  Seen from the
  // mirrored tile H[j][i] a quad is 4 consecutive floats of one row, so the read-modify-write
  // runs there with 16-byte accesses (4x fewer, 4x larger requests in flight); the tile
  // H[i][j] itself then only needs stores, which are row-contiguous across lanes.
  if (FAST_EPI && i0 + BT <= K && j0 + BT <= K) {
    // interior tile: no bounds checks, so the 16-byte loads of a whole row of MFMA tiles are
    // issued back to back before the first use
#pragma unroll
    for (int a = 0; a < MI; ++a) {
      float4 old[MI][4];
#pragma unroll
      for (int b = 0; b < MI; ++b) {
        const int col = j0 + wn * (BT / 2) + b * 32 + (lane & 31);
        const int rbase = i0 + wm * (BT / 2) + a * 32 + (lane >> 5) * 4;
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) old[b][vq] = *(const float4*)(H + (int64_t)col * ldh + rbase + vq * 8);
      }
#pragma unroll
      for (int b = 0; b < MI; ++b) {
        const int col = j0 + wn * (BT / 2) + b * 32 + (lane & 31);
        const int rbase = i0 + wm * (BT / 2) + a * 32 + (lane >> 5) * 4;
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int r0 = rbase + vq * 8;
          float4 o;
          o.x = old[b][vq].x + alpha * acc[a][b][vq * 4 + 0];
          o.y = old[b][vq].y + alpha * acc[a][b][vq * 4 + 1];
          o.z = old[b][vq].z + alpha * acc[a][b][vq * 4 + 2];
          o.w = old[b][vq].w + alpha * acc[a][b][vq * 4 + 3];
          *(float4*)(H + (int64_t)col * ldh + r0) = o;
          if (!diag) {
            H[(int64_t)(r0 + 0) * ldh + col] = o.x;
            H[(int64_t)(r0 + 1) * ldh + col] = o.y;
            H[(int64_t)(r0 + 2) * ldh + col] = o.z;
            H[(int64_t)(r0 + 3) * ldh + col] = o.w;
          }
        }
      }
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < MI; ++a) {
#pragma unroll
    for (int b = 0; b < MI; ++b) {
      const int col = j0 + wn * (BT / 2) + b * 32 + (lane & 31);
      const int rbase = i0 + wm * (BT / 2) + a * 32 + (lane >> 5) * 4;
      if (col < K) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int r0 = rbase + vq * 8;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int row = r0 + e;
            if (row < K) {
              float* hp = H + (int64_t)row * ldh + col;
              const float out = *hp + alpha * acc[a][b][vq * 4 + e];
              *hp = out;
              if (!diag) {
                float* mp = H + (int64_t)col * ldh + row;
                *mp = assume_sym ? out : *mp + alpha * acc[a][b][vq * 4 + e];
              }
            }
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
  constexpr int SH = BT == 256 ? 4 : 8, SW = 8;  // must match the kernel
  const int nsi = (nb + SH - 1) / SH, nsj = (nb + SW - 1) / SW;
  int nsuper = 0;
  for (int si = 0; si < nsi; ++si) nsuper += nsj - (SH * si) / SW;
  const int nslots = nsuper * SH * SW;
  const int grid = ((nslots + 7) / 8) * 8;
  const bool aligned = (K % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)X & 15) == 0);
  const int sym = (flags & LLMC_HESSIAN_ASSUME_SYMMETRIC) ? 1 : 0;
  const int vec_ok = ((ldh & 3) == 0 && ((uintptr_t)H & 15) == 0) ? 1 : 0;
  constexpr int smem = 4 * BT * ROW_BYTES;
  // 16-byte read-modify-write epilogue needs a symmetric H and 16-byte aligned rows
  const bool fast = sym && vec_ok;
  auto kern = aligned ? (fast ? hessian_syrk_kernel<BT, DT, true, true> : hessian_syrk_kernel<BT, DT, true, false>)
                      : (fast ? hessian_syrk_kernel<BT, DT, false, true> : hessian_syrk_kernel<BT, DT, false, false>);
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return 1000 + (int)e;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, st, H, ldh, (const uint16_t*)X, ldx, (int)T,
                     (int)K, alpha, sym, vec_ok, nb, nslots);
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
