// fp32 GEMM carried by the 16-bit matrix cores: every fp32 operand element is split, on the way into LDS,
// into three bf16 values a = a0 + a1 + a2 (8 + 8 + 8 significand bits, same exponent range as fp32), and
// the product is formed from the six partial products whose weight is at least 2^-16 of the leading one,
//     a*b ~= a0*b0 + (a0*b1 + a1*b0) + (a0*b2 + a1*b1 + a2*b0),
// each an exact bf16 x bf16 product accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  The dropped terms are
// below 2^-24 of |a||b|, the rounding of an fp32 product, so the result is as accurate as the fp32 matrix
// instruction's while the 16-bit matrix pipe runs 16 times its rate (six products: 2.6x the fp32 peak).
//
// One workgroup owns a 256 x 256 tile of C (eight waves of 64 x 128) or a 128 x 128 one (four waves of
// 64 x 64).  A k-step is 16 deep.  Per k-step the workgroup fetches the fp32 slabs of both operands
// (tile edge x 16 each) into registers two steps ahead of their use, splits them into the three
// planes in the same step and stores them to one of three LDS stages k-contiguous (a row of a plane is 16 bf16
// = 32 bytes = two 16-byte chunks, the chunk index XOR-ed with bit 3 of the row: a 16-byte read is served
// sixteen lanes at a time over 64 banks, and the sixteen consecutive rows of one chunk that those lanes ask for
// then fall into distinct banks -- no conflicts counted), so that an MFMA operand (8 consecutive k of one row) is
// one ds_read_b128.  Operand B stored [Kc, N] (not transposed) is transposed on the way: a thread loads eight
// consecutive k rows of one column (a wave: two runs of 32 consecutive columns, one per half of the k-step) and
// writes that column's half row of every plane, so that a wave's stores cover whole rows of LDS one after the
// other.  The split/store work for a later step
// sits between the matrix instructions of the current one, one barrier per k-step.  Sustained rate on
// MI355X: about 200 TFLOP/s of fp32-equivalent work (1.2 PFLOP/s of bf16 matrix instructions, the rate
// the chip also sustains in the Hessian kernel) against about 130 TFLOP/s of the fp32 matrix instruction.
#include <type_traits>

#include "common.h"
#include "gemm_f32.h"
#include "qformat.h"

namespace {

constexpr int XK = 16;

__device__ __forceinline__ int plane_off(int row, int chunk) { return row * 32 + ((chunk ^ ((row >> 3) & 1)) << 4); }

// (x, y) -> the packed bf16 pairs of the three planes
__device__ __forceinline__ void split3(float x, float y, uint32_t& p0, uint32_t& p1, uint32_t& p2) {
  p0 = pack16<LLMC_BF16>(x, y);
  float rx = x - __uint_as_float(p0 << 16), ry = y - __uint_as_float(p0 & 0xffff0000u);
  p1 = pack16<LLMC_BF16>(rx, ry);
  rx -= __uint_as_float(p1 << 16);
  ry -= __uint_as_float(p1 & 0xffff0000u);
  p2 = pack16<LLMC_BF16>(rx, ry);
}

__device__ __forceinline__ f32x16_t mfma_bf16(const uint4& a, const uint4& b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0,
                                                 0, 0);
}

// WM x WN: tile of one wave; WAVES_M x WAVES_N waves form the workgroup tile BM x BN.  Both shipped shapes
// (256 x 256 with eight waves of 64 x 128, two per SIMD; 128 x 128 with four waves of 64 x 64 and two
// workgroups per CU) keep two waves on every SIMD, so that one wave's split/store and LDS reads run under the
// other's matrix instructions, and both give every thread two float4 loads per operand and k-step.
template <int WM, int WN, int WAVES_M, int WAVES_N, bool TRANS_B>
struct X3 {
  static constexpr int BM = WM * WAVES_M, BN = WN * WAVES_N;
  static constexpr int NTHREADS = 64 * WAVES_M * WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int PLANE_A = BM * 32, PLANE_B = BN * 32;  // bytes of one plane in one stage
  static constexpr int STAGE = 3 * (PLANE_A + PLANE_B);       // A planes 0..2, then B planes 0..2
  static constexpr int NLD_A = BM * 4 / NTHREADS, NLD_B = BN * 4 / NTHREADS;
  static_assert(NLD_A == 2 && NLD_B == 2 && NTHREADS == 2 * BN,
                "thread mapping below assumes two float4 per operand and thread, and two threads per column of B");
  static constexpr int CHUNKS = NLD_A + NLD_B;  // split/store chunks per k-step (A then B)

  struct Slab {
    float4 a[NLD_A], b[NLD_B];
  };

  // chunk c of a slab: c < NLD_A -> float4 i = c of A, else float4 i = c - NLD_A of B.
  // rows of A (and of B when TRANS_B): thread t, load i covers row (t + NTHREADS i) / 4, k quad (t & 3)
  template <int c>
  static __device__ __forceinline__ void load_chunk(const GemmF32& g, const float* A, const float* B, int m0, int n0,
                                                    int k, Slab& s) {
    const int tid = threadIdx.x;
    constexpr bool is_b = c >= NLD_A;
    constexpr int i = is_b ? c - NLD_A : c;
    if (!is_b) {
      const int f = tid + i * NTHREADS;
      s.a[i] = *(const float4*)(A + (int64_t)(m0 + (f >> 2)) * g.lda + k + ((f & 3) << 2));
    } else if (TRANS_B) {
      const int f = tid + i * NTHREADS;
      s.b[i] = *(const float4*)(B + (int64_t)(n0 + (f >> 2)) * g.ldb + k + ((f & 3) << 2));
    } else {
      // non-transposed B: thread t holds column t / 2, k rows 8 (t % 2) .. + 7; load i fetches four of them
      const float* src = B + (int64_t)(k + (tid & 1) * 8 + i * 4) * g.ldb + n0 + (tid >> 1);
      s.b[i] = make_float4(src[0], src[g.ldb], src[2 * g.ldb], src[3 * g.ldb]);
    }
  }
  static __device__ __forceinline__ void load(const GemmF32& g, const float* A, const float* B, int m0, int n0, int k,
                                              Slab& s) {
    load_chunk<0>(g, A, B, m0, n0, k, s);
    load_chunk<1>(g, A, B, m0, n0, k, s);
    load_chunk<2>(g, A, B, m0, n0, k, s);
    load_chunk<3>(g, A, B, m0, n0, k, s);
  }

  // chunk c of the split/store work of one slab: c < NLD_A -> A load c, else B
  template <int c>
  static __device__ __forceinline__ void split_store(const Slab& s, unsigned char* stage) {
    const int tid = threadIdx.x;
    constexpr bool is_b = c >= NLD_A;
    constexpr int i = is_b ? c - NLD_A : c;
    if (!is_b || TRANS_B) {
      const float4 v = is_b ? s.b[i] : s.a[i];
      const int f = tid + i * NTHREADS, row = f >> 2, kq = f & 3;
      uint32_t p[3][2];
      split3(v.x, v.y, p[0][0], p[1][0], p[2][0]);
      split3(v.z, v.w, p[0][1], p[1][1], p[2][1]);
      constexpr int plane = is_b ? PLANE_B : PLANE_A;
      unsigned char* base = stage + (is_b ? 3 * PLANE_A : 0) + plane_off(row, kq >> 1) + ((kq & 1) << 3);
#pragma unroll
      for (int q = 0; q < 3; ++q) *(uint2*)(base + q * plane) = make_uint2(p[q][0], p[q][1]);
    } else {
      // non-transposed B: load i holds the k rows 8 (t % 2) + 4 i .. + 3 of column t / 2, i.e. 8 bytes of that
      // column's row in every plane; the two threads of a column and their neighbours write consecutive bytes
      const float4 v = s.b[i];
      const int row = tid >> 1, half = tid & 1;
      uint32_t p[3][2];
      split3(v.x, v.y, p[0][0], p[1][0], p[2][0]);
      split3(v.z, v.w, p[0][1], p[1][1], p[2][1]);
      unsigned char* base = stage + 3 * PLANE_A + plane_off(row, half) + (i << 3);
#pragma unroll
      for (int q = 0; q < 3; ++q) *(uint2*)(base + q * PLANE_B) = make_uint2(p[q][0], p[q][1]);
    }
  }
};

template <int WM, int WN, int WAVES_M, int WAVES_N, bool TRANS_B>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_x3_kernel(GemmF32 g, int tiles_x, int tiles_y) {
  using C = X3<WM, WN, WAVES_M, WAVES_N, TRANS_B>;
  constexpr int BM = C::BM, BN = C::BN, TM = C::TM, TN = C::TN;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [3 stages][A0 A1 A2 B0 B1 B2][rows][32 B]

  // Workgroup ids are dealt round-robin to the 8 XCDs.  XCD x takes the tile rows x, 15 - x, 16 + x, 31 - x, ...
  // (a row's tiles share the A panel in that XCD's L2; the back-and-forth order balances the XCDs when the
  // work of a row grows with its index, as it does for triangular operands), longest rows first.  With a lower
  // triangular B the work of a tile falls with its column instead, so there the roles of rows and columns are
  // swapped: tile columns are dealt to the XCDs (sharing the B panel), first columns first.
  // With fewer than 8 rows left in a group of 8, some XCDs get no row of this problem; the slot is rotated
  // by the problem index times that remainder, so that the rows of successive problems fill the XCDs in turn.
  const bool by_columns = g.b_lower_tri && !g.a_lower_tri && !g.c_lower;
  const int major = by_columns ? tiles_x : tiles_y, minor = by_columns ? tiles_y : tiles_x;
  const int id = blockIdx.x;
  const int x = (id + (int)blockIdx.z * (major & 7)) & 7, j = id >> 3;
  const int i = j / minor, t = j - i * minor;
  const int rrow = 8 * i + ((i & 1) ? 7 - x : x);
  if (rrow >= major) return;
  const int ty = by_columns ? t : ((g.a_lower_tri || g.c_lower) ? tiles_y - 1 - rrow : rrow);
  const int tx = by_columns ? rrow : t;
  const int m0 = ty * BM, n0 = tx * BN;
  if (g.c_lower && n0 > m0 + BM - 1) return;
  const int b1 = (int)blockIdx.z % g.batch, b2 = (int)blockIdx.z / g.batch;
  const float* A = g.A + (int64_t)b1 * g.stride_a + (int64_t)b2 * g.stride2_a;
  const float* B = g.B + (int64_t)b1 * g.stride_b + (int64_t)b2 * g.stride2_b;
  float* Cm = g.C + (int64_t)b1 * g.stride_c + (int64_t)b2 * g.stride2_c;
  const int k_begin = g.b_lower_tri ? (n0 / XK) * XK : 0;
  int k_end = (g.kc_last > 0 && b1 == g.batch - 1) ? g.kc_last : g.Kc;
  if (g.a_lower_tri && m0 + BM < k_end) k_end = m0 + BM;
  const int nsteps = (k_end - k_begin) / XK;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  typename C::Slab slab;
  const int r = lane & 31, ch = lane >> 5;

  // One k-step: the matrix instructions on `cur`; meanwhile the slab in registers (the planes of step ks + 2,
  // fetched during the previous step) is split and stored into `nxt`, and each of its registers is refilled
  // with the data of step ks + 3 (address `kf`) as soon as it has been consumed, so that a load has a whole
  // step to land.
  auto step = [&](const unsigned char* cur, unsigned char* nxt, int kf) {
    uint4 af[TM][3];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int q = 0; q < 3; ++q)
        af[a][q] = *(const uint4*)(cur + q * C::PLANE_A + plane_off(wm * WM + a * 32 + r, ch));
    // the six partial products of one column of accumulator tiles, smallest first; the row index alternates so
    // that consecutive matrix instructions go to different accumulators
    constexpr int PA[6] = {2, 1, 0, 1, 0, 0};
    constexpr int PB[6] = {0, 1, 2, 0, 1, 0};
    auto column = [&](int b) {
      uint4 bf[3];
#pragma unroll
      for (int q = 0; q < 3; ++q)
        bf[q] = *(const uint4*)(cur + 3 * C::PLANE_A + q * C::PLANE_B + plane_off(wn * WN + b * 32 + r, ch));
#pragma unroll
      for (int pr = 0; pr < 6; ++pr)
#pragma unroll
        for (int a = 0; a < TM; ++a) acc[a][b] = mfma_bf16(af[a][PA[pr]], bf[PB[pr]], acc[a][b]);
    };
    auto chunk = [&](auto tag) {
      constexpr int c = decltype(tag)::value;
      C::template split_store<c>(slab, nxt);
      C::template load_chunk<c>(g, A, B, m0, n0, kf, slab);
    };
    // four chunks of split/store work per step: one after each column of the wide wave tile, two after each
    // column of the narrow one
    if (TN == 4) {
      column(0);
      chunk(std::integral_constant<int, 0>{});
      column(1);
      chunk(std::integral_constant<int, 1>{});
      column(TN == 4 ? 2 : 0);
      chunk(std::integral_constant<int, 2>{});
      column(TN == 4 ? 3 : 0);
      chunk(std::integral_constant<int, 3>{});
    } else {
      column(0);
      chunk(std::integral_constant<int, 0>{});
      chunk(std::integral_constant<int, 1>{});
      column(1);
      chunk(std::integral_constant<int, 2>{});
      chunk(std::integral_constant<int, 3>{});
    }
  };
  using yes = std::true_type;
  using no = std::false_type;

  // Three LDS stages: at the start of step ks the stages ks % 3 and (ks + 1) % 3 hold their steps' planes and
  // the registers hold the fp32 slab of step ks + 2; the step multiplies from the first stage, stores the
  // slab into the third (last read in step ks - 1: every wave has passed that step's barrier) and fetches
  // step ks + 3.  Fetches past the end of the contraction re-read the final slab; what they store is never
  // multiplied.
  if (nsteps > 0) {
    auto store_all = [&](unsigned char* st) {
      C::template split_store<0>(slab, st);
      C::template split_store<1>(slab, st);
      C::template split_store<2>(slab, st);
      C::template split_store<3>(slab, st);
    };
    const int k_last = k_end - XK;
    auto clampk = [&](int k) { return k < k_last ? k : k_last; };
    C::load(g, A, B, m0, n0, k_begin, slab);
    store_all(smem);
    C::load(g, A, B, m0, n0, clampk(k_begin + XK), slab);
    store_all(smem + C::STAGE);
    C::load(g, A, B, m0, n0, clampk(k_begin + 2 * XK), slab);
    __syncthreads();
    int cur = 0;
    for (int ks = 0; ks < nsteps; ++ks) {
      const int nxt = cur == 0 ? 2 : cur - 1;  // (cur + 2) % 3
      step(smem + cur * C::STAGE, smem + nxt * C::STAGE, clampk(k_begin + (ks + 3) * XK));
      __syncthreads();
      cur = cur == 2 ? 0 : cur + 1;
    }
  }

  // epilogue: C = alpha * acc + beta * C through buffer addressing (one descriptor for the wave's strip);
  // the values of a whole row of 32 x 32 sub-tiles are fetched together, then combined and stored.  Tiles
  // on the diagonal of a lower-triangular C write only the elements on or below it.
  const bool diag = g.c_lower && n0 + BN - 1 > m0;
  const int wm_u = __builtin_amdgcn_readfirstlane(wm), wn_u = __builtin_amdgcn_readfirstlane(wn);
  float* const c0 = Cm + (int64_t)(m0 + wm_u * WM) * g.ldc + n0 + wn_u * WN;
  const int lane_bytes = ((lane >> 5) * 4 * (int)g.ldc + (lane & 31)) * 4;
  const int row_bytes = (int)g.ldc * 4;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(c0, 0, 0x7fffffff, 0x00020000);
  constexpr int EB = 2;  // sub-tiles fetched together
  auto write_out = [&](auto diag_tag) {
    constexpr bool DIAG = decltype(diag_tag)::value;
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int bb = 0; bb < TN; bb += EB) {
        float cv[EB][16];
        if (g.beta != 0.f) {
#pragma unroll
          for (int e = 0; e < EB; ++e)
#pragma unroll
            for (int v = 0; v < 16; ++v)
              cv[e][v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                  rsrc, lane_bytes, (a * 32 + (v / 4) * 8 + (v & 3)) * row_bytes + (bb + e) * 128, 0));
        }
#pragma unroll
        for (int e = 0; e < EB; ++e)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int b = bb + e;
            float res = g.alpha * acc[a][b][v];
            if (g.beta != 0.f) res += g.beta * cv[e][v];
            if (DIAG) {
              const int row = m0 + wm * WM + a * 32 + (v / 4) * 8 + (lane >> 5) * 4 + (v & 3);
              const int col = n0 + wn * WN + b * 32 + (lane & 31);
              if (col > row) continue;
            }
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, res), rsrc, lane_bytes,
                                                  (a * 32 + (v / 4) * 8 + (v & 3)) * row_bytes + b * 128, 0);
          }
      }
  };
  if (diag)
    write_out(yes{});
  else
    write_out(no{});
}

template <int WM, int WN, int WAVES_M, int WAVES_N, bool TRANS_B>
int launch_x3(const GemmF32& g, hipStream_t st) {
  using C = X3<WM, WN, WAVES_M, WAVES_N, TRANS_B>;
  const int tiles_x = g.N / C::BN, tiles_y = g.M / C::BM;
  const int nb2 = g.batch2 > 1 ? g.batch2 : 1;
  const size_t smem = 3 * (size_t)C::STAGE;
  auto kern = gemm_x3_kernel<WM, WN, WAVES_M, WAVES_N, TRANS_B>;
  static bool configured = false;  // per instantiation; the attribute is idempotent, a race only repeats it
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return 1000 + (int)e;
    configured = true;
  }
  const bool by_columns = g.b_lower_tri && !g.a_lower_tri && !g.c_lower;  // as in the kernel's tile order
  const int major = by_columns ? tiles_x : tiles_y, minor = by_columns ? tiles_y : tiles_x;
  const unsigned grid_x = 8u * (unsigned)((major + 7) / 8) * (unsigned)minor;
  hipLaunchKernelGGL(kern, dim3(grid_x, 1, (unsigned)(g.batch * nb2)), dim3(C::NTHREADS), smem, st, g, tiles_x, tiles_y);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : 1000 + (int)e;
}

int g_x3_mode = 1;  // 0 = never, 1 = when the shape fits and is big enough

}  // namespace

void llmc_gemm_x3_set_mode(int mode) { g_x3_mode = mode; }

// returns -1 when the product is left to the fp32 kernel
int llmc_gemm_x3(const GemmF32& g, hipStream_t st) {
  if (!g_x3_mode || g.trans_a) return -1;
  const int nb2 = g.batch2 > 1 ? g.batch2 : 1;
  const bool aligned = (g.lda & 3) == 0 && (g.ldb & 3) == 0 && (((uintptr_t)g.A | (uintptr_t)g.B) & 15) == 0 &&
                       (g.stride_a & 3) == 0 && (g.stride_b & 3) == 0 &&
                       (nb2 == 1 || ((g.stride2_a & 3) == 0 && (g.stride2_b & 3) == 0));
  if (!aligned || g.Kc % XK || g.Kc < 64 || g.kc_last % XK) return -1;
  // the epilogue addresses a wave's strip of C with 32-bit byte offsets (up to 68 rows of ldc floats from the
  // strip's origin): wider rows than this go to the fp32 kernel's 64-bit path
  if (g.ldc >= (1 << 22)) return -1;
  // Whether a product is split depends on its own shape only, never on how many independent problems
  // (batch2) share the launch, so that a grouped call gives the bits of its single calls.  Both tile shapes
  // add the partial products of an element in the same order, so the choice between them is free.
  if (g.M % 128 || g.N % 128 || (int64_t)(g.M / 128) * (g.N / 128) * g.batch < 16) return -1;
  const int64_t nbatch = (int64_t)g.batch * nb2;
  // 256-wide tiles when they alone fill the chip (one workgroup per CU), 128-wide ones otherwise
  const bool fit256 = g.M % 256 == 0 && g.N % 256 == 0;
  int64_t t256 = fit256 ? (int64_t)(g.M / 256) * (g.N / 256) * nbatch : 0;
  if (g.c_lower && fit256) t256 = t256 / 2 + (g.M / 256) * nbatch / 2;
  if (fit256 && t256 >= 192)
    return g.trans_b ? launch_x3<64, 128, 4, 2, true>(g, st) : launch_x3<64, 128, 4, 2, false>(g, st);
  return g.trans_b ? launch_x3<64, 64, 2, 2, true>(g, st) : launch_x3<64, 64, 2, 2, false>(g, st);
}
