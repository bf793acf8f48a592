// Grouped bf16 Linear for the experts of an MoE block: y[rows of expert e] = x[rows of expert e] . W_e^T for
// every expert in one launch (reference loop: modeling/moe/linear_experts.py:235-268, one F.linear per expert
// and projection).  The routed token rows of all experts lie one expert after the other in one buffer; a
// small table names, per tile of up to 128 rows, its expert, first row and row count, so ragged token counts
// (also zero) cost no empty workgroups.  `splits` projections that read the same rows (gate and up) share a
// launch: split s takes its weights from w[s * E + e] and writes the columns s * N .. s * N + N - 1 of y.
// A tile's results go to the rows of y that its fourth table entry names (its input rows' numbers plus that
// offset), so several experts can read the same rows of x and write apart: every expert on every token.
//
// One workgroup of four waves owns a 128 x 128 tile of y (64 x 64 per wave, 2 x 2 accumulator tiles of
// v_mfma_f32_32x32x16_bf16, fp32 accumulation, one rounding to bf16 at the end as F.linear does).  A k-step is
// 64 deep: both operands arrive as 16-byte pieces (8 consecutive k of one row), are held in registers for two
// steps (two register sets, so a load has two steps to land) and stored k-contiguous into one of two LDS
// stages, a row being 128 bytes = 8 pieces with the piece index XOR-ed with bits 1..3 of the row: the sixteen
// lanes of one ds_read_b128 phase (sixteen consecutive rows, one piece index) then fall into distinct banks, and
// so do the sixteen lanes of a store (two rows, eight pieces).  Two workgroups share a CU (64 KiB of LDS each).
//
// Workgroups are dealt round-robin to the 8 XCDs; XCD x takes the row tiles x, 8 + x, ... and walks all column
// tiles of a row tile in turn, so the 128 token rows stay in that XCD's L2 while the weights stream.
#include "common.h"

namespace {

constexpr int GL_BM = 128, GL_BN = 128, GL_BK = 64;
constexpr int GL_STAGE = (GL_BM + GL_BN) * GL_BK * 2;  // bytes

struct GroupedLinear {
  const uint16_t* x;
  int64_t ldx;
  const void* const* w;
  int64_t ldw;
  uint16_t* y;
  int64_t ldy;
  const int32_t* tiles;  // [ntiles][4]: expert, first row, rows (1..128), output row of the first row minus first row
  int ntiles, experts, N, K, ncol;
};

__device__ __forceinline__ int piece_off(int row, int piece) { return row * 128 + ((piece ^ ((row >> 1) & 7)) << 4); }

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void grouped_linear_kernel(
    GroupedLinear g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [2 stages][A 128 rows | B 128 rows][128 B]
  const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const int rt = (slot / g.ncol) * 8 + xcd, ct = slot % g.ncol;
  if (rt >= g.ntiles) return;
  const int4 tile = ((const int4*)g.tiles)[rt];
  const int expert = tile.x, row0 = tile.y, nrows = tile.z;
  const int col = ct * GL_BN, split = col / g.N, n0 = col - split * g.N;
  const uint16_t* X = g.x + (int64_t)row0 * g.ldx;
  const uint16_t* W = (const uint16_t*)g.w[split * g.experts + expert] + (int64_t)n0 * g.ldw;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // piece f = tid + 256 i (i = 0..3): row f / 8, piece f % 8; rows past the tile's last re-read that last row
  const uint16_t* pa[4];
  const uint16_t* pb[4];
  int so[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int f = tid + 256 * i, row = f >> 3, piece = f & 7;
    const int ra = row < nrows ? row : nrows - 1;
    pa[i] = X + (int64_t)ra * g.ldx + piece * 8;
    pb[i] = W + (int64_t)row * g.ldw + piece * 8;
    so[i] = piece_off(row, piece);
  }
  // two register sets (p, q) of eight 16-byte pieces each; plain named registers, so none lands in scratch
#define GL_FETCH(S, k)                      \
  S##a0 = *(const uint4*)(pa[0] + (k));     \
  S##a1 = *(const uint4*)(pa[1] + (k));     \
  S##a2 = *(const uint4*)(pa[2] + (k));     \
  S##a3 = *(const uint4*)(pa[3] + (k));     \
  S##b0 = *(const uint4*)(pb[0] + (k));     \
  S##b1 = *(const uint4*)(pb[1] + (k));     \
  S##b2 = *(const uint4*)(pb[2] + (k));     \
  S##b3 = *(const uint4*)(pb[3] + (k));
#define GL_PUT(S, stage)                               \
  *(uint4*)((stage) + so[0]) = S##a0;                  \
  *(uint4*)((stage) + so[1]) = S##a1;                  \
  *(uint4*)((stage) + so[2]) = S##a2;                  \
  *(uint4*)((stage) + so[3]) = S##a3;                  \
  *(uint4*)((stage) + GL_BM * 128 + so[0]) = S##b0;    \
  *(uint4*)((stage) + GL_BM * 128 + so[1]) = S##b1;    \
  *(uint4*)((stage) + GL_BM * 128 + so[2]) = S##b2;    \
  *(uint4*)((stage) + GL_BM * 128 + so[3]) = S##b3;
  uint4 pa0, pa1, pa2, pa3, pb0, pb1, pb2, pb3, qa0, qa1, qa2, qa3, qb0, qb1, qb2, qb3;

  f32x16_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  const int r = lane & 31, ch = lane >> 5;
  auto multiply = [&](const unsigned char* stage) {
#pragma unroll
    for (int ks = 0; ks < GL_BK / 16; ++ks) {
      uint4 af[2], bf[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) af[a] = *(const uint4*)(stage + piece_off(wm * 64 + a * 32 + r, 2 * ks + ch));
#pragma unroll
      for (int b = 0; b < 2; ++b)
        bf[b] = *(const uint4*)(stage + GL_BM * 128 + piece_off(wn * 64 + b * 32 + r, 2 * ks + ch));
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[a]),
                                                              __builtin_bit_cast(bf16x8_t, bf[b]), acc[a][b], 0, 0, 0);
    }
  };

  // At the start of step s, LDS stage s % 2 holds the operands of step s, register set (s + 1) % 2 holds those of
  // step s + 1 and set s % 2 is being filled with those of step s + 2.  The step stores set (s + 1) % 2 into the
  // other stage (last read in step s - 1, which every wave has left through the barrier), refills that set with
  // step s + 3 and multiplies from its own stage.  Fetches past the end re-read the last slab; what they store is
  // never multiplied.
  const int nsteps = g.K / GL_BK;
  const int k_last = g.K - GL_BK;
  auto clampk = [&](int k) { return k < k_last ? k : k_last; };
  GL_FETCH(p, 0)
  GL_FETCH(q, clampk(GL_BK))
  GL_PUT(p, smem)
  GL_FETCH(p, clampk(2 * GL_BK))
  __syncthreads();
  for (int s = 0; s < nsteps; s += 2) {
    GL_PUT(q, smem + GL_STAGE)
    GL_FETCH(q, clampk((s + 3) * GL_BK))
    multiply(smem);
    __syncthreads();
    if (s + 1 < nsteps) {
      GL_PUT(p, smem)
      GL_FETCH(p, clampk((s + 4) * GL_BK))
      multiply(smem + GL_STAGE);
      __syncthreads();
    }
  }
#undef GL_FETCH
#undef GL_PUT

  // element v of an accumulator tile: row (v / 4) * 8 + (lane / 32) * 4 + v % 4, column lane % 32
  uint16_t* Y = g.y + ((int64_t)row0 + tile.w) * g.ldy + col;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = wm * 64 + a * 32 + (v >> 2) * 8 + ch * 4 + (v & 3);
      if (m < nrows) {
#pragma unroll
        for (int b = 0; b < 2; ++b) Y[(int64_t)m * g.ldy + wn * 64 + b * 32 + r] = f32_to_bf16_bits(acc[a][b][v]);
      }
    }
}

}  // namespace

extern "C" int llmc_grouped_linear(const void* x, int32_t dtype, int64_t ldx, const void* const* w, int64_t ldw,
                                   int32_t experts, int32_t splits, void* y, int64_t ldy, const int32_t* tiles,
                                   int32_t ntiles, int64_t N, int64_t K, void* stream) {
  LLMC_CHECK_ARG(x && w && y && tiles, 1);
  LLMC_CHECK_ARG(dtype == LLMC_BF16, 2);
  LLMC_CHECK_ARG(experts > 0 && splits > 0 && ntiles >= 0, 3);
  LLMC_CHECK_ARG(N > 0 && N % GL_BN == 0 && K > 0 && K % GL_BK == 0 && N * splits < (1 << 30) && K < (1 << 30), 4);
  LLMC_CHECK_ARG(ldx >= K && ldw >= K && ldy >= N * splits && ldx % 8 == 0 && ldw % 8 == 0, 5);
  LLMC_CHECK_ARG((((uintptr_t)x) & 15) == 0 && (((uintptr_t)tiles) & 15) == 0, 6);
  if (ntiles == 0) return 0;
  GroupedLinear g;
  g.x = (const uint16_t*)x;
  g.ldx = ldx;
  g.w = w;
  g.ldw = ldw;
  g.y = (uint16_t*)y;
  g.ldy = ldy;
  g.tiles = tiles;
  g.ntiles = ntiles;
  g.experts = experts;
  g.N = (int)N;
  g.K = (int)K;
  g.ncol = (int)(N * splits / GL_BN);
  const int64_t grid = 8 * (((int64_t)ntiles + 7) / 8) * g.ncol;
  LLMC_CHECK_ARG(grid < (1ll << 31), 7);
  static const hipError_t configured = hipFuncSetAttribute(
      (const void*)grouped_linear_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * GL_STAGE);
  if (configured != hipSuccess) return 1000 + (int)configured;
  hipLaunchKernelGGL(grouped_linear_kernel, dim3((unsigned)grid), dim3(256), 2 * GL_STAGE, (hipStream_t)stream, g);
  LLMC_LAUNCH_STATUS();
  return 0;
}
