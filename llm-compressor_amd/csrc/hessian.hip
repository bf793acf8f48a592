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
#include "gemm_f32.h"

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

// Work decomposition.  The upper-triangle tiles are numbered compactly in super-tile order (below).
// A launch is a list of phases; phase p covers tiles [tile0, tile0+ntiles) and cuts the token range
// into `split` equal chunks, one workgroup per (chunk, tile).  split == 1 is a whole tile with a
// read-modify-write epilogue.  With split > 1 every chunk stores its partial tile into the
// workspace (slot ws_tile0 + tile*split + chunk) and a second kernel sums a tile's chunks in fixed
// order and runs the same epilogue: that is how the tiles left over after the last full round of
// 256 workgroups still fill the chip, with results that do not depend on timing.
constexpr int MAX_PHASES = 4;
constexpr int PACE_SLABS = 4;          // slabs between two pacing ticks
constexpr int PACE_WINDOW = 2;         // ticks a workgroup may be ahead of the slowest member of its group
constexpr int PACE_SPIN_LIMIT = 24;    // polls before a workgroup gives up pacing
constexpr int PACE_MAX_GROUPS = 512;   // 32 slots each, at the head of the workspace
constexpr int PACE_BYTES = PACE_MAX_GROUPS * 32 * 4;
struct Phase {
  int first_wg, tile0, ntiles, split, ws_tile0;
};
struct Plan {
  int nphase;
  Phase ph[MAX_PHASES];
};

// Compact tile number c -> (I, J), J >= I.  Tiles are grouped into SH x SW super-tiles (as many
// tiles as run concurrently on one XCD), super-tiles row-major over those that reach the upper
// triangle, tiles row-major inside: workgroups sharing an L2 then touch only about SH + SW feature
// panels of X per slab instead of two each.
__device__ __forceinline__ void tile_coords(int c, int nb, int SH, int SW, int& I, int& J) {
  const int nsi = (nb + SH - 1) / SH, nsj = (nb + SW - 1) / SW;
  for (int si = 0; si < nsi; ++si) {
    for (int sj = (SH * si) / SW; sj < nsj; ++sj) {
      const int c_lo = sj * SW, c_hi = min(nb, c_lo + SW);
      for (int i = si * SH; i < min(nb, si * SH + SH); ++i) {
        const int lo = max(c_lo, i);
        const int n = c_hi - lo;
        if (n <= 0) continue;
        if (c < n) {
          I = i;
          J = lo + c;
          return;
        }
        c -= n;
      }
    }
  }
  I = J = -1;
}

// Adds alpha * acc to the BT x BT tile of H at (i0, j0) and to its mirror image.
// 32x32 accumulator layout: lane holds column n = lane&31; register v holds row
// (v/4)*8 + (lane>>5)*4 + (v&3), i.e. 4 consecutive rows per register quad.  Seen from the
// mirrored tile H[j][i] a quad is 4 consecutive floats of one row, so the read-modify-write
// runs there with 16-byte accesses (4x fewer, 4x larger requests in flight); the tile
// H[i][j] itself then only needs stores, which are row-contiguous across lanes.
template <int BT, bool FAST_EPI>
__device__ __forceinline__ void tile_epilogue(float* __restrict__ H, int64_t ldh, int K, float alpha,
                                              int assume_sym, int i0, int j0, f32x16_t (&acc)[BT / 64][BT / 64],
                                              int a_only = -1,              // >= 0: only MFMA tile row a_only
                                              float* __restrict__ slot = nullptr) {  // partial tile: raw store
  constexpr int MI = BT / 64;
  if (slot) {
    // a token chunk's partial tile: raw accumulators in register order (16 bytes per lane, coalesced)
#pragma unroll
    for (int a = 0; a < MI; ++a) {
#pragma unroll
      for (int b = 0; b < MI; ++b) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
          *(float4*)(slot + (((a * MI + b) * 4 + vq) * 256 + threadIdx.x) * 4) =
              make_float4(acc[a][b][vq * 4], acc[a][b][vq * 4 + 1], acc[a][b][vq * 4 + 2], acc[a][b][vq * 4 + 3]);
        // one MFMA tile at a time: moving many accumulators out of the AGPRs at once spills
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const bool diag = i0 == j0;
  if (FAST_EPI && i0 + BT <= K && j0 + BT <= K) {
    // interior tile: no bounds checks, so the 16-byte loads of a whole row of MFMA tiles are
    // issued back to back before the first use
#pragma unroll
    for (int a = 0; a < MI; ++a) {
      if (a_only >= 0 && a != a_only) continue;
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
    if (a_only >= 0 && a != a_only) continue;
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

// BT x BT output tile, 256 threads = 2x2 waves, each wave (BT/2)x(BT/2) = MI x MI MFMA tiles.
// LDS holds two stages of the two feature-major panels; global loads for slab s+2 are in
// flight while slab s is multiplied and slab s+1 is transposed into the other stage.
// Up to GROUP_MAX independent problems of one width K in one launch (blockIdx.y = problem), each
// with its own Hessian, activation block and token count -- the per-expert Hessians of an MoE
// layer.  The pointer table travels in the kernel arguments, so the call needs no device-side
// table and no copy.  Problems without tokens leave their Hessian untouched.
constexpr int GROUP_MAX = 128;
struct GroupArgs {
  static constexpr bool grouped = true;
  static constexpr bool segmented = false;
  float* H[GROUP_MAX];
  const uint16_t* X[GROUP_MAX];
  int T[GROUP_MAX];
};
struct NoGroup {
  static constexpr bool grouped = false;
  static constexpr bool segmented = false;
};
// One problem whose token rows lie in up to SEG_MAX separate buffers of seg_tokens rows each (a
// multiple of the slab depth, so no slab straddles two buffers; the last one may hold fewer): the
// calibration batches as the forward hook received them, without first copying them together.
constexpr int SEG_MAX = 64;
struct SegArgs {
  static constexpr bool grouped = false;
  static constexpr bool segmented = true;
  const uint16_t* X[SEG_MAX];
  int seg_tokens;
};

template <int BT, int DT, bool ALIGNED, bool FAST_EPI, class GRP>
__global__ __launch_bounds__(256) void hessian_syrk_kernel(float* __restrict__ H, int64_t ldh,
                                                            const uint16_t* __restrict__ Xfull, int64_t ldx,
                                                            int Tfull, int K, float alpha, int assume_sym,
                                                            int nb, Plan plan, float* __restrict__ ws, GRP grp,
                                                            unsigned* __restrict__ pace) {
  if constexpr (GRP::grouped) {
    Tfull = grp.T[blockIdx.y];
    if (Tfull <= 0) return;
    H = grp.H[blockIdx.y];
    Xfull = grp.X[blockIdx.y];
  }
  constexpr int RT = BT / 32;  // token rows per thread per panel
  constexpr int GI = BT / 8;   // 8-feature groups per panel
  constexpr int MI = BT / 64;
  constexpr int PANEL = BT * ROW_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [2 stages][A,B][BT][128 B]

  // Which (tile, token chunk).  Workgroups are dealt round-robin to the 8 XCDs (each with a private
  // L2), so block b runs on XCD b%8 (phases start at multiples of 8); `item` makes every XCD walk a
  // contiguous range of the phase's items, chunk-major, so the workgroups that share an L2 work on
  // neighbouring tiles over the same tokens.
  constexpr int SH = BT == 256 ? 4 : 8, SW = 8;
  int pi = 0;
  while (pi + 1 < plan.nphase && (int)blockIdx.x >= plan.ph[pi + 1].first_wg) ++pi;
  const Phase ph = plan.ph[pi];
  const int bl = blockIdx.x - ph.first_wg;
  const int items = ph.ntiles * ph.split;
  const int per_xcd = (items + 7) / 8;
  const int item = (bl % 8) * per_xcd + bl / 8;
  if (item >= items || bl / 8 >= per_xcd) return;
  const int chunk = item / ph.ntiles;
  const int nslab_all = (Tfull + BK - 1) / BK;
  const int cs = (nslab_all + ph.split - 1) / ph.split;  // slabs per chunk
  const int s_begin = chunk * cs;
  if (s_begin >= nslab_all) return;
  const int t_begin = s_begin * BK;
  const int T = min(Tfull, (s_begin + cs) * BK) - t_begin;  // tokens of this chunk
  const uint16_t* X = Xfull + (int64_t)t_begin * ldx;
  const bool partial = ph.split > 1;
  int I, J;
  tile_coords(ph.tile0 + item % ph.ntiles, nb, SH, SW, I, J);
  if (I < 0) return;
  const int i0 = I * BT, j0 = J * BT;
  const bool diag = (I == J);

  const int tid = threadIdx.x;
  // Pacing.  The 32 workgroups that run together on one XCD share feature panels through that XCD's
  // L2, but only while they work on nearby slabs; nothing in the kernel keeps them together (the
  // loads run two slabs ahead, so a workgroup that is ahead is not slowed by its cache misses), and
  // over a thousand slabs they drift apart until every panel is fetched once per workgroup.  Every
  // PACE_SLABS slabs a workgroup publishes its tick number in its own slot of the group's 128-byte
  // line and its first wave reads all 32 slots; a slab later, when the values have arrived, it holds
  // the workgroup back while it is more than PACE_WINDOW ticks ahead of the slowest member.  Plain
  // stores and loads to distinct words, no read-modify-write.  The wait is bounded: a workgroup that
  // times out (its group is not resident together) stops pacing for good.
  unsigned* const my_group = pace + 32 * ((bl % 8) + 8 * ((bl / 8) / 32));
  const int my_member = (bl / 8) % 32;
  bool pacing = pace != nullptr && pi == 0 && ph.split == 1 && ph.ntiles % (8 * 32) == 0 && tid < 64;
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
  // Segmented input: address of token t0 of this chunk (t0 a slab start, uniform over the workgroup, so
  // the table of buffers is indexed by a scalar).  A slab that does not exist maps to the last one.
  auto slab_base = [&](int t0) -> const uint16_t* {
    if constexpr (GRP::segmented) {
      const int g = __builtin_amdgcn_readfirstlane(t_begin + min(t0, ((T - 1) / BK) * BK));
      const int sg = g / grp.seg_tokens;
      return grp.X[sg] + (int64_t)(g - sg * grp.seg_tokens) * ldx;
    } else {
      return X + (int64_t)t0 * ldx;
    }
  };
  // row r of this thread's RT token rows of the slab at t0, features col0 + g_i*8 .. (+8)
  auto load_row = [&](int t0, int r, int col0) -> uint4 {
    if constexpr (GRP::segmented) {
      const int t0c = min(t0, ((T - 1) / BK) * BK);
      const int tt = min(t0 + g_t * RT + r, T - 1) - t0c;  // rows past T: the last row (masked by the caller)
      return *(const uint4*)(slab_base(t0) + (int64_t)tt * ldx + min(col0 + g_i * 8, K - 8));
    } else {
      return load8<ALIGNED>(X, ldx, t0 + g_t * RT + r, col0 + g_i * 8, T, K);
    }
  };
  auto load_panel = [&](uint4* rg, int t0, int col0) {
#pragma unroll
    for (int r = 0; r < RT; ++r) rg[r] = load_row(t0, r, col0);
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
  // fragment number n of 16-token group ks of the stage at `stA`, in the order the matrix ops first
  // need them: A rows 0, then all B rows, then the remaining A rows.  Two register sets (ks & 1).
  uint4 fa[2][MI], fb[2][MI];
  auto read_frag = [&](const unsigned char* stA, int ks, int n) {
    const int f = n == 0 ? 0 : (n <= MI ? MI + n - 1 : n - MI);  // f < MI -> A rows, else B rows
    const int q = ks * 2 + (lane >> 5);
    if (f < MI)
      fa[ks & 1][f] = *(const uint4*)(stA + chunk_off(wm * (BT / 2) + f * 32 + (lane & 31), q));
    else
      fb[ks & 1][f - MI] = *(const uint4*)(stA + PANEL + chunk_off(wn * (BT / 2) + (f - MI) * 32 + (lane & 31), q));
  };
  // One slab of matrix ops from stage `cur`, written out as an explicit software pipeline: the
  // slab is four groups of 16 tokens, each group NSTEP steps of two MFMAs, and every step also
  // issues its share of (1) the LDS reads of the next group's operand fragments (double-buffered
  // in registers), (2) when STORE, the transposing LDS writes of the next slab -- first panel
  // during group 0, second during group 2 -- and (3) the global loads that refill each register
  // set during the following group (slab after next, starting at token t2).  A scheduling fence
  // after every step keeps the compiler from regrouping them; with one wave per SIMD nothing
  // else would cover a stall.
  // The fragments of the slab's first group are already in registers.  The workgroup barrier
  // sits after the third group: by then every wave has issued all its reads of stage `cur` and all
  // its writes of stage `nxt`, so the fourth group can already fetch the next slab's first
  // fragments from `nxt` and the slab boundary costs neither a barrier wait nor an LDS round trip.
  // Row pointers of the slab the steady state loads next (token t2 + g_t*RT, this thread's 8 features
  // of either panel): while that slab is a full one no clamping is needed and a load is one 64-bit
  // add away from them.
  const uint16_t* pA = slab_base(2 * BK) + (int64_t)(g_t * RT) * ldx + min(i0 + g_i * 8, K - 8);
  const uint16_t* pB = slab_base(2 * BK) + (int64_t)(g_t * RT) * ldx + min(j0 + g_i * 8, K - 8);
  // after the iteration that loaded slab s+2: on to slab s+3, which may begin another buffer
  auto advance = [&](int s_done) {
    if constexpr (GRP::segmented) {
      const int g = __builtin_amdgcn_readfirstlane(t_begin + (s_done + 3) * BK);
      if (g % grp.seg_tokens == 0) {
        pA = slab_base((s_done + 3) * BK) + (int64_t)(g_t * RT) * ldx + min(i0 + g_i * 8, K - 8);
        pB = slab_base((s_done + 3) * BK) + (int64_t)(g_t * RT) * ldx + min(j0 + g_i * 8, K - 8);
        return;
      }
    }
    pA += (int64_t)BK * ldx;
    pB += (int64_t)BK * ldx;
  };
  auto compute = [&](unsigned char* curA, unsigned char* nxtA, int t2, auto store_tag, auto mask_tag,
                     auto direct_tag) {
    constexpr bool STORE = decltype(store_tag)::value;
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr bool DIRECT = decltype(direct_tag)::value && ALIGNED;  // unclamped loads through pA / pB
    constexpr int MPS = 2, NSTEP = MI * MI / MPS;  // matrix ops per step, steps per 16-token group
    constexpr int FPS = 2 * MI / NSTEP, CPS = 8 / NSTEP, LPS = RT / NSTEP;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (STORE && MASK && ks == 0) mask_tail(ra, t2 - BK);
      if (STORE && MASK && ks == 2) mask_tail(rb, t2 - BK);
#pragma unroll
      for (int st = 0; st < NSTEP; ++st) {
#pragma unroll
        for (int f = st * FPS; f < (st + 1) * FPS; ++f) {
          if (ks + 1 < BK / 16)
            read_frag(curA, ks + 1, f);
          else if (STORE)
            read_frag(nxtA, 0, f);
        }
        if (STORE) {
#pragma unroll
          for (int c = st * CPS; c < (st + 1) * CPS; ++c) {
            if (ks == 0) store_col(nxtA, ra, c);
            if (ks == 2) store_col(nxtA + PANEL, rb, c);
          }
#pragma unroll
          for (int r = st * LPS; r < (st + 1) * LPS; ++r) {
            if (DIRECT) {
              if (ks == 1) ra[r] = *(const uint4*)(pA + (int64_t)r * ldx);
              if (ks == 3) rb[r] = *(const uint4*)(pB + (int64_t)r * ldx);
            } else {
              if (ks == 1) ra[r] = load_row(t2, r, i0);
              if (ks == 3) rb[r] = load_row(t2, r, j0);
            }
          }
        }
#pragma unroll
        for (int m = st * MPS; m < (st + 1) * MPS; ++m)
          acc[m / MI][m % MI] = Mfma<DT>::run(fa[ks & 1][m / MI], fb[ks & 1][m % MI], acc[m / MI][m % MI]);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (STORE && ks == 2) {
        __syncthreads();
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
#pragma unroll
  for (int f = 0; f < 2 * MI; ++f) read_frag(smem, 0, f);
  __builtin_amdgcn_sched_barrier(0);
  // steady state: slab s multiplied, slab s+1 transposed into the other stage, slab s+2 in flight;
  // first the iterations whose slab s+2 is a full one (direct loads), then at most one with clamped loads
  const int nfull = T / BK;
  int s = 0;
  const int ndirect = max(0, min(nslab - 2, nfull - 2));  // iterations whose slab s+2 is a full one
  unsigned seen = 0xffffffffu;  // the group's slots as read one period ago (lane m: member m)
  for (; s + PACE_SLABS <= ndirect; s += PACE_SLABS) {
    if (pacing) {  // uniform over the first wave, false in the others
      const unsigned my_tick = (unsigned)(s / PACE_SLABS);
      int spins = 0;
      while (true) {
        // lanes 32..63 hold 0xffffffff; any member more than PACE_WINDOW ticks behind holds us back
        if (__builtin_amdgcn_ballot_w64(my_tick > seen && my_tick - seen > (unsigned)PACE_WINDOW) == 0) break;
        if (++spins == PACE_SPIN_LIMIT) {
          pacing = false;
          break;
        }
        __builtin_amdgcn_s_sleep(8);
        if (tid < 32) seen = __hip_atomic_load(my_group + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (tid == 0) __hip_atomic_store(my_group + my_member, my_tick + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tid < 32) seen = __hip_atomic_load(my_group + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    for (int i = 0; i < PACE_SLABS; ++i) {
      compute(smem + ((s + i) & 1) * 2 * PANEL, smem + ((s + i + 1) & 1) * 2 * PANEL, (s + i + 2) * BK,
              std::true_type{}, std::false_type{}, std::true_type{});
      advance(s + i);
    }
  }
  for (; s < ndirect; ++s) {
    compute(smem + (s & 1) * 2 * PANEL, smem + ((s + 1) & 1) * 2 * PANEL, (s + 2) * BK, std::true_type{},
            std::false_type{}, std::true_type{});
    advance(s);
  }
  for (; s + 2 < nslab; ++s)
    compute(smem + (s & 1) * 2 * PANEL, smem + ((s + 1) & 1) * 2 * PANEL, (s + 2) * BK, std::true_type{},
            std::false_type{}, std::false_type{});
  if (nslab >= 2) {
    s = nslab - 2;
    compute(smem + (s & 1) * 2 * PANEL, smem + ((s + 1) & 1) * 2 * PANEL, (s + 2) * BK, std::true_type{},
            std::true_type{}, std::false_type{});
  }
  compute(smem + ((nslab - 1) & 1) * 2 * PANEL, smem, 0, std::false_type{}, std::false_type{}, std::false_type{});

  float* slot = partial ? ws + (int64_t)(ph.ws_tile0 + (item % ph.ntiles) * ph.split + chunk) * (BT * BT) : nullptr;
  tile_epilogue<BT, FAST_EPI>(H, ldh, K, alpha, assume_sym, i0, j0, acc, -1, slot);
}

// Sums the chunks of a split tile in fixed order and applies the tile epilogue; one workgroup per
// (tile, row of MFMA tiles), the loads of two chunks in flight at a time.
template <int BT, bool FAST_EPI>
__global__ __launch_bounds__(256) void hessian_reduce_kernel(float* __restrict__ H, int64_t ldh, int Tfull, int K,
                                                              float alpha, int assume_sym, int nb, Plan plan,
                                                              int first_split_phase, const float* __restrict__ ws) {
  constexpr int MI = BT / 64;
  constexpr int SH = BT == 256 ? 4 : 8, SW = 8;
  int pi = first_split_phase, t = blockIdx.x / MI;
  const int a = blockIdx.x % MI;
  while (t >= plan.ph[pi].ntiles) t -= plan.ph[pi++].ntiles;
  const Phase ph = plan.ph[pi];
  int I, J;
  tile_coords(ph.tile0 + t, nb, SH, SW, I, J);
  if (I < 0) return;
  const int nslab_all = (Tfull + BK - 1) / BK;
  const int cs = (nslab_all + ph.split - 1) / ph.split;
  int nchunk = ph.split;
  while (nchunk > 0 && (nchunk - 1) * cs >= nslab_all) --nchunk;  // trailing chunks without tokens wrote nothing
  float4 sum[MI][4];
#pragma unroll
  for (int b = 0; b < MI; ++b)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) sum[b][vq] = make_float4(0.f, 0.f, 0.f, 0.f);
  const float* base = ws + (int64_t)(ph.ws_tile0 + t * ph.split) * (BT * BT) + (a * MI * 4 * 256 + threadIdx.x) * 4;
  auto load = [&](int chunk, float4 (&p)[MI][4]) {
#pragma unroll
    for (int b = 0; b < MI; ++b)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq)
        p[b][vq] = *(const float4*)(base + (int64_t)chunk * (BT * BT) + ((b * 4 + vq) * 256) * 4);
  };
  auto add = [&](const float4 (&p)[MI][4]) {
#pragma unroll
    for (int b = 0; b < MI; ++b)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        sum[b][vq].x += p[b][vq].x;
        sum[b][vq].y += p[b][vq].y;
        sum[b][vq].z += p[b][vq].z;
        sum[b][vq].w += p[b][vq].w;
      }
  };
  int chunk = 0;
  for (; chunk + 1 < nchunk; chunk += 2) {
    float4 p0[MI][4], p1[MI][4];
    load(chunk, p0);
    load(chunk + 1, p1);
    add(p0);
    add(p1);
  }
  if (chunk < nchunk) {
    float4 p0[MI][4];
    load(chunk, p0);
    add(p0);
  }
  f32x16_t acc[MI][MI];
#pragma unroll
  for (int aa = 0; aa < MI; ++aa)
#pragma unroll
    for (int b = 0; b < MI; ++b)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const bool mine = aa == a;
        acc[aa][b][vq * 4] = mine ? sum[b][vq].x : 0.f;
        acc[aa][b][vq * 4 + 1] = mine ? sum[b][vq].y : 0.f;
        acc[aa][b][vq * 4 + 2] = mine ? sum[b][vq].z : 0.f;
        acc[aa][b][vq * 4 + 3] = mine ? sum[b][vq].w : 0.f;
      }
  tile_epilogue<BT, FAST_EPI>(H, ldh, K, alpha, assume_sym, I * BT, J * BT, acc, a);
}

constexpr int NUM_WG = 256;  // workgroups that run at once: one per CU (LDS and registers allow no more)

struct Choice {
  int bt = 0;
  Plan plan;
  int first_split_phase = 0;  // == plan.nphase when no phase is split
  int nsplit_tiles = 0;
  int64_t ws_bytes = 0;
  double time_us = 0;
  int grid = 0;
};

// Phases for BT-wide tiles.  Whole rounds of NUM_WG tiles first.  When `split`, the R tiles left
// over are cut along the tokens so that they fill a round too: R <= 128 -> one phase of
// floor(256/R) chunks per tile; R > 128 -> 128 tiles in two chunks, then the rest as before.  A
// chunk keeps at least 4 slabs.  time_us is a rough model (measured microseconds per slab and per
// epilogue of one tile, partial tiles through the workspace at 3 TB/s) used only to pick between
// candidates.
Choice make_choice(int bt, int64_t T, int64_t K, bool split) {
  Choice c;
  c.bt = bt;
  const int nb = (int)((K + bt - 1) / bt);
  const int nt = nb * (nb + 1) / 2;
  const int nslab = (int)((T + BK - 1) / BK);
  const double slab_us = bt == 256 ? 1.75 : 0.7, epi_us = bt == 256 ? 35.0 : 10.0, chunk_epi_us = 5.0;
  Plan& plan = c.plan;
  plan.nphase = 0;
  int wg = 0, tile0 = 0, ws_tile = 0;
  auto push = [&](int ntiles, int sp) {
    Phase& p = plan.ph[plan.nphase++];
    p.first_wg = wg;
    p.tile0 = tile0;
    p.ntiles = ntiles;
    p.split = sp;
    p.ws_tile0 = ws_tile;
    const int items = ntiles * sp;
    wg += ((items + 7) / 8) * 8;
    tile0 += ntiles;
    if (sp > 1) ws_tile += items;
    const int rounds = (items + NUM_WG - 1) / NUM_WG;
    c.time_us += rounds * (((nslab + sp - 1) / sp) * slab_us + (sp > 1 ? chunk_epi_us : epi_us));
  };
  int slimit = nslab / 4;
  if (slimit > 16) slimit = 16;
  int rem = nt;
  if (!split || slimit < 2) {
    push(nt, 1);
    rem = 0;
  } else {
    const int whole = (rem / NUM_WG) * NUM_WG;
    if (whole > 0) push(whole, 1);
    rem -= whole;
  }
  c.first_split_phase = plan.nphase;
  if (rem > NUM_WG / 2) {
    push(NUM_WG / 2, 2);
    rem -= NUM_WG / 2;
  }
  if (rem > 0) {
    int sp = NUM_WG / rem;
    if (sp > slimit) sp = slimit;
    push(rem, sp);  // (sp == 1 cannot happen here: rem <= 128 and slimit >= 2)
  }
  c.nsplit_tiles = nt - (c.first_split_phase < plan.nphase ? plan.ph[c.first_split_phase].tile0 : nt);
  c.ws_bytes = (int64_t)ws_tile * bt * bt * 4;
  c.time_us += c.ws_bytes * 2 / 3e6 + (ws_tile ? 15.0 : 0.0);  // partial tiles written and read back, reduce kernel
  c.grid = wg;
  return c;
}

// the fastest of {128, 256}-wide tiles x {whole tiles, token chunks} that fits the workspace
Choice choose(int64_t T, int64_t K, int64_t ws_avail) {
  Choice best;
  for (int bt : {256, 128})
    for (int split = 0; split < 2; ++split) {
      const Choice c = make_choice(bt, T, K, split != 0);
      if (c.ws_bytes > ws_avail) continue;
      if (best.bt == 0 || c.time_us < best.time_us) best = c;
    }
  return best;
}

__global__ void zero_u32_kernel(unsigned* p, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) p[i] = 0u;
}

template <int BT, int DT>
int launch(const Choice& c, float* H, int64_t ldh, const void* X, int64_t ldx, int64_t T, int64_t K, float alpha,
           int flags, float* ws, unsigned* pace, hipStream_t st, const SegArgs* segs = nullptr) {
  const int nb = (int)((K + BT - 1) / BT);
  const bool aligned = segs || ((K % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)X & 15) == 0));
  const int sym = (flags & LLMC_HESSIAN_ASSUME_SYMMETRIC) ? 1 : 0;
  const int vec_ok = ((ldh & 3) == 0 && ((uintptr_t)H & 15) == 0) ? 1 : 0;
  constexpr int smem = 4 * BT * ROW_BYTES;
  // 16-byte read-modify-write epilogue needs a symmetric H and 16-byte aligned rows
  const bool fast = sym && vec_ok;
  auto kern = aligned ? (fast ? hessian_syrk_kernel<BT, DT, true, true, NoGroup> : hessian_syrk_kernel<BT, DT, true, false, NoGroup>)
                      : (fast ? hessian_syrk_kernel<BT, DT, false, true, NoGroup> : hessian_syrk_kernel<BT, DT, false, false, NoGroup>);
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return 1000 + (int)e;
  }
  // pacing slots: 32 per (round of whole tiles, XCD); only worth it for long token loops
  const Phase& p0 = c.plan.ph[0];
  const int pace_groups = (p0.split == 1 && p0.ntiles % NUM_WG == 0) ? p0.ntiles / 32 : 0;
  if (pace_groups == 0 || pace_groups > PACE_MAX_GROUPS || T < 64 * BK) pace = nullptr;
  if (pace) {
    hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(256), 0, st, pace, pace_groups * 32);
    LLMC_LAUNCH_STATUS();
  }
  if (segs) {
    auto skern = fast ? hessian_syrk_kernel<BT, DT, true, true, SegArgs> : hessian_syrk_kernel<BT, DT, true, false, SegArgs>;
    if (smem > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void*)skern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return 1000 + (int)e;
    }
    hipLaunchKernelGGL(skern, dim3(c.grid), dim3(256), smem, st, H, ldh, (const uint16_t*)nullptr, ldx, (int)T,
                       (int)K, alpha, sym, nb, c.plan, ws, *segs, pace);
  } else {
    hipLaunchKernelGGL(kern, dim3(c.grid), dim3(256), smem, st, H, ldh, (const uint16_t*)X, ldx, (int)T,
                       (int)K, alpha, sym, nb, c.plan, ws, NoGroup{}, pace);
  }
  LLMC_LAUNCH_STATUS();
  if (c.nsplit_tiles > 0) {
    if (fast)
      hipLaunchKernelGGL((hessian_reduce_kernel<BT, true>), dim3(c.nsplit_tiles * (BT / 64)), dim3(256), 0, st, H, ldh,
                         (int)T, (int)K, alpha, sym, nb, c.plan, c.first_split_phase, ws);
    else
      hipLaunchKernelGGL((hessian_reduce_kernel<BT, false>), dim3(c.nsplit_tiles * (BT / 64)), dim3(256), 0, st, H, ldh,
                         (int)T, (int)K, alpha, sym, nb, c.plan, c.first_split_phase, ws);
    LLMC_LAUNCH_STATUS();
  }
  return 0;
}

}  // namespace

extern "C" int64_t llmc_hessian_workspace_bytes(int64_t T, int64_t K) {
  if (T <= 0 || K <= 0 || K >= (1 << 30)) return 0;
  return choose(T, K, INT64_MAX).ws_bytes + PACE_BYTES;
}

extern "C" int llmc_hessian_accumulate(float* H, int64_t ldh, const void* X, int64_t ldx, int64_t T,
                                       int64_t K, int32_t x_dtype, float alpha, int32_t flags,
                                       void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(H != nullptr, 1);
  LLMC_CHECK_ARG(K > 0 && K < (1 << 30) && ldh >= K, 2);
  LLMC_CHECK_ARG(T >= 0 && T < (1ll << 31), 5);
  if (T == 0) return 0;
  LLMC_CHECK_ARG(X != nullptr, 3);
  LLMC_CHECK_ARG(ldx >= K, 4);
  LLMC_CHECK_ARG(x_dtype == LLMC_BF16 || x_dtype == LLMC_F16 || x_dtype == LLMC_F32, 7);
  LLMC_CHECK_ARG(workspace_bytes >= 0 && (workspace_bytes == 0 || workspace != nullptr), 10);
  LLMC_CHECK_ARG((((uintptr_t)workspace) & 15) == 0, 10);
  hipStream_t st = (hipStream_t)stream;
  if (x_dtype == LLMC_F32) {
    // fp32 activations: the whole K x K product X^T X on the fp32 matrix-core GEMM (every element of H is
    // read-modify-written; tile (i,j) and tile (j,i) form the same products in the same order, so a
    // symmetric H stays bitwise symmetric)
    LLMC_CHECK_ARG(K < (1ll << 31) - 256 && T < (1ll << 31) - 256, 5);
    GemmF32 g = {};
    g.A = (const float*)X;
    g.lda = ldx;
    g.trans_a = 1;
    g.B = (const float*)X;
    g.ldb = ldx;
    g.C = H;
    g.ldc = ldh;
    g.M = (int)K;
    g.N = (int)K;
    g.Kc = (int)T;
    g.alpha = alpha;
    g.beta = 1.f;
    g.batch = 1;
    return llmc_gemm_f32(g, st);
  }
  // 256-wide tiles need half the LDS traffic per matrix op of 128-wide ones; token chunks spread a
  // tile count that is not a multiple of the CU count over the whole chip
  // workspace layout: [pacing counters, PACE_BYTES][partial tiles of the token chunks]
  const int64_t avail = workspace ? workspace_bytes : 0;
  const bool pace_room = avail >= PACE_BYTES;
  const Choice c = choose(T, K, pace_room ? avail - PACE_BYTES : avail);
  unsigned* pace = pace_room ? (unsigned*)workspace : nullptr;
  float* ws = (float*)((char*)workspace + (pace_room ? PACE_BYTES : 0));
  if (x_dtype == LLMC_BF16)
    return c.bt == 256 ? launch<256, LLMC_BF16>(c, H, ldh, X, ldx, T, K, alpha, flags, ws, pace, st)
                       : launch<128, LLMC_BF16>(c, H, ldh, X, ldx, T, K, alpha, flags, ws, pace, st);
  return c.bt == 256 ? launch<256, LLMC_F16>(c, H, ldh, X, ldx, T, K, alpha, flags, ws, pace, st)
                     : launch<128, LLMC_F16>(c, H, ldh, X, ldx, T, K, alpha, flags, ws, pace, st);
}

extern "C" int llmc_hessian_accumulate_segments(float* H, int64_t ldh, const void* const* X, int32_t n_seg,
                                                int64_t seg_tokens, int64_t last_tokens, int64_t ldx, int64_t K,
                                                int32_t x_dtype, float alpha, int32_t flags, void* workspace,
                                                int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(H != nullptr, 1);
  LLMC_CHECK_ARG(K > 0 && K < (1 << 30) && K % 8 == 0 && ldh >= K, 8);
  LLMC_CHECK_ARG(X != nullptr, 3);
  LLMC_CHECK_ARG(n_seg >= 0 && n_seg <= SEG_MAX, 4);
  if (n_seg == 0) return 0;
  LLMC_CHECK_ARG(seg_tokens > 0 && seg_tokens % BK == 0 && seg_tokens < (1ll << 30), 5);
  LLMC_CHECK_ARG(last_tokens > 0 && last_tokens <= seg_tokens, 6);
  LLMC_CHECK_ARG(ldx >= K && ldx % 8 == 0, 7);
  LLMC_CHECK_ARG(x_dtype == LLMC_BF16 || x_dtype == LLMC_F16, 9);
  LLMC_CHECK_ARG(workspace_bytes >= 0 && (workspace_bytes == 0 || workspace != nullptr), 12);
  LLMC_CHECK_ARG((((uintptr_t)workspace) & 15) == 0, 12);
  const int64_t T = (int64_t)(n_seg - 1) * seg_tokens + last_tokens;
  LLMC_CHECK_ARG(T < (1ll << 31), 5);
  SegArgs segs;
  for (int i = 0; i < SEG_MAX; ++i) {
    const void* p = X[i < n_seg ? i : n_seg - 1];
    LLMC_CHECK_ARG(p != nullptr && (((uintptr_t)p) & 15) == 0, 3);
    segs.X[i] = (const uint16_t*)p;
  }
  segs.seg_tokens = (int)seg_tokens;
  hipStream_t st = (hipStream_t)stream;
  const int64_t avail = workspace ? workspace_bytes : 0;
  const bool pace_room = avail >= PACE_BYTES;
  const Choice c = choose(T, K, pace_room ? avail - PACE_BYTES : avail);
  unsigned* pace = pace_room ? (unsigned*)workspace : nullptr;
  float* ws = (float*)((char*)workspace + (pace_room ? PACE_BYTES : 0));
  if (x_dtype == LLMC_BF16)
    return c.bt == 256 ? launch<256, LLMC_BF16>(c, H, ldh, nullptr, ldx, T, K, alpha, flags, ws, pace, st, &segs)
                       : launch<128, LLMC_BF16>(c, H, ldh, nullptr, ldx, T, K, alpha, flags, ws, pace, st, &segs);
  return c.bt == 256 ? launch<256, LLMC_F16>(c, H, ldh, nullptr, ldx, T, K, alpha, flags, ws, pace, st, &segs)
                     : launch<128, LLMC_F16>(c, H, ldh, nullptr, ldx, T, K, alpha, flags, ws, pace, st, &segs);
}

template <int BT, int DT>
int launch_grouped(const GroupArgs& grp, int n, int64_t ldh, int64_t ldx, int64_t K, float alpha, int sym, bool fast,
                   hipStream_t st) {
  const Choice c = make_choice(BT, /*T=*/64, K, /*split=*/false);  // whole tiles: one phase over all of them
  const int nb = (int)((K + BT - 1) / BT);
  constexpr int smem = 4 * BT * ROW_BYTES;
  auto kern = fast ? hessian_syrk_kernel<BT, DT, true, true, GroupArgs> : hessian_syrk_kernel<BT, DT, true, false, GroupArgs>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return 1000 + (int)e;
  }
  hipLaunchKernelGGL(kern, dim3(c.grid, n), dim3(256), smem, st, (float*)nullptr, ldh, (const uint16_t*)nullptr, ldx, 0,
                     (int)K, alpha, sym, nb, c.plan, (float*)nullptr, grp, (unsigned*)nullptr);
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int llmc_hessian_accumulate_grouped(float* const* H, int64_t ldh, const void* const* X, int64_t ldx,
                                               const int64_t* T, int32_t n, int64_t K, int32_t x_dtype,
                                               float alpha, int32_t flags, void* stream) {
  LLMC_CHECK_ARG(H != nullptr && n >= 0, 1);
  LLMC_CHECK_ARG(K > 0 && K < (1 << 30) && K % 8 == 0 && ldh >= K, 2);
  LLMC_CHECK_ARG(X != nullptr, 3);
  LLMC_CHECK_ARG(ldx >= K && ldx % 8 == 0, 4);
  LLMC_CHECK_ARG(T != nullptr, 5);
  LLMC_CHECK_ARG(x_dtype == LLMC_BF16 || x_dtype == LLMC_F16, 8);
  hipStream_t st = (hipStream_t)stream;
  const int sym = (flags & LLMC_HESSIAN_ASSUME_SYMMETRIC) ? 1 : 0;
  bool fast = sym && (ldh & 3) == 0;
  for (int i = 0; i < n; ++i) {
    LLMC_CHECK_ARG(T[i] >= 0 && T[i] < (1ll << 31), 5);
    if (T[i] == 0) continue;
    LLMC_CHECK_ARG(H[i] != nullptr, 1);
    LLMC_CHECK_ARG(X[i] != nullptr && (((uintptr_t)X[i]) & 15) == 0, 3);
    if (((uintptr_t)H[i]) & 15) fast = false;
  }
  const bool big = K >= 512;
  for (int base = 0; base < n; base += GROUP_MAX) {
    const int cnt = (n - base) < GROUP_MAX ? (n - base) : GROUP_MAX;
    GroupArgs grp;
    bool any = false;
    for (int i = 0; i < cnt; ++i) {
      grp.H[i] = H[base + i];
      grp.X[i] = (const uint16_t*)X[base + i];
      grp.T[i] = (int)T[base + i];
      any = any || T[base + i] > 0;
    }
    if (!any) continue;
    int rc;
    if (x_dtype == LLMC_BF16)
      rc = big ? launch_grouped<256, LLMC_BF16>(grp, cnt, ldh, ldx, K, alpha, sym, fast, st)
               : launch_grouped<128, LLMC_BF16>(grp, cnt, ldh, ldx, K, alpha, sym, fast, st);
    else
      rc = big ? launch_grouped<256, LLMC_F16>(grp, cnt, ldh, ldx, K, alpha, sym, fast, st)
               : launch_grouped<128, LLMC_F16>(grp, cnt, ldh, ldx, K, alpha, sym, fast, st);
    if (rc) return rc;
  }
  return 0;
}

extern "C" int llmc_version(void) { return 1; }
