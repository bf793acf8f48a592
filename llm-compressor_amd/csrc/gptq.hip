// GPTQ quantize_weight: blocked column loop with error feedback.
//
// Rows of W are independent given the inverse-Hessian factor U, so a workgroup owns a set of rows and never
// synchronises with another one inside a block of columns.  The block's 128x128 slice of U sits in LDS, a
// row's columns of the block in registers.  Per column: quantise, form err = (w - q)/U[i][i] and subtract
// err * U[i][c] from the columns behind it (U is zero below the diagonal, so no masking is needed).
//   * quantiser (gptq_block_kernel): 4 lanes per row, 32 columns per lane as 8 runs of 4 neighbouring
//     columns; a run is quantised start to finish inside its lane (layout described at the Q* constants).
//   * SparseGPT (sgpt_block_kernel): 16 lanes per row, 8 columns per lane; the column's value and prune flag
//     are broadcast inside the team and every lane forms the error.
// After the block, W[:, i2:] -= Err * U[i1:i2, i2:] runs as a matrix-core GEMM (llmc_gemm_f32).
#include <vector>

#include "gemm_f32.h"
#include "qformat.h"

namespace {

constexpr int GB = 128;       // widest column block held on chip
constexpr int GROUP = 4;      // column blocks whose updates of the far columns are applied together
constexpr int TEAM = 16;      // lanes per row
constexpr int CPL = GB / TEAM;  // columns per lane (8)
constexpr int ROWS_PER_WG = 256 / TEAM;

// One problem of a grouped call (llmc_gptq_quantize_grouped); the kernels pick theirs by a grid index and
// find its work buffers at a fixed stride behind those of problem 0.
struct GptqItem {
  const void* weight;
  const void* scale;
  const int8_t* zp;
  const float* gscale;
  const int32_t* g_idx;
  void* out;
};

template <int WDT>
__global__ __launch_bounds__(256) void gptq_prepare_w_kernel(const void* __restrict__ w, int64_t ldw, int R,
                                                             int K, const int32_t* __restrict__ perm,
                                                             const uint8_t* __restrict__ dead,
                                                             float* __restrict__ Wf,
                                                             const GptqItem* __restrict__ items = nullptr) {
  if (items) {  // grouped: problem blockIdx.z, perm / dead rows of [n,K] arrays
    w = items[blockIdx.z].weight;
    if (perm) perm += (int64_t)blockIdx.z * K;
    if (dead) dead += (int64_t)blockIdx.z * K;
    Wf += (int64_t)blockIdx.z * R * K;
  }
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (c >= K) return;
  const int src = perm ? perm[c] : c;
  float v = load_as_f32<WDT>(w, (int64_t)r * ldw + src);
  if (dead && dead[c]) v = 0.f;
  Wf[(int64_t)r * K + c] = v;
}

// Row-at-a-time forms of the column gather / scatter for a permuted column order (activation ordering): one
// workgroup moves one row through LDS, so global memory sees whole rows and the random accesses stay on chip.
// Rows of up to ROW_STAGE_MAX fp32 values fit; wider ones keep the element-wise kernels.
constexpr int ROW_STAGE_MAX = 16384;

template <int WDT>
__global__ __launch_bounds__(1024) void gptq_prepare_w_rows_kernel(const void* __restrict__ w, int64_t ldw, int R,
                                                                  int K, const int32_t* __restrict__ perm,
                                                                  const uint8_t* __restrict__ dead,
                                                                  float* __restrict__ Wf,
                                                                  const GptqItem* __restrict__ items) {
  extern __shared__ float rowbuf[];
  if (items) {
    w = items[blockIdx.y].weight;
    perm += (int64_t)blockIdx.y * K;
    if (dead) dead += (int64_t)blockIdx.y * K;
    Wf += (int64_t)blockIdx.y * R * K;
  }
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;  // 256 threads, 1024 for rows above 8192 values
  constexpr int BATCH = 8;
  for (int c0 = 0; c0 < K; c0 += nt * BATCH) {
    float v[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      v[b] = load_as_f32<WDT>(w, (int64_t)r * ldw + (c < K ? c : K - 1));
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      if (c < K) rowbuf[c] = v[b];
    }
  }
  __syncthreads();
  for (int c = tid; c < K; c += nt) {
    float v = rowbuf[perm[c]];
    if (dead && dead[c]) v = 0.f;
    Wf[(int64_t)r * K + c] = v;
  }
}

template <int WDT>
__global__ __launch_bounds__(1024) void gptq_finalize_rows_kernel(const float* __restrict__ Wf, int R, int K,
                                                                 const int32_t* __restrict__ perm,
                                                                 void* __restrict__ out, int64_t ldo,
                                                                 const GptqItem* __restrict__ items) {
  extern __shared__ float rowbuf[];
  if (items) {
    out = items[blockIdx.y].out;
    perm += (int64_t)blockIdx.y * K;
    Wf += (int64_t)blockIdx.y * R * K;
  }
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;  // 256 threads, 1024 for rows above 8192 values
  constexpr int BATCH = 8;
  for (int c0 = 0; c0 < K; c0 += nt * BATCH) {
    float v[BATCH];
    int dst[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      const int cc = c < K ? c : K - 1;
      v[b] = Wf[(int64_t)r * K + cc];
      dst[b] = perm[cc];
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int c = c0 + b * nt + tid;
      if (c < K) rowbuf[dst[b]] = v[b];
    }
  }
  __syncthreads();
  for (int c = tid; c < K; c += nt) store_from_f32<WDT>(out, (int64_t)r * ldo + c, rowbuf[c]);
}

// dynamic LDS above 48 KB has to be asked for once per kernel
template <typename KernT>
inline int allow_row_stage(KernT kern, int K) {
  if ((size_t)K * 4 <= 48 * 1024) return 0;
  const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, K * 4);
  return e == hipSuccess ? 0 : 1000 + (int)e;
}


// The block's [GB][GB] slice of U into LDS, zero outside the upper triangle and past `count`.  Addresses are
// clamped into the block instead of predicated, so the loads of a batch are all in flight together.
__device__ __forceinline__ void load_u_block(float* __restrict__ Hs, const float* __restrict__ U, int64_t ldu,
                                             int i1, int count, int tid) {
  const float* base = U + (int64_t)i1 * ldu + i1;
  if (count == GB && (ldu & 3) == 0 && (i1 & 3) == 0 && ((uintptr_t)U & 15) == 0) {
    // full block, rows 16-byte aligned: one batch of 16 four-wide loads per thread
    constexpr int PER = GB * GB / 4 / 256;
    const int c4 = (tid % (GB / 4)) * 4, r0 = tid / (GB / 4);
    float4 v[PER];
#pragma unroll
    for (int b = 0; b < PER; ++b) v[b] = *(const float4*)&base[(int64_t)(b * (1024 / GB) + r0) * ldu + c4];
#pragma unroll
    for (int b = 0; b < PER; ++b) {
      const int i = b * (1024 / GB) + r0;
      float4 o;
      o.x = c4 + 0 >= i ? v[b].x : 0.f;
      o.y = c4 + 1 >= i ? v[b].y : 0.f;
      o.z = c4 + 2 >= i ? v[b].z : 0.f;
      o.w = c4 + 3 >= i ? v[b].w : 0.f;
      *(float4*)&Hs[i * GB + c4] = o;
    }
    return;
  }
  const int c = tid % GB;
  const int cc = c < count ? c : count - 1;
  constexpr int BATCH = 16;
  for (int it0 = 0; it0 < GB * GB / 256; it0 += BATCH) {
    float v[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int i = (it0 + b) * (256 / GB) + tid / GB;
      const int ic = i < count ? i : count - 1;
      v[b] = base[(int64_t)ic * ldu + cc];
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int i = (it0 + b) * (256 / GB) + tid / GB;
      Hs[(it0 + b) * 256 + tid] = (c >= i && c < count) ? v[b] : 0.f;
    }
  }
}

struct GptqBlockParams {
  float* Wf;        // [R,K] fp32 work copy (permuted columns)
  int R, K;
  const float* U;   // inverse-Hessian upper factor
  int64_t ldu;
  int i1, count;    // block = columns [i1, i1+count)
  const void* scale;
  int scale_dt;
  const int8_t* zp;
  const float* gscale;
  const int32_t* g_idx;  // group of each (permuted) column, or NULL
  int64_t row_div, srow;
  int fmt, bits;
  int sd;           // dtype the dequantised value is formed in
  float* E;         // scaled errors of this block, row stride ldE
  int ldE;
  float* loss_rows; // [R]
  // grouped call: problem blockIdx.y takes scale / zp / gscale / g_idx from items and its Wf, U, E and
  // loss rows at these strides (in elements)
  const GptqItem* items;
  int64_t u_stride;
};

// Layout of the quantiser's block kernel: a row is spread over a team of QTEAM lanes (one DPP quad), each
// holding QCPL columns of the block in registers as QNCH runs of QG neighbouring columns; run j of lane t
// covers columns j*QCW + t*QG .. +QG-1.  The lane that owns a run quantises its QG columns by itself (the
// serial chain of a row never crosses lanes inside a run), then the QG scaled errors are broadcast to the team
// once and every lane applies them, in column order, to the runs that are still open.
// Two team sizes are built.  Four lanes per row (one DPP quad, 32 columns per lane, 64 rows per workgroup) is the
// layout for many rows: few waves, each doing as little redundant work as possible.  Sixteen lanes per row (8
// columns per lane, 16 rows per workgroup) spreads a problem of a few thousand rows over every CU, one wave per
// SIMD, and each wave applies a run's errors to two runs per lane instead of eight: the per-block time is bound
// by one wave's instruction issue, so it falls with the instruction count.  Both apply the same operations to
// every element in the same order, so they give the same bits.
constexpr int QG = 4;              // neighbouring columns per run
template <int TEAM>
struct QLayout {
  static constexpr int QTEAM = TEAM;
  static constexpr int QCPL = GB / TEAM;   // columns per lane
  static constexpr int QNCH = QCPL / QG;   // runs per lane
  static constexpr int QCW = TEAM * QG;    // columns per round of the team
  static constexpr int ROWS_PER_WG = 256 / TEAM;
};
// rows (of all problems of a launch) up to which the sixteen-lane layout is used
constexpr int64_t Q_WIDE_TEAM_MAX_ROWS = 8192;

// ---- divisions of the column loop.  x / s goes through the hoisted reciprocal y of s (see make_fastdiv():
// the steps of the correctly rounded division with the divisor's part taken out).  The short form gives the
// IEEE quotient while |q| stays in [2^-40, 2^100) or both x and q are zero; `worst` collects, without a
// branch, how far outside that window any quotient of a run fell, and the caller redoes the run with plain
// divisions when it did.  A divisor outside make_fastdiv()'s range has a NaN reciprocal, which lands outside
// the window as well.
constexpr uint32_t QDIV_LO = 0x2b800000u;  // bits of 2^-40
constexpr uint32_t QDIV_SPAN = 0x71800000u - QDIV_LO;  // up to 2^100
__device__ __forceinline__ float shared_reciprocal(float s) {
  const FastDiv d = make_fastdiv(s);
  return d.ok ? d.y : __builtin_nanf("");
}
template <bool EXACT>
__device__ __forceinline__ float run_div(float x, float s, float y, uint32_t& worst) {
  if (EXACT) return x / s;
  float q = x * y;
  float r = fmaf(-s, q, x);
  q = fmaf(r, y, q);
  r = fmaf(-s, q, x);
  q = fmaf(r, y, q);
  const uint32_t qb = __float_as_uint(q) & 0x7fffffffu, xb = __float_as_uint(x) & 0x7fffffffu;
  const uint32_t t = (qb | xb) == 0u ? QDIV_LO : qb;
  worst = max(worst, t - QDIV_LO);
  return q;
}

template <int SD>
__device__ __forceinline__ float round_sd(float x) {
  if (SD == LLMC_BF16) return round16_finite<LLMC_BF16>(x);
  if (SD == LLMC_F16) return round16_finite<LLMC_F16>(x);
  return x;
}

struct QRun {
  float4 q, e;  // dequantised values and scaled errors of the run's QG columns
};

// One run of QG neighbouring columns of one row, start to finish inside a lane: column m is quantised, its
// scaled error err = (w - q) / d is applied to the columns of the run behind it (one fused multiply-subtract
// per element; the reference rounds the outer product before it subtracts, the fused form keeps the product
// exact), and so on.  u0..u2 are rows 0..2 of the run's QG x QG diagonal block of U.
template <int FMT, int SD, bool HAS_ZP, bool EXACT>
__device__ __forceinline__ QRun gptq_run(float4 w, float4 s, float4 y, float4 z, float4 d, float4 dy,
                                         float4 u0, float4 u1, float4 u2, const QFormat& f, uint32_t& worst) {
  QRun o;
  auto column = [&](float wv, float sc, float yc, float zp, float dc, float dyc, float& q, float& err) {
    // quantize_value() with the quotient formed by run_div()
    float v = run_div<EXACT>(wv, sc, yc, worst);
    v = HAS_ZP ? v + zp : v + 0.0f;
    const float qc = round_to_grid(v, f);
    float dq = qc;
    if (HAS_ZP) dq = round_sd<SD>(dq - zp);
    q = round_sd<SD>(dq * sc);
    err = run_div<EXACT>(__fsub_rn(wv, q), dc, dyc, worst);
  };
  column(w.x, s.x, y.x, z.x, d.x, dy.x, o.q.x, o.e.x);
  w.y = fmaf(-o.e.x, u0.y, w.y);
  w.z = fmaf(-o.e.x, u0.z, w.z);
  w.w = fmaf(-o.e.x, u0.w, w.w);
  column(w.y, s.y, y.y, z.y, d.y, dy.y, o.q.y, o.e.y);
  w.z = fmaf(-o.e.y, u1.z, w.z);
  w.w = fmaf(-o.e.y, u1.w, w.w);
  column(w.z, s.z, y.z, z.z, d.z, dy.z, o.q.z, o.e.z);
  w.w = fmaf(-o.e.z, u2.w, w.w);
  column(w.w, s.w, y.w, z.w, d.w, dy.w, o.q.w, o.e.w);
  return o;
}
static_assert(QG == 4, "gptq_run() is written out for runs of four columns");

// the rare way round: plain divisions, kept out of line
template <int FMT, int SD, bool HAS_ZP>
__device__ __noinline__ QRun gptq_run_exact(float4 w, float4 s, float4 z, float4 d, float4 u0, float4 u1,
                                            float4 u2, int bits) {
  const QFormat f = make_qformat(FMT, bits);
  uint32_t unused = 0;
  return gptq_run<FMT, SD, HAS_ZP, true>(w, s, s, z, d, d, u0, u1, u2, f, unused);
}

// the registers of one lane: QCPL columns of one row, their scales, the scales' reciprocals, zero points
template <bool HAS_ZP, int TEAM>
struct QLane {
  static constexpr int QNCH = QLayout<TEAM>::QNCH;
  float4 w[QNCH], sv[QNCH], yv[QNCH], zv[HAS_ZP ? QNCH : 1];
};

// Round J of the team: for each lane in turn, its run J is quantised and the errors applied to everything
// that is still open.  Columns at or past `count` hold w = 0, scale 1, d = 1 and zero rows of U: they
// quantise to zero with zero error, so only the stores look at `count`.
template <int J, int FMT, int SD, bool HAS_ZP, int TEAM>
__device__ __forceinline__ void gptq_round(QLane<HAS_ZP, TEAM>& r, const float* __restrict__ Hs,
                                           const float* __restrict__ Dd, const float* __restrict__ Dy, int tl,
                                           int count, bool live, float* __restrict__ wrow,
                                           float* __restrict__ erow, const QFormat& f, int bits, float& loss) {
  constexpr int QTEAM = TEAM, QNCH = QLayout<TEAM>::QNCH, QCW = QLayout<TEAM>::QCW;
#pragma unroll 1
  for (int li = 0; li < QTEAM; ++li) {
    const int i0 = J * QCW + li * QG;  // first column of this run
    if (i0 >= count) break;            // uniform across the workgroup
    const float* diag = Hs + i0 * GB + i0;
    const float4 d = *(const float4*)&Dd[i0], dy = *(const float4*)&Dy[i0];
    const float4 u0 = *(const float4*)&diag[0], u1 = *(const float4*)&diag[GB], u2 = *(const float4*)&diag[2 * GB];
    const float4 z = r.zv[HAS_ZP ? J : 0];
    const bool own = tl == li;
    // every lane runs the chain on its own run J; only the owner's is due, the others' results are dropped
    uint32_t worst = 0;
    QRun o = gptq_run<FMT, SD, HAS_ZP, false>(r.w[J], r.sv[J], r.yv[J], z, d, dy, u0, u1, u2, f, worst);
    if (own && worst >= QDIV_SPAN) o = gptq_run_exact<FMT, SD, HAS_ZP>(r.w[J], r.sv[J], z, d, u0, u1, u2, bits);
    if (own && live) {
      if (i0 + 0 < count) wrow[i0 + 0] = o.q.x;
      if (i0 + 1 < count) wrow[i0 + 1] = o.q.y;
      if (i0 + 2 < count) wrow[i0 + 2] = o.q.z;
      if (i0 + 3 < count) wrow[i0 + 3] = o.q.w;
      erow[i0 + 0] = o.e.x;
      erow[i0 + 1] = o.e.y;
      erow[i0 + 2] = o.e.z;
      erow[i0 + 3] = o.e.w;
    }
    const float eb[QG] = {__shfl(o.e.x, li, QTEAM), __shfl(o.e.y, li, QTEAM), __shfl(o.e.z, li, QTEAM),
                          __shfl(o.e.w, li, QTEAM)};
#pragma unroll
    for (int m = 0; m < QG; ++m) {
      loss += eb[m] * eb[m];  // (w-q)^2 / d^2
      // this round's run: lanes before the owner see zeros of U, the owner is already done
      const float eff = own ? 0.f : eb[m];
      const float* hrow = Hs + (i0 + m) * GB + tl * QG;
      const float4 h = *(const float4*)&hrow[J * QCW];
      r.w[J].x = fmaf(-eff, h.x, r.w[J].x);
      r.w[J].y = fmaf(-eff, h.y, r.w[J].y);
      r.w[J].z = fmaf(-eff, h.z, r.w[J].z);
      r.w[J].w = fmaf(-eff, h.w, r.w[J].w);
#pragma unroll
      for (int j2 = J + 1; j2 < QNCH; ++j2) {
        const float4 g = *(const float4*)&hrow[j2 * QCW];
        r.w[j2].x = fmaf(-eb[m], g.x, r.w[j2].x);
        r.w[j2].y = fmaf(-eb[m], g.y, r.w[j2].y);
        r.w[j2].z = fmaf(-eb[m], g.z, r.w[j2].z);
        r.w[j2].w = fmaf(-eb[m], g.w, r.w[j2].w);
      }
    }
  }
}

// the block's weights, scales and zero points of one lane; SDT = dtype of the stored scales
template <int SDT, bool HAS_ZP, int TEAM>
__device__ __forceinline__ void gptq_load_lane(QLane<HAS_ZP, TEAM>& r, const GptqBlockParams& p, int row, int tl,
                                               bool live) {
  constexpr int QCPL = QLayout<TEAM>::QCPL, QNCH = QLayout<TEAM>::QNCH, QCW = QLayout<TEAM>::QCW;
  const int rowc = live ? row : p.R - 1;  // every load stays inside the arrays; dead lanes are blanked below
  const float* wsrc = p.Wf + (int64_t)rowc * p.K + p.i1;
  const int64_t sbase = ((int64_t)rowc / p.row_div) * p.srow;
  const float gs = p.gscale ? p.gscale[0] : 1.f;
  float w[QCPL], s[QCPL], zp[QCPL];
  int gi[QCPL];
  // three sweeps, each with all its loads in flight: group numbers, then what they index
#pragma unroll
  for (int e = 0; e < QCPL; ++e) gi[e] = 0;
  if (p.g_idx) {
#pragma unroll
    for (int e = 0; e < QCPL; ++e) {
      const int cb = (e / QG) * QCW + tl * QG + (e % QG);
      gi[e] = p.g_idx[p.i1 + (cb < p.count ? cb : p.count - 1)];
    }
  }
#pragma unroll
  for (int e = 0; e < QCPL; ++e) {
    const int cb = (e / QG) * QCW + tl * QG + (e % QG);
    w[e] = wsrc[cb < p.count ? cb : p.count - 1];
    s[e] = load_as_f32<SDT>(p.scale, sbase + gi[e]);
    zp[e] = HAS_ZP ? (float)p.zp[sbase + gi[e]] : 0.f;
  }
#pragma unroll
  for (int e = 0; e < QCPL; ++e) {
    const int cb = (e / QG) * QCW + tl * QG + (e % QG);
    if (p.gscale) s[e] = s[e] / gs;
    if (!live || cb >= p.count) {
      w[e] = 0.f;
      s[e] = 1.f;
      zp[e] = 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < QNCH; ++j) {
    r.w[j] = make_float4(w[j * QG], w[j * QG + 1], w[j * QG + 2], w[j * QG + 3]);
    r.sv[j] = make_float4(s[j * QG], s[j * QG + 1], s[j * QG + 2], s[j * QG + 3]);
    r.yv[j] = make_float4(shared_reciprocal(s[j * QG]), shared_reciprocal(s[j * QG + 1]),
                          shared_reciprocal(s[j * QG + 2]), shared_reciprocal(s[j * QG + 3]));
    if (HAS_ZP) r.zv[j] = make_float4(zp[j * QG], zp[j * QG + 1], zp[j * QG + 2], zp[j * QG + 3]);
  }
  if (!HAS_ZP) r.zv[0] = make_float4(0.f, 0.f, 0.f, 0.f);
}

template <int FMT, int SD, bool HAS_ZP, int TEAM>
__global__ __launch_bounds__(256) void gptq_block_kernel(GptqBlockParams p) {
  constexpr int QTEAM = TEAM, QNCH = QLayout<TEAM>::QNCH, QCW = QLayout<TEAM>::QCW;
  constexpr int Q_ROWS_PER_WG = QLayout<TEAM>::ROWS_PER_WG;
  // [GB][GB] slice of U, zero outside the upper triangle; then its diagonal and the diagonal's reciprocals
  extern __shared__ __attribute__((aligned(16))) float Hs[];
  float* Dd = Hs + GB * GB;
  float* Dy = Dd + GB;
  if (p.items) {
    const GptqItem it = p.items[blockIdx.y];
    p.scale = it.scale; p.zp = it.zp; p.gscale = it.gscale; p.g_idx = it.g_idx;
    p.Wf += (int64_t)blockIdx.y * p.R * p.K;
    p.U += (int64_t)blockIdx.y * p.u_stride;
    p.E += (int64_t)blockIdx.y * p.R * p.ldE;
    p.loss_rows += (int64_t)blockIdx.y * p.R;
  }
  const int tid = threadIdx.x;
  const int count = p.count;
  load_u_block(Hs, p.U, p.ldu, p.i1, count, tid);
  if (tid < GB) {
    const float d = tid < count ? p.U[(int64_t)(p.i1 + tid) * p.ldu + p.i1 + tid] : 1.f;
    Dd[tid] = d;
    Dy[tid] = shared_reciprocal(d);
  }
  const int tl = tid % QTEAM;
  const int row = blockIdx.x * Q_ROWS_PER_WG + tid / QTEAM;
  const bool live = row < p.R;
  const QFormat f = make_qformat(FMT, p.bits);  // the format is a compile-time constant here
  float* wrow = p.Wf + (int64_t)row * p.K + p.i1;
  float* erow = p.E + (int64_t)row * p.ldE;

  QLane<HAS_ZP, TEAM> r;
  if (p.scale_dt == LLMC_BF16)
    gptq_load_lane<LLMC_BF16, HAS_ZP, TEAM>(r, p, row, tl, live);
  else if (p.scale_dt == LLMC_F16)
    gptq_load_lane<LLMC_F16, HAS_ZP, TEAM>(r, p, row, tl, live);
  else
    gptq_load_lane<LLMC_F32, HAS_ZP, TEAM>(r, p, row, tl, live);
  __syncthreads();

  float loss = 0.f;
#define LLMC_ROUND(J)                                                                                          \
  if constexpr (J < QNCH) {                                                                                    \
    if (J * QCW < count)                                                                                       \
      gptq_round<J, FMT, SD, HAS_ZP, TEAM>(r, Hs, Dd, Dy, tl, count, live, wrow, erow, f, p.bits, loss);       \
  }
  LLMC_ROUND(0) LLMC_ROUND(1) LLMC_ROUND(2) LLMC_ROUND(3)
  LLMC_ROUND(4) LLMC_ROUND(5) LLMC_ROUND(6) LLMC_ROUND(7)
#undef LLMC_ROUND
  static_assert(QNCH <= 8, "one LLMC_ROUND per run of a lane");

  if (live) {
    // the runs that were never reached carry no error into the trailing products
#pragma unroll
    for (int j = 0; j < QNCH; ++j) {
      if (j * QCW >= count) {
#pragma unroll
        for (int m = 0; m < QG; ++m) erow[j * QCW + tl * QG + m] = 0.f;
      }
    }
    if (tl == 0) p.loss_rows[row] += loss * 0.5f;
  }
}

// The product inside a group of column blocks, W[:, c0:c1] -= E_b * U[i1:i1+128, c0:c1] with at most 384 columns:
// 15 MB of traffic for a 4096-row weight, a few microseconds of matrix-core time -- a general tiled product
// spends most of its 19 us ramping its pipeline up and down.  Here a workgroup owns 16 rows and all columns: each
// wave takes every fourth 16-column tile, holds the 16 x 128 slice of E (negated) in registers for all its tiles,
// fetches a tile's 128 x 16 slice of U straight from global memory (every workgroup reads the same 128 x 384
// block, which stays in the L2) one tile ahead, and runs 32 v_mfma_f32_16x16x4_f32 per tile with the tile of W
// as the accumulator's start value.  Lane group q = lane / 16 contributes the inner indices 32 q .. 32 q + 31, one
// per instruction, so a lane's E values are eight consecutive float4.  Sums are fp32 fused multiply-adds of
// exact products, as in the fp32 matrix kernel.
struct GroupUpdate {
  const float* E;   // [R, ldE]: the block's scaled errors (128 columns)
  int64_t ldE;
  const float* U;   // first row of the block's 128 rows of the factor, at column c0
  int64_t ldu;
  float* W;         // [R, K] work copy, at column c0
  int64_t ldw;
  int R, ntiles;    // ntiles = (c1 - c0) / 16
  int64_t stride_e, stride_u, stride_w;  // per problem (blockIdx.y)
};

__global__ __launch_bounds__(256) void gptq_group_update_kernel(GroupUpdate g) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, q = lane >> 4;
  const float* E = g.E + (int64_t)blockIdx.y * g.stride_e;
  const float* U = g.U + (int64_t)blockIdx.y * g.stride_u;
  float* W = g.W + (int64_t)blockIdx.y * g.stride_w;
  const int row0 = blockIdx.x * 16;
  const int ra = row0 + c < g.R ? row0 + c : g.R - 1;  // A operand: row c of the 16, inner indices 32 q + j
  float a[32];
  {
    const float4* src = (const float4*)(E + (int64_t)ra * g.ldE + 32 * q);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float4 v = src[j];
      a[4 * j] = -v.x; a[4 * j + 1] = -v.y; a[4 * j + 2] = -v.z; a[4 * j + 3] = -v.w;
    }
  }
  auto fetch_b = [&](float* b, int tile) {  // B operand: column c of the tile, inner indices 32 q + j
    const float* src = U + (int64_t)(32 * q) * g.ldu + tile * 16 + c;
#pragma unroll
    for (int j = 0; j < 32; ++j) b[j] = src[(int64_t)j * g.ldu];
  };
  float b0[32], b1[32];
  int tile = wave;
  if (tile < g.ntiles) fetch_b(b0, tile);
  // accumulator element i of a lane: row 4 q + i, column c
  auto run = [&](const float* b, int t) {
    float* dst = W + (int64_t)(row0 + 4 * q) * g.ldw + t * 16 + c;
    f32x4_t acc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = row0 + 4 * q + i < g.R ? dst[(int64_t)i * g.ldw] : 0.f;
#pragma unroll
    for (int j = 0; j < 32; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], acc, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (row0 + 4 * q + i < g.R) dst[(int64_t)i * g.ldw] = acc[i];
  };
  while (tile < g.ntiles) {
    if (tile + 4 < g.ntiles) fetch_b(b1, tile + 4);
    run(b0, tile);
    tile += 4;
    if (tile >= g.ntiles) break;
    if (tile + 4 < g.ntiles) fetch_b(b0, tile + 4);
    run(b1, tile);
    tile += 4;
  }
}


template <int WDT>
__global__ __launch_bounds__(256) void gptq_finalize_kernel(const float* __restrict__ Wf, int R, int K,
                                                            const int32_t* __restrict__ perm,
                                                            void* __restrict__ out, int64_t ldo,
                                                            const GptqItem* __restrict__ items = nullptr) {
  if (items) {
    out = items[blockIdx.z].out;
    if (perm) perm += (int64_t)blockIdx.z * K;
    Wf += (int64_t)blockIdx.z * R * K;
  }
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (c >= K) return;
  const int dst = perm ? perm[c] : c;
  store_from_f32<WDT>(out, (int64_t)r * ldo + dst, Wf[(int64_t)r * K + c]);
}

__global__ __launch_bounds__(256) void sum_rows_kernel(const float* __restrict__ v, int n, float* out) {
  __shared__ float red[4];
  v += (int64_t)blockIdx.x * n;  // grouped call: one workgroup per problem
  out += blockIdx.x;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) s += v[i];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) out[0] = red[0] + red[1] + red[2] + red[3];
}

__global__ __launch_bounds__(256) void zero_f32_kernel(float* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

inline int64_t align256(int64_t b) { return (b + 255) / 256 * 256; }

// ---------------------------------------------------------------------------------------------
// SparseGPT: the same blocked column loop with a pruning mask in place of the quantiser.
//
// Unstructured pruning takes, per block of columns, the elements whose saliency w^2 / d^2
// (d = diagonal of the inverse-Hessian factor) is not above the k-th smallest of the whole
// [R x count] block, k = int(numel * sparsity).  That order statistic is found exactly by a
// three-pass radix selection on the float bit patterns (11 + 11 + 10 bits; saliencies are
// non-negative, so their bit patterns order like the values): every pass builds a histogram
// of the next digit over the elements that match the digits found so far.  The histograms of
// a block live in their own slice of the workspace, so nothing is cleared between blocks.
// N:M pruning (M in {2, 4, 8}: a group lies inside one lane's 8 columns) picks, when the loop
// reaches a group, the N least salient of its current values.
constexpr int SG_BINS = 2048;
constexpr int SG_HIST_WORDS = 3 * SG_BINS + 64;  // three histograms + the masked-element count
constexpr int SG_MIN_BLOCK = 32;                 // narrowest unstructured block (sizes the histogram slices)

struct SgptParams {
  float* Wf;
  int R, K;
  const float* U;
  int64_t ldu;
  int i1, count;
  const uint8_t* mask;   // [R,K] bytes, 1 = was zero before pruning (preserve mode), or NULL
  unsigned* hist;        // this block's SG_HIST_WORDS words
  unsigned k;            // rank of the threshold element (0-based) in the ascending order
  int prune_n, prune_m;  // 0:0 = unstructured
  float* E;
  int ldE;
  float* loss_rows;
};

__device__ __forceinline__ float sgpt_saliency(float w, float d, bool masked) {
  const float num = masked ? 0.f : __fmul_rn(w, w);
  return __fdiv_rn(num, __fmul_rn(d, d));
}

// First bin whose running total exceeds k (the last bin when none does); k becomes the rank inside that bin.
// All 256 threads of the workgroup take part; `scratch` holds 258 words.  Thread t sums its nbins / 256
// consecutive bins, a scan over the 256 sums (shuffles inside a wave, the four wave totals through LDS) finds
// the one thread whose bins contain rank k, and that thread walks its few bins.
__device__ __forceinline__ unsigned sgpt_find_bin(const unsigned* __restrict__ hist, int nbins, unsigned& k,
                                                  unsigned* scratch) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = nbins / 256;
  unsigned local = 0;
  for (int b = 0; b < per; ++b) local += hist[tid * per + b];
  unsigned incl = local;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  for (int w = 0; w < wave; ++w) incl += scratch[w];
  const unsigned excl = incl - local;
  if (excl <= k && (k < incl || tid == 255)) {
    unsigned run = excl, bin = (unsigned)(tid * per);
    for (int b = 0; b < per - 1; ++b) {
      const unsigned h = hist[tid * per + b];
      if (run + h > k) break;
      run += h;
      ++bin;
    }
    scratch[256] = bin;
    scratch[257] = k - run;
  }
  __syncthreads();
  const unsigned bin = scratch[256];
  k = scratch[257];
  __syncthreads();
  return bin;
}

template <int PASS>
__global__ __launch_bounds__(256) void sgpt_hist_kernel(SgptParams p) {
  __shared__ unsigned lh[SG_BINS];
  __shared__ unsigned scratch[258];
  __shared__ unsigned nmasked;
  const int tid = threadIdx.x;
  for (int b = tid; b < SG_BINS; b += 256) lh[b] = 0;
  if (tid == 0) nmasked = 0;
  unsigned k = p.k, prefix = 0;
  if (PASS >= 1) prefix = sgpt_find_bin(p.hist, SG_BINS, k, scratch);
  if (PASS >= 2) prefix = (prefix << 11) | sgpt_find_bin(p.hist + SG_BINS, SG_BINS, k, scratch);
  __syncthreads();
  const int64_t n = (int64_t)p.R * p.count;
  for (int64_t e = (int64_t)blockIdx.x * 256 + tid; e < n; e += (int64_t)gridDim.x * 256) {
    // a full block is 128 wide: shift and mask instead of a 64-bit division per element
    const int r = p.count == GB ? (int)(e >> 7) : (int)(e / p.count);
    const int c = p.count == GB ? (int)(e & (GB - 1)) : (int)(e % p.count);
    const int col = p.i1 + c;
    const bool masked = p.mask && p.mask[(int64_t)r * p.K + col];
    const float t = sgpt_saliency(p.Wf[(int64_t)r * p.K + col], p.U[(int64_t)col * p.ldu + col], masked);
    const unsigned bits = __float_as_uint(t);
    if (PASS == 0) {
      atomicAdd(&lh[bits >> 21], 1u);
      if (masked) atomicAdd(&nmasked, 1u);
    } else if (PASS == 1) {
      if ((bits >> 21) == prefix) atomicAdd(&lh[(bits >> 10) & 2047u], 1u);
    } else {
      if ((bits >> 10) == prefix) atomicAdd(&lh[bits & 1023u], 1u);
    }
  }
  __syncthreads();
  unsigned* gh = p.hist + PASS * SG_BINS;
  for (int b = tid; b < SG_BINS; b += 256)
    if (lh[b]) atomicAdd(&gh[b], lh[b]);
  if (PASS == 0 && tid == 0 && nmasked) atomicAdd(&p.hist[3 * SG_BINS], nmasked);
}

template <bool NM>
__global__ __launch_bounds__(256) void sgpt_block_kernel(SgptParams p) {
  extern __shared__ __attribute__((aligned(16))) float Hs[];  // [GB][GB], zero outside the upper triangle
  __shared__ unsigned scratch[258];
  const int tid = threadIdx.x;
  load_u_block(Hs, p.U, p.ldu, p.i1, p.count, tid);
  // unstructured: the block's threshold from its three histograms
  float thresh = 0.f;
  bool use_thresh = false;
  if (!NM) {
    unsigned k = p.k;
    unsigned bits = sgpt_find_bin(p.hist, SG_BINS, k, scratch);
    bits = (bits << 11) | sgpt_find_bin(p.hist + SG_BINS, SG_BINS, k, scratch);
    bits = (bits << 10) | sgpt_find_bin(p.hist + 2 * SG_BINS, 1024, k, scratch);
    thresh = __uint_as_float(bits);
    // with a mask to preserve, the mask is only extended when the target asks for more zeros than it holds
    use_thresh = p.mask == nullptr || p.k > p.hist[3 * SG_BINS];
  }
  __syncthreads();
  const int tl = tid % TEAM;
  const int row = blockIdx.x * ROWS_PER_WG + tid / TEAM;
  const bool live = row < p.R;

  float w[CPL], qv[CPL], ev[CPL];
  unsigned pruned = 0, masked = 0;  // bit e: column tl*CPL + e of the block
#pragma unroll
  for (int e = 0; e < CPL; ++e) {
    const int cb = tl * CPL + e;
    w[e] = 0.f;
    qv[e] = 0.f;
    ev[e] = 0.f;
    if (live && cb < p.count) {
      const int c = p.i1 + cb;
      w[e] = p.Wf[(int64_t)row * p.K + c];
      if (p.mask && p.mask[(int64_t)row * p.K + c]) masked |= 1u << e;
    }
  }
  __syncthreads();  // Hs complete
  if (!NM) {
    if (use_thresh) {
#pragma unroll
      for (int e = 0; e < CPL; ++e) {
        const int cb = tl * CPL + e;
        if (cb < p.count && sgpt_saliency(w[e], Hs[cb * GB + cb], (masked >> e) & 1u) <= thresh) pruned |= 1u << e;
      }
    } else {
      pruned = masked;
    }
  } else {
    pruned = masked;
  }

  float loss = 0.f;
  for (int li = 0; li < TEAM; ++li) {
    if (li * CPL >= p.count) break;
#pragma unroll
    for (int e = 0; e < CPL; ++e) {
      const int i = li * CPL + e;
      if (i < p.count) {  // uniform across the workgroup
        if (NM && (e % p.prune_m) == 0 && tl == li) {
          // the N least salient of the group's current values (ties: the lower column first)
          float t[CPL];
#pragma unroll
          for (int j = 0; j < CPL; ++j) {
            const int cb = tl * CPL + j;
            t[j] = sgpt_saliency(w[j], Hs[(cb < GB ? cb : 0) * GB + (cb < GB ? cb : 0)], (masked >> j) & 1u);
          }
#pragma unroll
          for (int j = 0; j < CPL; ++j) {
            if (j >= e && j < e + p.prune_m && tl * CPL + j < p.count) {
              int rank = 0;
#pragma unroll
              for (int l = 0; l < CPL; ++l)
                if (l >= e && l < e + p.prune_m && tl * CPL + l < p.count && (t[l] < t[j] || (t[l] == t[j] && l < j)))
                  ++rank;
              if (rank < p.prune_n) pruned |= 1u << j;
            }
          }
        }
        const float wv = __shfl(w[e], li, TEAM);
        const unsigned flags = __shfl((int)pruned, li, TEAM);
        const float q = ((flags >> e) & 1u) ? 0.f : wv;
        const float d = Hs[i * GB + i];
        const float diff = __fsub_rn(wv, q);
        const float err = diff / d;
        loss += err * err;  // (w-q)^2 / d^2
        const float4 h0 = *(const float4*)&Hs[i * GB + tl * CPL];
        const float4 h1 = *(const float4*)&Hs[i * GB + tl * CPL + 4];
        // one fused multiply-subtract per element, as in the quantiser's kernel
        w[0] = fmaf(-err, h0.x, w[0]);
        w[1] = fmaf(-err, h0.y, w[1]);
        w[2] = fmaf(-err, h0.z, w[2]);
        w[3] = fmaf(-err, h0.w, w[3]);
        w[4] = fmaf(-err, h1.x, w[4]);
        w[5] = fmaf(-err, h1.y, w[5]);
        w[6] = fmaf(-err, h1.z, w[6]);
        w[7] = fmaf(-err, h1.w, w[7]);
        if (tl == li) {
          qv[e] = q;
          ev[e] = err;
        }
      }
    }
  }

  if (live) {
#pragma unroll
    for (int e = 0; e < CPL; ++e) {
      const int cb = tl * CPL + e;
      if (cb < p.count) p.Wf[(int64_t)row * p.K + p.i1 + cb] = qv[e];
      p.E[(int64_t)row * p.ldE + cb] = ev[e];
    }
    if (tl == 0) p.loss_rows[row] += loss * 0.5f;
  }
}

// mask[r,c] = (Wf[r,c] == 0): the sparsity pattern to preserve
__global__ __launch_bounds__(256) void sgpt_mask_kernel(const float* __restrict__ Wf, int64_t n, uint8_t* mask) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) mask[i] = Wf[i] == 0.f ? 1 : 0;
}

// the trailing updates leave preserved zeros alone: put them back after an unmasked product.  In the left-looking
// form the update that is thrown away here has to stay visible to the later groups (their share of the earlier
// errors is computed from W0 - Q, which equals Err U only while every update is kept): it is taken out of the
// group's copy of W0 in Df, so that W0 - Q becomes what Err U is.
__global__ __launch_bounds__(256) void sgpt_rezero_kernel(float* __restrict__ Wf, const uint8_t* __restrict__ mask,
                                                          int K, int c0, int c1, float* __restrict__ Df) {
  const int c = c0 + blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  const int64_t at = (int64_t)r * K + c;
  if (c < c1 && mask[at]) {
    if (Df) Df[at] -= Wf[at];
    Wf[at] = 0.f;
  }
}

__global__ __launch_bounds__(256) void zero_u32_words_kernel(unsigned* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

}  // namespace

// enqueue gptq_group_update_kernel when the shapes fit it (a full 128-column block, a multiple of 16 columns to
// update); returns -1 when the product is left to the general kernels
static int launch_group_update(const float* Eb, int64_t ldE, const float* U, int64_t ldu, int64_t u_stride, float* Wf,
                               int64_t R, int64_t K, int n, int64_t i1, int count, int64_t c0, int64_t c1,
                               hipStream_t st) {
  if (count != GB || (c1 - c0) % 16 != 0 || (ldE & 3) != 0 || K >= (1 << 30)) return -1;
  GroupUpdate gu;
  gu.E = Eb; gu.ldE = ldE; gu.U = U + i1 * ldu + c0; gu.ldu = ldu; gu.W = Wf + c0; gu.ldw = K;
  gu.R = (int)R; gu.ntiles = (int)((c1 - c0) / 16);
  gu.stride_e = R * ldE; gu.stride_u = u_stride; gu.stride_w = R * K;
  hipLaunchKernelGGL(gptq_group_update_kernel, dim3((unsigned)((R + 15) / 16), (unsigned)n), dim3(256), 0, st, gu);
  LLMC_LAUNCH_STATUS();
  return 0;
}

// ---- left-looking form of the far updates (LLMC_FACTOR_GROUPS) ------------------------------------------------
// With E = Err and D = W0 - Q (weights before the loop minus quantised weights) the loop's invariants are
// D = E U and E = D V (V = U^-1 upper triangular, V V^T = H), so what the columns of a group G owe to all
// earlier columns, -E[:, :g0] U[:g0, G], equals (D[:, :g0] V[:g0, G]) U[G, G]: the factor of H itself outside
// the diagonal blocks and the inverse only inside them.  Per group: one product with a contraction over all
// earlier columns, cut into pieces so that it fills the chip; a pass that adds the pieces in a fixed order,
// keeps W0's columns and negates the sum; one 512-wide product with the group's diagonal block; the group's
// blocks as in the other form; a pass that turns the kept W0 into D.
// The groups are the chain's diagonal blocks, which are aligned to the END of the column range (the chain works
// in reversed index order): 512 columns each, except that the first one holds the K % 512 columns that are left
// over when K is not a multiple of 512.
constexpr int LEFT_MAX_SPLITS = 16;
constexpr int64_t LEFT_GW = LLMC_FACTOR_GROUP_WIDTH;

// end of the group that starts at column g0
inline int64_t left_group_end(int64_t g0, int64_t K) {
  const int64_t first = K % LEFT_GW ? K % LEFT_GW : LEFT_GW;
  const int64_t e = g0 == 0 ? first : g0 + LEFT_GW;
  return e < K ? e : K;
}

// pieces of the contraction for a weight of R rows: enough 256 x 256 (128 x 128 below 256 rows' multiple) tiles
// for one per CU.  Depends on R only, never on how many problems share a launch.
inline int left_split_cap(int64_t R) {
  const int64_t tiles = (R % 256 == 0) ? (R / 256) * (LEFT_GW / 256) : ((R + 127) / 128) * (LEFT_GW / 128);
  int64_t s = (256 + tiles - 1) / tiles;
  return (int)(s < 1 ? 1 : (s > LEFT_MAX_SPLITS ? LEFT_MAX_SPLITS : s));
}

// workspace behind the other buffers, for the left-looking form only: D (W0, then W0 - Q), the pieces of the
// product (never more of them than there are earlier groups), the negated sum
inline int64_t left_pieces_max(int64_t R, int64_t K) {
  const int64_t earlier = (K + LEFT_GW - 1) / LEFT_GW - 1;
  const int64_t cap = left_split_cap(R);
  return earlier < 1 ? 1 : (earlier < cap ? earlier : cap);
}
inline int64_t left_extra_bytes(int64_t n, int64_t R, int64_t K, int form) {
  if (form != LLMC_FACTOR_GROUPS) return 0;
  return align256(n * R * K * 4) + align256(n * left_pieces_max(R, K) * R * LEFT_GW * 4) + align256(n * R * LEFT_GW * 4);
}
inline bool left_form_fits(int64_t K, int blocksize) { return K % GB == 0 && blocksize >= GB; }

// D[:, G] = W[:, G] (the untouched columns of the group, gw of them) and, when there are pieces (gw = 512 then),
// C = -(P_0 + P_1 + ...)
__global__ __launch_bounds__(256) void left_begin_group_kernel(const float* __restrict__ Wf, float* __restrict__ Df,
                                                               int64_t K, int64_t g0, int gw, int64_t R,
                                                               const float* __restrict__ P, int pieces,
                                                               int64_t piece_stride, int64_t problem_stride_p,
                                                               float* __restrict__ Cn) {
  const int64_t b = blockIdx.y;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;  // element of the [R, gw] group slice
  if (idx >= R * gw) return;
  const int64_t row = idx / gw, col = idx % gw;
  const int64_t w = b * R * K + row * K + g0 + col;
  *(float4*)(Df + w) = *(const float4*)(Wf + w);
  if (pieces > 0) {
    const float* p = P + b * problem_stride_p + idx;
    float4 a = *(const float4*)p;
    for (int s = 1; s < pieces; ++s) {
      const float4 v = *(const float4*)(p + s * piece_stride);
      a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
    }
    *(float4*)(Cn + b * R * gw + idx) = make_float4(-a.x, -a.y, -a.z, -a.w);
  }
}

// D[:, G] -= W[:, G] (W holds the quantised values of the group now)
__global__ __launch_bounds__(256) void left_end_group_kernel(const float* __restrict__ Wf, float* __restrict__ Df,
                                                             int64_t K, int64_t g0, int gw, int64_t R) {
  const int64_t b = blockIdx.y;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= R * gw) return;
  const int64_t w = b * R * K + (idx / gw) * K + g0 + idx % gw;
  float4 d = *(const float4*)(Df + w);
  const float4 q = *(const float4*)(Wf + w);
  d.x -= q.x; d.y -= q.y; d.z -= q.z; d.w -= q.w;
  *(float4*)(Df + w) = d;
}

// what the group that starts at g0 owes to the columns before it, added to Wf[:, G]; `extra` is the memory behind
// the other work buffers (left_extra_bytes)
static int left_begin_group(int n, int64_t R, int64_t K, int64_t g0, const float* U, int64_t ldu, int64_t u_stride,
                            float* Wf, char* extra, hipStream_t st) {
  constexpr int64_t GW = LEFT_GW;
  const int gw = (int)(left_group_end(g0, K) - g0);  // 512 for every group but possibly the first
  float* Df = (float*)extra;
  float* P = (float*)(extra + align256(n * R * K * 4));
  const int cap = left_split_cap(R);
  const int64_t slots = left_pieces_max(R, K);  // pieces the workspace holds per problem (pieces <= slots below)
  float* Cn = (float*)((char*)P + align256(n * slots * R * GW * 4));
  const int64_t piece_stride = R * GW, problem_stride_p = slots * piece_stride;
  int pieces = 0;
  if (g0 > 0) {
    const int64_t m = (g0 + GW - 1) / GW;           // earlier groups (the first one may be short)
    const int64_t per = (m + cap - 1) / cap;        // groups' worth of columns per piece
    const int64_t chunk = per * GW;
    pieces = (int)((g0 + chunk - 1) / chunk);
    const int64_t last = g0 - (pieces - 1) * chunk;
    GemmF32 g = {};
    g.A = Df; g.lda = K; g.B = U + g0; g.ldb = ldu; g.C = P; g.ldc = GW;
    g.M = (int)R; g.N = (int)GW; g.Kc = (int)(pieces == 1 ? last : chunk); g.alpha = 1.f; g.beta = 0.f;
    g.batch = pieces; g.stride_a = chunk; g.stride_b = chunk * ldu; g.stride_c = piece_stride;
    g.kc_last = (pieces == 1 || last == chunk) ? 0 : (int)last;
    g.batch2 = n; g.stride2_a = R * K; g.stride2_b = u_stride; g.stride2_c = problem_stride_p;
    const int rc = llmc_gemm_f32(g, st);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(left_begin_group_kernel, dim3((unsigned)((R * gw / 4 + 255) / 256), (unsigned)n), dim3(256), 0, st,
                     (const float*)Wf, Df, K, g0, gw, R, (const float*)P, pieces, piece_stride, problem_stride_p, Cn);
  LLMC_LAUNCH_STATUS();
  if (g0 > 0) {
    GemmF32 h = {};  // Wf[:, G] -= Cn U[G, G]; U holds exact zeros below the diagonal
    h.A = Cn; h.lda = GW; h.B = U + g0 * ldu + g0; h.ldb = ldu; h.C = Wf + g0; h.ldc = K;
    h.M = (int)R; h.N = (int)GW; h.Kc = (int)GW; h.alpha = -1.f; h.beta = 1.f;
    h.batch = 1; h.batch2 = n; h.stride2_a = R * GW; h.stride2_b = u_stride; h.stride2_c = R * K;
    const int rc = llmc_gemm_f32(h, st);
    if (rc) return rc;
  }
  return 0;
}

static int left_end_group(int n, int64_t R, int64_t K, int64_t g0, const float* Wf, char* extra, hipStream_t st) {
  const int gw = (int)(left_group_end(g0, K) - g0);
  hipLaunchKernelGGL(left_end_group_kernel, dim3((unsigned)((R * gw / 4 + 255) / 256), (unsigned)n), dim3(256), 0, st, Wf,
                     (float*)extra, K, g0, gw, R);
  LLMC_LAUNCH_STATUS();
  return 0;
}

extern "C" int64_t llmc_sparsegpt_workspace_bytes(int64_t R, int64_t K, int32_t form) {
  const int64_t slices = (K + SG_MIN_BLOCK - 1) / SG_MIN_BLOCK;
  return align256(R * K * 4) + align256(R * GROUP * GB * 4) + align256(R * 4) +
         align256(slices * SG_HIST_WORDS * 4) + align256(R * K) + left_extra_bytes(1, R, K, form);
}

extern "C" int llmc_sparsegpt_sparsify(const void* weight, int32_t w_dtype, int64_t R, int64_t K, int64_t ldw,
                                       const float* U, int64_t ldu, const uint8_t* dead, double sparsity,
                                       int32_t prune_n, int32_t prune_m, int32_t blocksize, int32_t form,
                                       int32_t preserve_sparsity_mask, void* out_weight, int64_t ldo,
                                       float* loss_out, void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(weight != nullptr, 1);
  LLMC_CHECK_ARG(form == LLMC_FACTOR_INVERSE ||
                     (form == LLMC_FACTOR_GROUPS && left_form_fits(K, blocksize) && blocksize == GB), 13);
  LLMC_CHECK_ARG(w_dtype >= 0 && w_dtype <= 2, 2);
  LLMC_CHECK_ARG(R > 0 && R < (1ll << 24), 3);
  LLMC_CHECK_ARG(K > 0 && K < (1ll << 31), 4);
  LLMC_CHECK_ARG(ldw >= K, 5);
  LLMC_CHECK_ARG(U != nullptr && ldu >= K, 6);
  const bool nm = prune_n != 0;
  LLMC_CHECK_ARG(nm || (sparsity >= 0.0 && sparsity < 1.0), 9);
  LLMC_CHECK_ARG(!nm || ((prune_m == 2 || prune_m == 4 || prune_m == 8) && prune_n > 0 && prune_n <= prune_m), 11);
  // the block width decides which elements compete for the unstructured threshold, so it is not
  // clamped the way the quantiser's is
  LLMC_CHECK_ARG(blocksize > 0 && blocksize <= GB && (nm ? blocksize % prune_m == 0 : blocksize >= SG_MIN_BLOCK), 12);
  LLMC_CHECK_ARG(out_weight != nullptr && ldo >= K, 14);
  LLMC_CHECK_ARG(workspace != nullptr && (((uintptr_t)workspace) & 255) == 0, 17);
  LLMC_CHECK_ARG(workspace_bytes >= llmc_sparsegpt_workspace_bytes(R, K, form), 18);
  hipStream_t st = (hipStream_t)stream;
  const int bs = blocksize;
  const int64_t nblocks = (K + bs - 1) / bs;

  char* wp = (char*)workspace;
  float* Wf = (float*)wp; wp += align256(R * K * 4);
  float* E = (float*)wp; wp += align256(R * GROUP * GB * 4);
  float* loss_rows = (float*)wp; wp += align256(R * 4);
  unsigned* hist = (unsigned*)wp; wp += align256(((K + SG_MIN_BLOCK - 1) / SG_MIN_BLOCK) * SG_HIST_WORDS * 4);
  uint8_t* mask = preserve_sparsity_mask ? (uint8_t*)wp : nullptr;
  wp += align256(R * K);
  char* extra = wp;
  const bool left = form == LLMC_FACTOR_GROUPS;

  dim3 grid2((unsigned)((K + 255) / 256), (unsigned)R);
#define LLMC_PREP(DT) \
  hipLaunchKernelGGL((gptq_prepare_w_kernel<DT>), grid2, dim3(256), 0, st, weight, ldw, (int)R, (int)K, \
                     (const int32_t*)nullptr, dead, Wf)
  if (w_dtype == LLMC_BF16) LLMC_PREP(LLMC_BF16);
  else if (w_dtype == LLMC_F16) LLMC_PREP(LLMC_F16);
  else LLMC_PREP(LLMC_F32);
#undef LLMC_PREP
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0, st, loss_rows, R);
  LLMC_LAUNCH_STATUS();
  if (!nm) {
    const int64_t words = nblocks * SG_HIST_WORDS;
    hipLaunchKernelGGL(zero_u32_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, hist, words);
    LLMC_LAUNCH_STATUS();
  }
  if (mask) {
    hipLaunchKernelGGL(sgpt_mask_kernel, dim3((unsigned)((R * K + 255) / 256)), dim3(256), 0, st, Wf, R * K, mask);
    LLMC_LAUNCH_STATUS();
  }

  SgptParams p;
  p.Wf = Wf; p.R = (int)R; p.K = (int)K; p.U = U; p.ldu = ldu; p.mask = mask;
  p.prune_n = prune_n; p.prune_m = nm ? prune_m : 1; p.loss_rows = loss_rows;
  const int smem = GB * GB * 4;
  void (*kern)(SgptParams) = nm ? sgpt_block_kernel<true> : sgpt_block_kernel<false>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return 1000 + (int)e;
  const unsigned wgs = (unsigned)((R + ROWS_PER_WG - 1) / ROWS_PER_WG);
  const int ldE = GROUP * GB;
  p.ldE = ldE;
  auto rezero = [&](int64_t c0, int64_t c1) {  // preserved zeros in columns [c0, c1) back to zero
    if (!mask || c0 >= c1) return;
    hipLaunchKernelGGL(sgpt_rezero_kernel, dim3((unsigned)((c1 - c0 + 255) / 256), (unsigned)R), dim3(256), 0, st, Wf,
                       mask, (int)K, (int)c0, (int)c1, left ? (float*)extra : (float*)nullptr);
  };
  // the same two-level lazy updates as the quantiser's loop
  int64_t blk = 0;
  for (int64_t g0 = 0, gend = 0; g0 < K; g0 = gend) {
    gend = left ? left_group_end(g0, K) : ((g0 + (int64_t)GROUP * bs) < K ? g0 + (int64_t)GROUP * bs : K);
    if (left && (g0 > 0 || gend < K)) {  // what the group owes to the earlier columns, from the factor of H
      const int rc = left_begin_group(1, R, K, g0, U, ldu, 0, Wf, extra, st);
      if (rc) return rc;
      if (g0 > 0) rezero(g0, gend);
      LLMC_LAUNCH_STATUS();
    }
    for (int64_t i1 = g0; i1 < gend; i1 += bs, ++blk) {
      const int count = (int)((gend - i1) < bs ? (gend - i1) : bs);
      p.i1 = (int)i1;
      p.count = count;
      p.E = E + (i1 - g0);
      p.hist = hist + blk * SG_HIST_WORDS;
      p.k = (unsigned)((double)(R * count) * sparsity);
      if (!nm) {
        const unsigned hw = (unsigned)((R * count + 256 * 16 - 1) / (256 * 16));
        hipLaunchKernelGGL(sgpt_hist_kernel<0>, dim3(hw), dim3(256), 0, st, p);
        hipLaunchKernelGGL(sgpt_hist_kernel<1>, dim3(hw), dim3(256), 0, st, p);
        hipLaunchKernelGGL(sgpt_hist_kernel<2>, dim3(hw), dim3(256), 0, st, p);
        LLMC_LAUNCH_STATUS();
      }
      hipLaunchKernelGGL(kern, dim3(wgs), dim3(256), smem, st, p);
      LLMC_LAUNCH_STATUS();
      const int64_t i2 = i1 + count;
      if (i2 < gend) {
        int rc = launch_group_update(p.E, ldE, U, ldu, 0, Wf, R, K, 1, i1, count, i2, gend, st);
        if (rc < 0) {
          GemmF32 g = {};
          g.A = p.E; g.lda = ldE; g.B = U + i1 * ldu + i2; g.ldb = ldu; g.C = Wf + i2; g.ldc = K;
          g.M = (int)R; g.N = (int)(gend - i2); g.Kc = count; g.alpha = -1.f; g.beta = 1.f; g.batch = 1;
          rc = llmc_gemm_f32(g, st);
        }
        if (rc) return rc;
        rezero(i2, gend);
        LLMC_LAUNCH_STATUS();
      }
    }
    if (gend < K && left) {
      const int rc = left_end_group(1, R, K, g0, Wf, extra, st);
      if (rc) return rc;
    } else if (gend < K) {
      GemmF32 g = {};
      g.A = E; g.lda = ldE; g.B = U + g0 * ldu + gend; g.ldb = ldu; g.C = Wf + gend; g.ldc = K;
      g.M = (int)R; g.N = (int)(K - gend); g.Kc = (int)(gend - g0); g.alpha = -1.f; g.beta = 1.f; g.batch = 1;
      const int rc = llmc_gemm_f32(g, st);
      if (rc) return rc;
      rezero(gend, K);
      LLMC_LAUNCH_STATUS();
    }
  }

#define LLMC_FIN(DT) \
  hipLaunchKernelGGL((gptq_finalize_kernel<DT>), grid2, dim3(256), 0, st, Wf, (int)R, (int)K, \
                     (const int32_t*)nullptr, out_weight, ldo)
  if (w_dtype == LLMC_BF16) LLMC_FIN(LLMC_BF16);
  else if (w_dtype == LLMC_F16) LLMC_FIN(LLMC_F16);
  else LLMC_FIN(LLMC_F32);
#undef LLMC_FIN
  LLMC_LAUNCH_STATUS();
  if (loss_out) {
    hipLaunchKernelGGL(sum_rows_kernel, dim3(1), dim3(256), 0, st, loss_rows, (int)R, loss_out);
    LLMC_LAUNCH_STATUS();
  }
  return 0;
}

// The quantiser's blocked column loop for n problems of one shape (n = 1: the single call), lazy updates on
// two levels.  After a block is quantised its scaled errors E_b update only the columns left in its group of
// GROUP blocks (what the next block needs); the columns beyond the group get the whole group's errors in one
// rank-(GROUP*bs) product.  Same sums as updating everything after every block, regrouped -- but the big part
// of W is read and written a quarter as often, which is what bounds a rank-128 update.
static int gptq_column_loop(void (*kern)(GptqBlockParams), GptqBlockParams p, int smem, unsigned wgs, int n, int64_t R,
                            int64_t K, int bs, float* E, const float* U, int64_t ldu, int64_t u_stride, float* Wf,
                            int form, char* extra, hipStream_t st) {
  const int ldE = GROUP * GB;
  p.ldE = ldE;
  const int64_t gw = (int64_t)GROUP * bs;
  const bool left = form == LLMC_FACTOR_GROUPS;  // the callers have checked gw == 512 and K % 128 == 0
  auto product = [&](const float* A, int64_t k0, int64_t kc, int64_t c0, int64_t c1) {
    GemmF32 g = {};
    g.A = A; g.lda = ldE; g.B = U + k0 * ldu + c0; g.ldb = ldu; g.C = Wf + c0; g.ldc = K;
    g.M = (int)R; g.N = (int)(c1 - c0); g.Kc = (int)kc; g.alpha = -1.f; g.beta = 1.f;
    g.batch = 1; g.batch2 = n; g.stride2_a = R * (int64_t)ldE; g.stride2_b = u_stride; g.stride2_c = R * K;
    return llmc_gemm_f32(g, st);
  };
  for (int64_t g0 = 0, gend = 0; g0 < K; g0 = gend) {
    gend = left ? left_group_end(g0, K) : ((g0 + gw) < K ? g0 + gw : K);
    if (left && (g0 > 0 || gend < K)) {  // the only group of a narrow weight needs neither D nor a sum
      const int rc = left_begin_group(n, R, K, g0, U, ldu, u_stride, Wf, extra, st);
      if (rc) return rc;
    }
    for (int64_t i1 = g0; i1 < gend; i1 += bs) {
      const int count = (int)((gend - i1) < bs ? (gend - i1) : bs);
      p.i1 = (int)i1;
      p.count = count;
      p.E = E + (i1 - g0);
      hipLaunchKernelGGL(kern, dim3(wgs, (unsigned)n), dim3(256), smem, st, p);
      LLMC_LAUNCH_STATUS();
      const int64_t i2 = i1 + count;
      if (i2 < gend) {
        int rc = launch_group_update(p.E, ldE, U, ldu, u_stride, Wf, R, K, n, i1, count, i2, gend, st);
        if (rc < 0) rc = product(p.E, i1, count, i2, gend);
        if (rc) return rc;
      }
    }
    if (gend < K) {
      if (left) {
        const int rc = left_end_group(n, R, K, g0, Wf, extra, st);
        if (rc) return rc;
      } else {
        const int rc = product(E, g0, gend - g0, gend, K);
        if (rc) return rc;
      }
    }
  }
  return 0;
}

extern "C" int64_t llmc_gptq_quantize_workspace_bytes(int64_t R, int64_t K, int32_t form) {
  return align256(R * K * 4) + align256(R * GROUP * GB * 4) + align256(R * 4) + left_extra_bytes(1, R, K, form);
}

extern "C" int llmc_gptq_quantize(const void* weight, int32_t w_dtype, int64_t R, int64_t K, int64_t ldw,
                                  const float* U, int64_t ldu, const int32_t* perm, const uint8_t* dead,
                                  const void* scale, int32_t scale_dtype, const int8_t* zero_point,
                                  const float* global_scale, const int32_t* g_idx, int64_t row_div,
                                  int64_t scale_row_stride, int32_t fmt, int32_t num_bits, int32_t blocksize,
                                  int32_t form, void* out_weight, int64_t ldo, float* loss_out, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(weight != nullptr, 1);
  LLMC_CHECK_ARG(form == LLMC_FACTOR_INVERSE ||
                     (form == LLMC_FACTOR_GROUPS && left_form_fits(K, blocksize)), 20);
  LLMC_CHECK_ARG(w_dtype >= 0 && w_dtype <= 2, 2);
  LLMC_CHECK_ARG(R > 0 && R < (1ll << 31), 3);
  LLMC_CHECK_ARG(K > 0 && K < (1ll << 31), 4);
  LLMC_CHECK_ARG(ldw >= K, 5);
  LLMC_CHECK_ARG(U != nullptr && ldu >= K, 6);
  LLMC_CHECK_ARG(scale != nullptr, 10);
  LLMC_CHECK_ARG(scale_dtype >= 0 && scale_dtype <= 2, 11);
  LLMC_CHECK_ARG(row_div > 0 && scale_row_stride >= 0, 15);
  LLMC_CHECK_ARG(fmt >= 0 && fmt <= 2, 17);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || (num_bits >= 2 && num_bits <= 8), 18);
  LLMC_CHECK_ARG(blocksize > 0, 19);
  LLMC_CHECK_ARG(out_weight != nullptr && ldo >= K, 20);
  LLMC_CHECK_ARG(workspace != nullptr && (((uintptr_t)workspace) & 255) == 0, 23);
  LLMC_CHECK_ARG(workspace_bytes >= llmc_gptq_quantize_workspace_bytes(R, K, form), 24);
  hipStream_t st = (hipStream_t)stream;
  // the result does not depend on the block width mathematically (lazy batching only
  // regroups fp32 sums); widths above what fits on chip run as 128-wide blocks
  const int bs = blocksize > GB ? GB : blocksize;

  float* Wf = (float*)workspace;
  float* E = (float*)((char*)workspace + align256(R * K * 4));
  float* loss_rows = (float*)((char*)E + align256(R * GROUP * GB * 4));
  char* extra = (char*)loss_rows + align256(R * 4);

  dim3 grid2((unsigned)((K + 255) / 256), (unsigned)R);
  const bool by_rows = perm != nullptr && K <= ROW_STAGE_MAX;  // permuted columns: gather and scatter a row in LDS
#define LLMC_PREP(DT)                                                                                               \
  if (by_rows) {                                                                                                    \
    const int arc = allow_row_stage(gptq_prepare_w_rows_kernel<DT>, (int)K);                                        \
    if (arc) return arc;                                                                                            \
    hipLaunchKernelGGL((gptq_prepare_w_rows_kernel<DT>), dim3((unsigned)R), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4, st, weight, ldw, \
                       (int)R, (int)K, perm, dead, Wf, (const GptqItem*)nullptr);                                   \
  } else {                                                                                                          \
    hipLaunchKernelGGL((gptq_prepare_w_kernel<DT>), grid2, dim3(256), 0, st, weight, ldw, (int)R, (int)K, perm, dead, \
                       Wf);                                                                                         \
  }
  if (w_dtype == LLMC_BF16) LLMC_PREP(LLMC_BF16)
  else if (w_dtype == LLMC_F16) LLMC_PREP(LLMC_F16)
  else LLMC_PREP(LLMC_F32)
#undef LLMC_PREP
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0, st, loss_rows, R);
  LLMC_LAUNCH_STATUS();

  GptqBlockParams p;
  p.Wf = Wf; p.R = (int)R; p.K = (int)K; p.U = U; p.ldu = ldu;
  p.scale = scale; p.scale_dt = scale_dtype; p.zp = zero_point; p.gscale = global_scale; p.g_idx = g_idx;
  p.row_div = row_div; p.srow = scale_row_stride;
  p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.sd = global_scale ? LLMC_F32 : scale_dtype;
  p.E = E; p.loss_rows = loss_rows;
  p.items = nullptr; p.u_stride = 0;

  const int smem = (GB * GB + 2 * GB) * 4;
  void (*kern)(GptqBlockParams) = nullptr;
  const bool hz = zero_point != nullptr;
  const bool wide_team = R <= Q_WIDE_TEAM_MAX_ROWS;
#define LLMC_PICK(F, S)                                                                                  \
  if (p.fmt == F && p.sd == S)                                                                           \
    kern = wide_team ? (hz ? gptq_block_kernel<F, S, true, 16> : gptq_block_kernel<F, S, false, 16>)     \
                     : (hz ? gptq_block_kernel<F, S, true, 4> : gptq_block_kernel<F, S, false, 4>);
  LLMC_PICK(LLMC_FMT_INT, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_INT, LLMC_F16)
  LLMC_PICK(LLMC_FMT_INT, LLMC_F32)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_F16)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_F32)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_F16)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_F32)
#undef LLMC_PICK
  if (kern == nullptr) return -17;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return 1000 + (int)e;
  const int rows_per_wg = wide_team ? QLayout<16>::ROWS_PER_WG : QLayout<4>::ROWS_PER_WG;
  const unsigned wgs = (unsigned)((R + rows_per_wg - 1) / rows_per_wg);
  {
    const int rc = gptq_column_loop(kern, p, smem, wgs, 1, R, K, bs, E, U, ldu, 0, Wf, form, extra, st);
    if (rc) return rc;
  }

#define LLMC_FIN(DT)                                                                                                \
  if (by_rows) {                                                                                                    \
    const int arc = allow_row_stage(gptq_finalize_rows_kernel<DT>, (int)K);                                         \
    if (arc) return arc;                                                                                            \
    hipLaunchKernelGGL((gptq_finalize_rows_kernel<DT>), dim3((unsigned)R), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4, st, Wf, (int)R,   \
                       (int)K, perm, out_weight, ldo, (const GptqItem*)nullptr);                                    \
  } else {                                                                                                          \
    hipLaunchKernelGGL((gptq_finalize_kernel<DT>), grid2, dim3(256), 0, st, Wf, (int)R, (int)K, perm, out_weight, ldo); \
  }
  if (w_dtype == LLMC_BF16) LLMC_FIN(LLMC_BF16)
  else if (w_dtype == LLMC_F16) LLMC_FIN(LLMC_F16)
  else LLMC_FIN(LLMC_F32)
#undef LLMC_FIN
  LLMC_LAUNCH_STATUS();
  if (loss_out) {
    hipLaunchKernelGGL(sum_rows_kernel, dim3(1), dim3(256), 0, st, loss_rows, (int)R, loss_out);
    LLMC_LAUNCH_STATUS();
  }
  return 0;
}

// ---- grouped form: n problems of one shape in lock-step (the expert Linears of an MoE layer) ---------
// Every kernel of llmc_gptq_quantize is launched once for all problems (one more grid dimension, GEMM batch):
// the serial chain of column blocks is as long as one problem's while each launch carries n times the rows.

extern "C" int64_t llmc_gptq_quantize_grouped_workspace_bytes(int64_t n, int64_t R, int64_t K, int32_t form) {
  return align256(n * (int64_t)sizeof(GptqItem)) + align256(n * R * K * 4) + align256(n * R * GROUP * GB * 4) +
         align256(n * R * 4) + left_extra_bytes(n, R, K, form);
}

extern "C" int llmc_gptq_quantize_grouped(const void* const* weight, int32_t w_dtype, int32_t n, int64_t R, int64_t K,
                                          int64_t ldw, const float* U, int64_t ldu, int64_t u_stride,
                                          const int32_t* perm, const uint8_t* dead, const void* const* scale,
                                          int32_t scale_dtype, const int8_t* const* zero_point,
                                          const float* const* global_scale, const int32_t* const* g_idx,
                                          int64_t row_div, int64_t scale_row_stride, int32_t fmt, int32_t num_bits,
                                          int32_t blocksize, int32_t form, void* const* out_weight, int64_t ldo,
                                          float* loss_out, void* workspace, int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(weight != nullptr, 1);
  LLMC_CHECK_ARG(form == LLMC_FACTOR_INVERSE ||
                     (form == LLMC_FACTOR_GROUPS && left_form_fits(K, blocksize)), 22);
  LLMC_CHECK_ARG(w_dtype >= 0 && w_dtype <= 2, 2);
  LLMC_CHECK_ARG(n >= 0 && n <= 4096, 3);
  if (n == 0) return 0;
  LLMC_CHECK_ARG(R > 0 && R < (1ll << 31), 4);
  LLMC_CHECK_ARG(K > 0 && K < (1ll << 31) && ldw >= K, 5);
  LLMC_CHECK_ARG(U != nullptr && ldu >= K && u_stride >= K * ldu, 7);
  LLMC_CHECK_ARG(scale != nullptr, 12);
  LLMC_CHECK_ARG(scale_dtype >= 0 && scale_dtype <= 2, 13);
  LLMC_CHECK_ARG(row_div > 0 && scale_row_stride >= 0, 17);
  LLMC_CHECK_ARG(fmt >= 0 && fmt <= 2, 19);
  LLMC_CHECK_ARG(fmt != LLMC_FMT_INT || (num_bits >= 2 && num_bits <= 8), 20);
  LLMC_CHECK_ARG(blocksize > 0, 21);
  LLMC_CHECK_ARG(out_weight != nullptr && ldo >= K, 22);
  LLMC_CHECK_ARG(workspace != nullptr && (((uintptr_t)workspace) & 255) == 0, 25);
  LLMC_CHECK_ARG(workspace_bytes >= llmc_gptq_quantize_grouped_workspace_bytes(n, R, K, form), 26);
  LLMC_CHECK_ARG(n < 65535 && (K + 255) / 256 < 65535, 3);
  hipStream_t st = (hipStream_t)stream;
  const int bs = blocksize > GB ? GB : blocksize;

  char* wp = (char*)workspace;
  GptqItem* items = (GptqItem*)wp; wp += align256(n * (int64_t)sizeof(GptqItem));
  float* Wf = (float*)wp; wp += align256(n * R * K * 4);
  float* E = (float*)wp; wp += align256(n * R * GROUP * GB * 4);
  float* loss_rows = (float*)wp; wp += align256(n * R * 4);
  char* extra = wp;
  std::vector<GptqItem> host(n);
  for (int b = 0; b < n; ++b) {
    LLMC_CHECK_ARG(weight[b] != nullptr && scale[b] != nullptr && out_weight[b] != nullptr, 1);
    host[b].weight = weight[b];
    host[b].scale = scale[b];
    host[b].zp = zero_point ? zero_point[b] : nullptr;
    host[b].gscale = global_scale ? global_scale[b] : nullptr;
    host[b].g_idx = g_idx ? g_idx[b] : nullptr;
    host[b].out = out_weight[b];
  }
  {
    const int urc = upload_items(host.data(), n, (GptqItem*)items, st);
    if (urc) return urc;
  }

  dim3 grid3((unsigned)((K + 255) / 256), (unsigned)R, (unsigned)n);
  const bool by_rows = perm != nullptr && K <= ROW_STAGE_MAX;  // as in the single-problem call
#define LLMC_PREP(DT)                                                                                           \
  if (by_rows) {                                                                                                \
    const int arc = allow_row_stage(gptq_prepare_w_rows_kernel<DT>, (int)K);                                    \
    if (arc) return arc;                                                                                        \
    hipLaunchKernelGGL((gptq_prepare_w_rows_kernel<DT>), dim3((unsigned)R, (unsigned)n), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4, \
                       st, (const void*)nullptr, ldw, (int)R, (int)K, perm, dead, Wf, (const GptqItem*)items);  \
  } else {                                                                                                      \
    hipLaunchKernelGGL((gptq_prepare_w_kernel<DT>), grid3, dim3(256), 0, st, (const void*)nullptr, ldw, (int)R, \
                       (int)K, perm, dead, Wf, (const GptqItem*)items);                                         \
  }
  if (w_dtype == LLMC_BF16) LLMC_PREP(LLMC_BF16)
  else if (w_dtype == LLMC_F16) LLMC_PREP(LLMC_F16)
  else LLMC_PREP(LLMC_F32)
#undef LLMC_PREP
  LLMC_LAUNCH_STATUS();
  hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n * R + 255) / 256)), dim3(256), 0, st, loss_rows, n * R);
  LLMC_LAUNCH_STATUS();

  GptqBlockParams p;
  p.Wf = Wf; p.R = (int)R; p.K = (int)K; p.U = U; p.ldu = ldu;
  p.scale = nullptr; p.scale_dt = scale_dtype; p.zp = nullptr; p.gscale = nullptr; p.g_idx = nullptr;
  p.row_div = row_div; p.srow = scale_row_stride;
  p.fmt = fmt; p.bits = fmt == LLMC_FMT_INT ? num_bits : (fmt == LLMC_FMT_FP8 ? 8 : 4);
  p.sd = global_scale ? LLMC_F32 : scale_dtype;
  p.E = E; p.loss_rows = loss_rows;
  p.items = items; p.u_stride = u_stride;

  const int smem = (GB * GB + 2 * GB) * 4;
  void (*kern)(GptqBlockParams) = nullptr;
  const bool hz = zero_point != nullptr;
  const bool wide_team = (int64_t)n * R <= Q_WIDE_TEAM_MAX_ROWS;
#define LLMC_PICK(F, S)                                                                                  \
  if (p.fmt == F && p.sd == S)                                                                           \
    kern = wide_team ? (hz ? gptq_block_kernel<F, S, true, 16> : gptq_block_kernel<F, S, false, 16>)     \
                     : (hz ? gptq_block_kernel<F, S, true, 4> : gptq_block_kernel<F, S, false, 4>);
  LLMC_PICK(LLMC_FMT_INT, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_INT, LLMC_F16)
  LLMC_PICK(LLMC_FMT_INT, LLMC_F32)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_F16)
  LLMC_PICK(LLMC_FMT_FP8, LLMC_F32)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_BF16)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_F16)
  LLMC_PICK(LLMC_FMT_FP4, LLMC_F32)
#undef LLMC_PICK
  if (kern == nullptr) return -19;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return 1000 + (int)e;
  const int rows_per_wg = wide_team ? QLayout<16>::ROWS_PER_WG : QLayout<4>::ROWS_PER_WG;
  const unsigned wgs = (unsigned)((R + rows_per_wg - 1) / rows_per_wg);
  {
    const int rc = gptq_column_loop(kern, p, smem, wgs, n, R, K, bs, E, U, ldu, u_stride, Wf, form, extra, st);
    if (rc) return rc;
  }

#define LLMC_FIN(DT)                                                                                            \
  if (by_rows) {                                                                                                \
    const int arc = allow_row_stage(gptq_finalize_rows_kernel<DT>, (int)K);                                     \
    if (arc) return arc;                                                                                        \
    hipLaunchKernelGGL((gptq_finalize_rows_kernel<DT>), dim3((unsigned)R, (unsigned)n), dim3(K > 8192 ? 1024 : 256), (size_t)K * 4,  \
                       st, Wf, (int)R, (int)K, perm, (void*)nullptr, ldo, (const GptqItem*)items);              \
  } else {                                                                                                      \
    hipLaunchKernelGGL((gptq_finalize_kernel<DT>), grid3, dim3(256), 0, st, Wf, (int)R, (int)K, perm,           \
                       (void*)nullptr, ldo, (const GptqItem*)items);                                            \
  }
  if (w_dtype == LLMC_BF16) LLMC_FIN(LLMC_BF16)
  else if (w_dtype == LLMC_F16) LLMC_FIN(LLMC_F16)
  else LLMC_FIN(LLMC_F32)
#undef LLMC_FIN
  LLMC_LAUNCH_STATUS();
  if (loss_out) {
    hipLaunchKernelGGL(sum_rows_kernel, dim3((unsigned)n), dim3(256), 0, st, loss_rows, (int)R, loss_out);
    LLMC_LAUNCH_STATUS();
  }
  return 0;
}
