// GPTQ quantize_weight: blocked column loop with error feedback.
//
// Rows of W are independent given the inverse-Hessian factor U, so a workgroup
// owns 16 rows and never synchronises with another one inside a block of
// columns.  A row is spread over a team of 16 lanes, 8 columns of the block per
// lane, held in registers.  The block's 128x128 slice of U sits in LDS.  Per
// column: the owning lane's value is broadcast inside the team, every lane
// quantises it, forms err = (w - q)/U[i][i] and subtracts err * U[i][c] from its
// own 8 columns (U is zero below the diagonal, so no masking is needed).
// After the block, W[:, i2:] -= Err * U[i1:i2, i2:] runs as an fp32 MFMA GEMM.
#include "gemm_f32.h"
#include "qformat.h"

namespace {

constexpr int GB = 128;       // widest column block held on chip
constexpr int GROUP = 4;      // column blocks whose updates of the far columns are applied together
constexpr int TEAM = 16;      // lanes per row
constexpr int CPL = GB / TEAM;  // columns per lane (8)
constexpr int ROWS_PER_WG = 256 / TEAM;

template <int WDT>
__global__ __launch_bounds__(256) void gptq_prepare_w_kernel(const void* __restrict__ w, int64_t ldw, int R,
                                                             int K, const int32_t* __restrict__ perm,
                                                             const uint8_t* __restrict__ dead,
                                                             float* __restrict__ Wf) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (c >= K) return;
  const int src = perm ? perm[c] : c;
  float v = load_as_f32<WDT>(w, (int64_t)r * ldw + src);
  if (dead && dead[c]) v = 0.f;
  Wf[(int64_t)r * K + c] = v;
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
};

template <int FMT, int SD, bool HAS_ZP>
__global__ __launch_bounds__(256) void gptq_block_kernel(GptqBlockParams p) {
  extern __shared__ __attribute__((aligned(16))) float Hs[];  // [GB][GB], zero outside the upper triangle
  const int tid = threadIdx.x;
  for (int e = tid; e < GB * GB; e += 256) {
    const int i = e / GB, c = e % GB;
    Hs[e] = (c >= i && c < p.count) ? p.U[(int64_t)(p.i1 + i) * p.ldu + p.i1 + c] : 0.f;
  }
  const int tl = tid % TEAM;
  const int row = blockIdx.x * ROWS_PER_WG + tid / TEAM;
  const bool live = row < p.R;
  const QFormat f = make_qformat(FMT, p.bits);  // the format is a compile-time constant here
  constexpr bool has_zp = HAS_ZP;
  const float gs = p.gscale ? p.gscale[0] : 1.f;

  float w[CPL], sv[CPL], zv[CPL], qv[CPL], ev[CPL];
#pragma unroll
  for (int e = 0; e < CPL; ++e) {
    const int cb = tl * CPL + e;
    const int c = p.i1 + cb;
    w[e] = 0.f;
    sv[e] = 1.f;
    zv[e] = 0.f;
    qv[e] = 0.f;
    ev[e] = 0.f;
    if (live && cb < p.count) {
      w[e] = p.Wf[(int64_t)row * p.K + c];
      const int64_t si = ((int64_t)row / p.row_div) * p.srow + (p.g_idx ? (int64_t)p.g_idx[c] : 0);
      float s = load_rt(p.scale, si, p.scale_dt);
      if (p.gscale) s = s / gs;
      sv[e] = s;
      if (has_zp) zv[e] = (float)p.zp[si];
    }
  }
  __syncthreads();

  float loss = 0.f;
  for (int li = 0; li < TEAM; ++li) {
    if (li * CPL >= p.count) break;
#pragma unroll
    for (int e = 0; e < CPL; ++e) {
      const int i = li * CPL + e;
      if (i < p.count) {  // uniform across the workgroup
        const float wv = __shfl(w[e], li, TEAM);
        const float s = __shfl(sv[e], li, TEAM);
        const float zp = has_zp ? __shfl(zv[e], li, TEAM) : 0.f;
        const float qc = quantize_value(wv, s, zp, has_zp, LLMC_F32, f);
        const float q = dequantize_value(qc, s, zp, has_zp, SD);
        const float d = Hs[i * GB + i];
        const float diff = __fsub_rn(wv, q);
        const float err = diff / d;
        loss += err * err;  // (w-q)^2 / d^2
        const float4 h0 = *(const float4*)&Hs[i * GB + tl * CPL];
        const float4 h1 = *(const float4*)&Hs[i * GB + tl * CPL + 4];
        // product rounded, then subtracted: the reference forms the outer product first
        w[0] = __fsub_rn(w[0], __fmul_rn(err, h0.x));
        w[1] = __fsub_rn(w[1], __fmul_rn(err, h0.y));
        w[2] = __fsub_rn(w[2], __fmul_rn(err, h0.z));
        w[3] = __fsub_rn(w[3], __fmul_rn(err, h0.w));
        w[4] = __fsub_rn(w[4], __fmul_rn(err, h1.x));
        w[5] = __fsub_rn(w[5], __fmul_rn(err, h1.y));
        w[6] = __fsub_rn(w[6], __fmul_rn(err, h1.z));
        w[7] = __fsub_rn(w[7], __fmul_rn(err, h1.w));
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

template <int WDT>
__global__ __launch_bounds__(256) void gptq_finalize_kernel(const float* __restrict__ Wf, int R, int K,
                                                            const int32_t* __restrict__ perm,
                                                            void* __restrict__ out, int64_t ldo) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (c >= K) return;
  const int dst = perm ? perm[c] : c;
  store_from_f32<WDT>(out, (int64_t)r * ldo + dst, Wf[(int64_t)r * K + c]);
}

__global__ __launch_bounds__(256) void sum_rows_kernel(const float* __restrict__ v, int n, float* out) {
  __shared__ float red[4];
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

}  // namespace

extern "C" int64_t llmc_gptq_quantize_workspace_bytes(int64_t R, int64_t K) {
  return align256(R * K * 4) + align256(R * GROUP * GB * 4) + align256(R * 4);
}

extern "C" int llmc_gptq_quantize(const void* weight, int32_t w_dtype, int64_t R, int64_t K, int64_t ldw,
                                  const float* U, int64_t ldu, const int32_t* perm, const uint8_t* dead,
                                  const void* scale, int32_t scale_dtype, const int8_t* zero_point,
                                  const float* global_scale, const int32_t* g_idx, int64_t row_div,
                                  int64_t scale_row_stride, int32_t fmt, int32_t num_bits, int32_t blocksize,
                                  void* out_weight, int64_t ldo, float* loss_out, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  LLMC_CHECK_ARG(weight != nullptr, 1);
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
  LLMC_CHECK_ARG(workspace_bytes >= llmc_gptq_quantize_workspace_bytes(R, K), 24);
  hipStream_t st = (hipStream_t)stream;
  // the result does not depend on the block width mathematically (lazy batching only
  // regroups fp32 sums); widths above what fits on chip run as 128-wide blocks
  const int bs = blocksize > GB ? GB : blocksize;

  float* Wf = (float*)workspace;
  float* E = (float*)((char*)workspace + align256(R * K * 4));
  float* loss_rows = (float*)((char*)E + align256(R * GROUP * GB * 4));

  dim3 grid2((unsigned)((K + 255) / 256), (unsigned)R);
#define LLMC_PREP(DT) \
  hipLaunchKernelGGL((gptq_prepare_w_kernel<DT>), grid2, dim3(256), 0, st, weight, ldw, (int)R, (int)K, perm, dead, Wf)
  if (w_dtype == LLMC_BF16) LLMC_PREP(LLMC_BF16);
  else if (w_dtype == LLMC_F16) LLMC_PREP(LLMC_F16);
  else LLMC_PREP(LLMC_F32);
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

  const int smem = GB * GB * 4;
  void (*kern)(GptqBlockParams) = nullptr;
  const bool hz = zero_point != nullptr;
#define LLMC_PICK(F, S)                                                         \
  if (p.fmt == F && p.sd == S) kern = hz ? gptq_block_kernel<F, S, true> : gptq_block_kernel<F, S, false>;
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
  const unsigned wgs = (unsigned)((R + ROWS_PER_WG - 1) / ROWS_PER_WG);
  // Lazy updates on two levels.  After a block is quantised its scaled errors E_b update only the
  // columns left in its group of GROUP blocks (what the next block needs); the columns beyond the
  // group get the whole group's errors in one rank-(GROUP*bs) product.  Same sums as updating
  // everything after every block, regrouped -- but the big part of W is read and written a
  // quarter as often, which is what bounds a rank-128 update.
  const int ldE = GROUP * GB;
  p.ldE = ldE;
  for (int64_t g0 = 0; g0 < K; g0 += (int64_t)GROUP * bs) {
    const int64_t gend = (g0 + (int64_t)GROUP * bs) < K ? g0 + (int64_t)GROUP * bs : K;
    for (int64_t i1 = g0; i1 < gend; i1 += bs) {
      const int count = (int)((gend - i1) < bs ? (gend - i1) : bs);
      p.i1 = (int)i1;
      p.count = count;
      p.E = E + (i1 - g0);
      hipLaunchKernelGGL(kern, dim3(wgs), dim3(256), smem, st, p);
      LLMC_LAUNCH_STATUS();
      const int64_t i2 = i1 + count;
      if (i2 < gend) {
        GemmF32 g = {};
        g.A = p.E; g.lda = ldE; g.B = U + i1 * ldu + i2; g.ldb = ldu; g.C = Wf + i2; g.ldc = K;
        g.M = (int)R; g.N = (int)(gend - i2); g.Kc = count; g.alpha = -1.f; g.beta = 1.f; g.batch = 1;
        const int rc = llmc_gemm_f32(g, st);
        if (rc) return rc;
      }
    }
    if (gend < K) {
      GemmF32 g = {};
      g.A = E; g.lda = ldE; g.B = U + g0 * ldu + gend; g.ldb = ldu; g.C = Wf + gend; g.ldc = K;
      g.M = (int)R; g.N = (int)(K - gend); g.Kc = (int)(gend - g0); g.alpha = -1.f; g.beta = 1.f; g.batch = 1;
      const int rc = llmc_gemm_f32(g, st);
      if (rc) return rc;
    }
  }

#define LLMC_FIN(DT) \
  hipLaunchKernelGGL((gptq_finalize_kernel<DT>), grid2, dim3(256), 0, st, Wf, (int)R, (int)K, perm, out_weight, ldo)
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
