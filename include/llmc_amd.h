/*
 * llmc_amd -- MI355X (gfx950) kernels for llm-compressor's calibration-time
 * quantization hot path, behind a plain C ABI.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless its name ends in _host.
 *   - Matrices are row-major with an explicit leading dimension in ELEMENTS.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all
 *     work is enqueued on it and the call returns without synchronising unless
 *     stated otherwise.
 *   - The library never allocates or frees caller-visible memory; scratch space
 *     is passed in as `workspace` and sized by the matching *_workspace_bytes().
 *   - Return value: 0 = ok; <0 = argument number (1-based, negated) that was
 *     rejected; >0 = algorithm-specific info.  No C++ exception crosses the ABI.
 *
 * "Reference" below is vllm-project/llm-compressor; paths are relative to its
 * tree.  compressed-tensors (CT) is the third-party package the reference calls
 * for number formats; it is cited through the reference's call sites.
 */
#ifndef LLMC_AMD_H
#define LLMC_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activation / weight buffers */
enum { LLMC_BF16 = 0, LLMC_F16 = 1, LLMC_F32 = 2 };

/* element formats of the quantised value */
enum {
  LLMC_FMT_INT = 0,  /* signed integer, num_bits in [2,8], round-half-even       */
  LLMC_FMT_FP8 = 1,  /* float8 e4m3fn, saturating                                */
  LLMC_FMT_FP4 = 2   /* float4 e2m1 grid {0,.5,1,1.5,2,3,4,6}                    */
};

/* how scales are derived / stored */
enum {
  LLMC_SCALE_PLAIN = 0, /* scale = absmax/(range/2) (or (max-min)/range), in the observed dtype */
  LLMC_SCALE_NVFP4 = 1, /* scale = e4m3(global_scale * absmax/6); effective = stored/global_scale */
  LLMC_SCALE_MXFP4 = 2  /* scale = 2^(e-127), e stored as uint8 (E8M0)                              */
};

int llmc_version(void);

/* ---- a1/a2: GPTQ Hessian -------------------------------------------------
 * Replaces accumulate_hessian() for nn.Linear inputs
 * (src/llmcompressor/modifiers/gptq/gptq_quantize.py:28-64):
 *     H[K,K] += alpha * X^T X,   X = [T,K] (tokens x in_features), alpha = 2.
 * bf16/f16 inputs are multiplied exactly and accumulated in fp32 on the MFMA
 * units.  fp32 inputs (x_dtype = LLMC_F32; this entry point only, not the grouped
 * and segmented forms) take the fp32 matrix-core GEMM over the full K x K matrix and
 * ignore flags and workspace.  Only the upper-triangular tiles are computed.  With
 * LLMC_HESSIAN_ASSUME_SYMMETRIC the mirrored lower tiles are stored from the
 * upper results (H must be bitwise symmetric on entry, which holds for a
 * buffer that started as zeros and was only ever updated by this call);
 * without it the lower tiles are read-modify-written too.
 * `workspace` (16-byte aligned device memory, llmc_hessian_workspace_bytes(T, K)
 * bytes; may be NULL/0) lets the tiles that do not fill a whole round of
 * workgroups be cut along the tokens: the chunks' partial tiles go through the
 * workspace and are summed in a fixed order, so the result does not depend on
 * timing.  Without it every tile is one workgroup (slower when the tile count
 * is not a multiple of the CU count).  Its first 64 KiB hold progress words with
 * which workgroups that share an L2 pace each other over long token loops (fewer
 * re-fetches of X; the result does not depend on them).  The workspace holds no
 * state between calls; calls that overlap in time need workspaces of their own.
 */
enum { LLMC_HESSIAN_ASSUME_SYMMETRIC = 1 };
int64_t llmc_hessian_workspace_bytes(int64_t T, int64_t K);
int llmc_hessian_accumulate(float* H, int64_t ldh, const void* X, int64_t ldx,
                            int64_t T, int64_t K, int32_t x_dtype, float alpha,
                            int32_t flags, void* workspace, int64_t workspace_bytes,
                            void* stream);

/* Grouped form for the per-expert Hessians of an MoE layer (the 128 x 3 accumulate_hessian calls
 * that LinearExperts2D.forward triggers per batch, modeling/moe/linear_experts.py:235-268): n
 * independent problems of one width K in one launch.  H, X and T are HOST arrays of n device
 * pointers / token counts (they are passed to the kernel by value, 128 problems per launch); all
 * problems share ldh, ldx and the dtype; K % 8 == 0 and every X[i] 16-byte aligned.  A problem
 * with T[i] == 0 (an expert that received no token) leaves its Hessian untouched. */
int llmc_hessian_accumulate_grouped(float* const* H, int64_t ldh, const void* const* X, int64_t ldx,
                                    const int64_t* T, int32_t n, int64_t K, int32_t x_dtype,
                                    float alpha, int32_t flags, void* stream);

/* Segmented form: the token rows of ONE problem lie in n_seg separate buffers (the calibration
 * batches exactly as GPTQModifier.calibrate_module receives them, modifiers/gptq/base.py:240-262),
 * so that accumulating several batches with one launch does not need them copied together first.
 * X is a HOST array of n_seg (<= 64) device pointers, each 16-byte aligned and holding seg_tokens
 * rows of stride ldx (seg_tokens % 64 == 0); the last buffer holds last_tokens <= seg_tokens rows.
 * K % 8 == 0 and ldx % 8 == 0.  The result is bit-identical to llmc_hessian_accumulate on the
 * concatenation.  Workspace as for llmc_hessian_accumulate with T = total rows. */
int llmc_hessian_accumulate_segments(float* H, int64_t ldh, const void* const* X, int32_t n_seg,
                                     int64_t seg_tokens, int64_t last_tokens, int64_t ldx, int64_t K,
                                     int32_t x_dtype, float alpha, int32_t flags, void* workspace,
                                     int64_t workspace_bytes, void* stream);

/* ---- a10/a11: min-max observers --------------------------------------------
 * Replace _get_min_max() = torch.amin/amax(observed, dim=(0,-1)) on the
 * flattened weight (src/llmcompressor/observers/min_max.py:70-74 with
 * observers/helpers.py:28-157).  Outputs are in the observed dtype.
 *   llmc_minmax_groups : weight [R,K], groups of `group` consecutive columns
 *                        (group = K: per channel; R=1, group=K=numel: per tensor)
 *                        -> [R, K/group]
 *   llmc_minmax_blocks : block strategy, zero-padded edges -> [ceil(R/bh), ceil(K/bw)]
 *   llmc_minmax_strided: generic (num_observations, n1, group) view with element
 *                        strides (stride0, stride1, 1) -> [n1]  (activations)
 */
int64_t llmc_minmax_workspace_bytes(void);
int llmc_minmax_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                       int64_t group, void* min_out, void* max_out, void* workspace,
                       int64_t workspace_bytes, void* stream);
int llmc_minmax_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                       int32_t block_h, int32_t block_w, void* min_out, void* max_out,
                       void* stream);
int llmc_minmax_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                        int64_t stride0, int64_t stride1, void* min_out, void* max_out,
                        void* stream);

/* ---- a13: MSE observers ------------------------------------------------------
 * Replace _grid_search_mse (eager path, src/llmcompressor/observers/mse_quant.py:19-141,
 * 255-285) for memoryless_mse / mse / nvfp4_expanded_mse: for i in range(steps):
 * p = 1 - i/grid; qparams from (p*min, p*max); err = sum |fq(x) - x|^norm over the
 * group; keep the first strict minimum per group; stop globally after `patience`
 * consecutive steps without any improvement.  steps = int(maxshrink*grid) <= 256.
 * All intermediates are rounded to the observed dtype as the eager ops do.
 * Outputs (min, max) in the observed dtype with the same shapes as the min-max calls.
 * scale_mode is LLMC_SCALE_PLAIN (the reference searches TENSOR_GROUP with
 * scale_dtype=None) or LLMC_SCALE_MXFP4.  workspace: llmc_mse_workspace_bytes(#groups).
 */
int64_t llmc_mse_workspace_bytes(int64_t n_groups);
int llmc_mse_observe_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                            int64_t group, int32_t fmt, int32_t num_bits, int32_t symmetric,
                            int32_t scale_mode, int32_t steps, double grid, int32_t patience,
                            float norm, float expand, void* min_out, void* max_out, void* workspace,
                            int64_t workspace_bytes, void* stream);
int llmc_mse_observe_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                             int64_t stride0, int64_t stride1, int32_t fmt, int32_t num_bits,
                             int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                             int32_t patience, float norm, float expand, void* min_out, void* max_out,
                             void* workspace, int64_t workspace_bytes, void* stream);
int llmc_mse_observe_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                            int32_t block_h, int32_t block_w, int32_t fmt, int32_t num_bits,
                            int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                            int32_t patience, float norm, float expand, void* min_out, void* max_out,
                            void* workspace, int64_t workspace_bytes, void* stream);

/* Importance-weighted search (a "next" row: observers/imatrix.py).
 *   llmc_sumsq_accumulate: sum[c] += sum_t x[t][c]^2 in fp32 -- the forward-pre hook's
 *     token_sum = x.float().pow(2).sum(leading dims) (imatrix.py:93-111) without the fp32 copy of x.
 *   llmc_imatrix_observe_groups: _grid_search (imatrix.py:255-328) on weight [R,K] in groups of `group`
 *     columns (group = K: per channel): candidates i = 0..steps-1 with p = 1 - i/grid, the error
 *     |fq(x) - x|^norm formed and summed in fp32 and multiplied by importance[column] (fp32 [K],
 *     already normalised to mean 1; NULL = uniform), global early stop after `patience` candidates
 *     without any improvement (0 = never).  Workspace as llmc_mse_workspace_bytes(#groups). */
int64_t llmc_sumsq_workspace_bytes(int64_t K);
int llmc_sumsq_accumulate(const void* x, int32_t dtype, int64_t T, int64_t K, int64_t ldx, float* sum,
                          void* workspace, int64_t workspace_bytes, void* stream);
/* llmc_sumsq_accumulate for callers that cannot allocate (code under HIP graph capture, tight loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same result as
 * llmc_sumsq_accumulate bit for bit, but the partial sums go to a 4 MiB device array that the library
 * itself holds on every GPU it runs on (until the process ends) instead of a caller's workspace, and the
 * call allocates and frees nothing.  K above LLMC_SUMSQ_NOALLOC_MAX_K is rejected (-4).  The first call
 * on a device looks up that device's copy of the array (make it before a capture begins).  All calls on
 * one GPU share the array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * on one stream, or ordered by events, do not. */
#define LLMC_SUMSQ_NOALLOC_MAX_K 16384
int llmc_sumsq_accumulate_noalloc(const void* x, int32_t dtype, int64_t T, int64_t K, int64_t ldx, float* sum,
                                  void* stream);
int llmc_imatrix_observe_groups(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                int64_t group, int32_t fmt, int32_t num_bits, int32_t symmetric,
                                int32_t scale_mode, int32_t steps, double grid, int32_t patience,
                                float norm, float expand, const float* importance, void* min_out,
                                void* max_out, void* workspace, int64_t workspace_bytes, void* stream);
/* The same search without weights on the other layouts (the reference routes block-wise weights and
 * non-weight observers to the uniform fall-back, imatrix.py:141-245); arguments as the llmc_mse_observe_*
 * twins, patience 0 = never stop. */
int llmc_imatrix_observe_strided(const void* x, int32_t dtype, int64_t n0, int64_t n1, int64_t group,
                                 int64_t stride0, int64_t stride1, int32_t fmt, int32_t num_bits,
                                 int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                 int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                 void* workspace, int64_t workspace_bytes, void* stream);
int llmc_imatrix_observe_blocks(const void* x, int32_t dtype, int64_t R, int64_t K, int64_t ldw,
                                int32_t block_h, int32_t block_w, int32_t fmt, int32_t num_bits,
                                int32_t symmetric, int32_t scale_mode, int32_t steps, double grid,
                                int32_t patience, float norm, float expand, void* min_out, void* max_out,
                                void* workspace, int64_t workspace_bytes, void* stream);

/* ---- a12/a16: qparams ------------------------------------------------------
 * llmc_absmax_accumulate + llmc_generate_gparam replace Observer.get_global_scale()
 * (src/llmcompressor/observers/base.py:78-96; CT generate_gparam): absmax_inout
 * (fp32, caller zero-initialised) takes max(absmax, -min, max) over the arrays of
 * every observer of a fused group, one call each; gparam = 448*6/absmax evaluated as
 * torch evaluates `float / Tensor` (reciprocal in the statistics' dtype, then the
 * product, rounded again), returned as fp32 [1].
 * llmc_calculate_qparams replaces CT calculate_qparams as called from
 * observers/base.py:114-119: n (min,max) pairs -> scale (scale_out_dtype; fp32
 * e4m3-grid values for LLMC_SCALE_NVFP4), int8 zero points (NULL when symmetric),
 * and optionally the stored scale code (e4m3 byte for NVFP4, E8M0 byte for MXFP4).
 */
int llmc_absmax_accumulate(const void* min_vals, const void* max_vals, int64_t n, int32_t dtype,
                           float* absmax_inout, void* stream);
int llmc_generate_gparam(const float* absmax, int32_t stats_dtype, float* global_scale_out,
                         void* stream);
int llmc_calculate_qparams(const void* min_vals, const void* max_vals, int64_t n,
                           int32_t stats_dtype, int32_t fmt, int32_t num_bits, int32_t symmetric,
                           int32_t scale_mode, const float* global_scale, void* scale_out,
                           int32_t scale_out_dtype, int8_t* zero_point_out,
                           uint8_t* scale_code_out, void* stream);

/* ---- a17/a18: quantise, fake-quantise, pack --------------------------------
 * Replaces CT fake_quantize / quantize (call sites gptq_quantize.py:184-225,
 * observers/mse_quant.py:275-280, modifiers/quantization/calibration.py:178-183)
 * and the compressors' pack step (pack_to_int32, pack_fp4_to_uint8, fp8 storage;
 * call site transformers/compression/compressed_tensors_utils.py:134-138).
 * The scale of element (r,c) is scale[(r/row_div)*scale_row_stride +
 * (g_idx ? g_idx[c] : c/col_div)]; with global_scale the effective scale is
 * float(scale)/global_scale[0].
 *   LLMC_OUT_FAKEQUANT: dequantised values, out_dtype, ldo in elements
 *   LLMC_OUT_CODES    : one byte per element (int8 code | e4m3 byte | e2m1 nibble)
 *   LLMC_OUT_PACKED   : int -> int32 words, 32/num_bits offset-binary fields per
 *                       word, field j at bit j*num_bits (ldo in words);
 *                       fp4 -> uint8, even column in the low nibble (ldo in bytes);
 *                       fp8 -> e4m3 bytes (ldo in bytes)
 */
enum { LLMC_OUT_FAKEQUANT = 0, LLMC_OUT_CODES = 1, LLMC_OUT_PACKED = 2 };
int llmc_quantize(const void* x, int32_t x_dtype, int64_t R, int64_t K, int64_t ldx,
                  const void* scale, int32_t scale_dtype, const int8_t* zero_point,
                  const int32_t* g_idx, const float* global_scale, int32_t fmt, int32_t num_bits,
                  int64_t row_div, int64_t scale_row_stride, int64_t col_div, int32_t out_mode,
                  void* out, int32_t out_dtype, int64_t ldo, void* stream);

/* Dynamic per-token quantisation (CT compute_dynamic_scales_and_zp + fake_quantize,
 * strategy "token", reached through forward_quantize, calibration.py:178-183):
 * per row absmax -> scale = absmax/(range/2) in the row dtype -> quantise.
 * out_mode FAKEQUANT (row dtype) or CODES (bytes). scale_out: [N] in the row dtype. */
int llmc_dynamic_per_token_quantize(const void* x, int32_t x_dtype, int64_t N, int64_t K,
                                    int64_t ldx, int32_t fmt, int32_t num_bits, int32_t out_mode,
                                    void* out, int64_t ldo, void* scale_out, void* stream);

/* ---- a4-a7: damped Cholesky chain --------------------------------------------
 * Replaces, in quantize_weight (gptq_quantize.py:107-108,144-164, with the
 * H/num_samples of modifiers/gptq/base.py:336 folded in):
 *     H = H / divisor; [H = H[perm][:,perm]]; dead = diag(H)==0; H[dead,dead] = 1;
 *     H += percdamp*mean(diag H) * I; H = cholesky(H); H = cholesky_inverse(H);
 *     Hinv = cholesky(H, upper=True)
 * H is overwritten by the upper factor U (U^T U = H^-1, zeros below the diagonal).
 * dead_out[K] (may be NULL) flags the zero-diagonal columns in permuted order.
 * *info_out (device int, may be NULL) = 0, or the 1-based index of the first
 * non-positive pivot; in that case H becomes the identity, which is the
 * reference's round-to-nearest fallback on _LinAlgError (gptq_quantize.py:157-164).
 * perm may be NULL.  workspace must be 256-byte aligned.
 *
 * form selects what H holds afterwards.  LLMC_FACTOR_INVERSE: U as above.  LLMC_FACTOR_GROUPS (K a multiple of
 * 128): inside every 512-column diagonal block the same U (a diagonal block of the inverse of a triangular matrix
 * is the inverse of its diagonal block); outside those blocks the upper Cholesky factor V of the damped H itself
 * (V V^T = H, V = U^-1), i.e. the chain stops before the triangular inverse is carried across blocks, which is a
 * third of its arithmetic.  The blocks are aligned to the last column: [K-512, K), [K-1024, K-512), ..., and a
 * first block of the K % 512 columns that are left.  llmc_gptq_quantize takes either form and gives the same
 * result up to fp32 rounding, and so does llmc_sparsegpt_sparsify (its block size must then be 128).
 * llmc_gptq_factor_form(K, blocksize) is the form the library prefers for a quantize_weight / sparsify_weight
 * call.
 */
enum {
  LLMC_FACTOR_INVERSE = 0,
  LLMC_FACTOR_GROUPS = 1,
  LLMC_FACTOR_GROUP_WIDTH = 512
};
int32_t llmc_gptq_factor_form(int64_t K, int32_t blocksize);
int64_t llmc_gptq_hinv_workspace_bytes(int64_t K);
int llmc_gptq_hinv(float* H, int64_t ldh, int64_t K, const int32_t* perm, float divisor,
                   float percdamp, int32_t form, uint8_t* dead_out, void* workspace,
                   int64_t workspace_bytes, int32_t* info_out, void* stream);

/* Column order of GPTQ's activation ordering (gptq_quantize.py:131-140: argsort of diag(H), descending): for each of
 * the n Hessians (HOST array of n device pointers, fp32 [K, K], row stride ldh) the column numbers ordered by
 * descending diagonal entry, equal entries in ascending column order (the result of a stable sort; the reference's
 * unstable torch.argsort leaves the order of exact ties unspecified), NaN before every number.  out: device int64
 * [n, K].  K <= 16384. */
int llmc_diag_argsort_desc(const float* const* H, int64_t ldh, int32_t n, int64_t K, int64_t* out, void* stream);

/* Grouped form for many small problems of one width (the experts of an MoE layer): the chain of
 * llmc_gptq_hinv run once for all n problems in lock-step, every kernel carrying one more batch
 * dimension.  H (and perm, or NULL) are HOST arrays of n device pointers, divisors a HOST array of n
 * floats; dead_out is device [n, K] bytes (or NULL), U_out device [n, K, ldu] floats (the factors; the
 * Hessians themselves are left untouched), info_out device [n].  Results are bit-identical to n single
 * calls. */
int64_t llmc_gptq_hinv_grouped_workspace_bytes(int64_t n, int64_t K);
int llmc_gptq_hinv_grouped(const float* const* H, int64_t ldh, int32_t n, int64_t K,
                           const int32_t* const* perm, const float* divisors, float percdamp,
                           int32_t form, uint8_t* dead_out, float* U_out, int64_t ldu, void* workspace,
                           int64_t workspace_bytes, int32_t* info_out, void* stream);

/* ---- a8/a9: GPTQ block column loop ---------------------------------------------
 * Replaces the loop of quantize_weight (gptq_quantize.py:88-92,144-146,167-250):
 * W = float(weight)[:, perm], dead columns zeroed; per block of `blocksize`
 * columns, per column: q = fake_quantize(w), err = (w-q)/U[i,i],
 * W1[:, i:] -= err (x) U[i, i:]; per block W[:, i2:] -= Err1 @ U[i1:i2, i2:];
 * finally out_weight[:, perm[c]] = W[:, c] cast to w_dtype and
 * *loss_out = sum over rows and columns of (w-q)^2 / U[i,i]^2 / 2.
 * The scale of (row r, permuted column c) is
 *   scale[(r/row_div)*scale_row_stride + (g_idx ? g_idx[c] : 0)]
 * (per tensor: row_div >= R; per channel: row_div 1, stride 1; per group: stride K/g and
 * g_idx[c] = group of permuted column c; block strategy: row_div = block height).
 * blocksize above 128 runs as 128-wide blocks (same result up to fp32 summation order).
 *
 * form says what U holds (see llmc_gptq_hinv).  With LLMC_FACTOR_GROUPS (blocksize >= 128) the columns beyond a
 * 512-column group are not updated after the group; instead each group first takes what all earlier groups owe it,
 *     W[:, G] += ((W0 - Q)[:, :g0] @ V[:g0, G]) @ U[G, G]        (W0: the weights before the loop, Q: quantised),
 * which equals -Err[:, :g0] @ U[:g0, G] without ever forming U outside the diagonal blocks.  That form needs more
 * workspace (a second [R, K] fp32 matrix and the pieces of the product), hence the form argument of the size query.
 */
int64_t llmc_gptq_quantize_workspace_bytes(int64_t R, int64_t K, int32_t form);
int llmc_gptq_quantize(const void* weight, int32_t w_dtype, int64_t R, int64_t K, int64_t ldw,
                       const float* U, int64_t ldu, const int32_t* perm, const uint8_t* dead,
                       const void* scale, int32_t scale_dtype, const int8_t* zero_point,
                       const float* global_scale, const int32_t* g_idx, int64_t row_div,
                       int64_t scale_row_stride, int32_t fmt, int32_t num_bits, int32_t blocksize,
                       int32_t form, void* out_weight, int64_t ldo, float* loss_out, void* workspace,
                       int64_t workspace_bytes, void* stream);

/* Grouped form of llmc_gptq_quantize for n problems of one shape and scheme (the expert Linears of an MoE
 * layer) in lock-step.  weight, scale, zero_point, global_scale, g_idx and out_weight are HOST arrays of n
 * device pointers (zero_point / global_scale / g_idx may be NULL as in the single call); U is device
 * [n][K][ldu] with problem stride u_stride (as written by llmc_gptq_hinv_grouped), perm device [n, K] int32
 * or NULL, dead device [n, K] bytes or NULL, loss_out device [n].  Results are bit-identical to n single calls. */
int64_t llmc_gptq_quantize_grouped_workspace_bytes(int64_t n, int64_t R, int64_t K, int32_t form);
int llmc_gptq_quantize_grouped(const void* const* weight, int32_t w_dtype, int32_t n, int64_t R, int64_t K,
                               int64_t ldw, const float* U, int64_t ldu, int64_t u_stride,
                               const int32_t* perm, const uint8_t* dead, const void* const* scale,
                               int32_t scale_dtype, const int8_t* const* zero_point,
                               const float* const* global_scale, const int32_t* const* g_idx,
                               int64_t row_div, int64_t scale_row_stride, int32_t fmt, int32_t num_bits,
                               int32_t blocksize, int32_t form, void* const* out_weight, int64_t ldo,
                               float* loss_out, void* workspace, int64_t workspace_bytes, void* stream);

/* ---- fp32 product of the lazy trailing updates ----------------------------------------------------
 * Replaces the matmul of W[:, i2:] -= Err1.matmul(Hinv[i1:i2, i2:]) (gptq_quantize.py:245) and the products
 * inside torch.linalg.cholesky / cholesky_inverse of gptq_quantize.py:153-155:
 *     C[M,N] = alpha * A[M,Kc] * B' + beta * C,  B' = B[Kc,N] (trans_b = 0) or B[N,Kc]^T (trans_b = 1),
 * all row-major fp32.  Products whose shape is a whole number of 128- or 256-wide tiles run on the 16-bit
 * matrix cores with every operand split into three bf16 terms (six partial products, the dropped ones below
 * the rounding of an fp32 product); other shapes, and every shape with LLMC_SGEMM_FP32_MFMA, use the fp32
 * matrix instruction.  Structure flags are tile-granular promises about exact zeros in the operands.
 * Non-finite operands: the split form turns an infinite operand, or a finite one whose magnitude rounds to infinity
 * in bf16 (above 3.39e38), into NaN (the remainder of the split is inf - inf), where the fp32 instruction gives an
 * infinity; results for finite operands below that bound are as accurate as stated above.  Pass
 * LLMC_SGEMM_FP32_MFMA when infinities must propagate as such. */
enum {
  LLMC_SGEMM_C_LOWER = 1,      /* only tiles touching the lower triangle of C are computed and written     */
  LLMC_SGEMM_A_LOWER_TRI = 2,  /* A[m,k] == 0 for k > m                                                    */
  LLMC_SGEMM_B_LOWER_TRI = 4,  /* B'[k,n] == 0 for k < n                                                   */
  LLMC_SGEMM_FP32_MFMA = 8     /* never split: v_mfma_f32_32x32x2_f32 only                                 */
};
int llmc_sgemm(const float* A, int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc, int64_t M,
               int64_t N, int64_t Kc, float alpha, float beta, int32_t trans_b, int32_t flags, void* stream);

/* ---- SparseGPT (a "next" row: the same Hessian / Cholesky / column-loop skeleton) ----------
 * Replaces the loop of sparsify_weight (src/llmcompressor/modifiers/pruning/sparsegpt/
 * sgpt_sparsify.py:125-213); the factor U comes from llmc_gptq_hinv (:97-118 are the same
 * dead-column / damping / Cholesky chain; pass divisor = number of samples to turn the summed
 * Hessian into the reference's running average of :48-53).
 *   prune_n == 0: unstructured.  Per block of `blocksize` columns the elements whose saliency
 *     w^2 / U[c][c]^2 is <= the int(R * count * sparsity)-th smallest of the block are zeroed
 *     (:141-156; an exact radix selection replaces the sort).  32 <= blocksize <= 128.
 *   prune_n : prune_m (m in {2, 4, 8}, blocksize % m == 0): when the column loop reaches a group
 *     of m columns, the n least salient of its current values are zeroed (:165-176).
 *   preserve_sparsity_mask: weights that are zero on entry stay zero, are not compensated by the
 *     trailing updates (:193-198) and count towards the target (:143-151).  The caller checks
 *     that the existing sparsity does not exceed the target (:127-133 raises).
 * out_weight receives the pruned weight in w_dtype, *loss_out the sum of (w - q)^2 / d^2 / 2. */
int64_t llmc_sparsegpt_workspace_bytes(int64_t R, int64_t K, int32_t form);
int llmc_sparsegpt_sparsify(const void* weight, int32_t w_dtype, int64_t R, int64_t K, int64_t ldw,
                            const float* U, int64_t ldu, const uint8_t* dead, double sparsity,
                            int32_t prune_n, int32_t prune_m, int32_t blocksize, int32_t form,
                            int32_t preserve_sparsity_mask, void* out_weight, int64_t ldo,
                            float* loss_out, void* workspace, int64_t workspace_bytes, void* stream);

/* Grouped Linear of the experts of an MoE block (the reference's loop: modeling/moe/linear_experts.py:235-268
 * calls each expert's gate_proj / up_proj / down_proj on its own routed rows, one F.linear each):
 *   y[r, s*N + n] = sum_k x[r, k] * W_{s,e(r)}[n, k]   for every routed row r, bf16 in, fp32 accumulation,
 * one rounding to bf16.  x [rows, K] (row stride ldx) holds the routed rows expert after expert; `tiles`
 * (device, int32 [ntiles][4], 16-byte aligned) lists runs of at most 128 rows of one expert as
 * {expert, first row, rows, shift}: the results of the tile's rows go to the rows first row + shift .. of y
 * (0: y has x's row numbering; another value lets several experts read the same rows of x and write apart, the
 * reference's calibrate_all_experts case, where every expert is called on every token); w (device array of splits * experts pointers, 16-byte aligned each) holds the
 * [N, K] weights (row stride ldw) of split s and expert e at w[s * experts + e]; splits that share their input
 * (gate and up) write side by side into y (row stride ldy >= splits * N).  N % 128 == 0, K % 64 == 0,
 * dtype LLMC_BF16.  Rows no tile names are not written; the caller sizes y for the largest row a tile names.  The sum over k runs in a different order than a
 * library GEMM's, so results agree with F.linear to the last bf16 digit, not bit for bit: use it where hooks do
 * not need the exact inputs of the reference's forward (the propagation pass of a sequential pipeline). */
int llmc_grouped_linear(const void* x, int32_t dtype, int64_t ldx, const void* const* w, int64_t ldw,
                        int32_t experts, int32_t splits, void* y, int64_t ldy, const int32_t* tiles,
                        int32_t ntiles, int64_t N, int64_t K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMC_AMD_H */
