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
 * units.  Only the upper-triangular tiles are computed.  With
 * LLMC_HESSIAN_ASSUME_SYMMETRIC the mirrored lower tiles are stored from the
 * upper results (H must be bitwise symmetric on entry, which holds for a
 * buffer that started as zeros and was only ever updated by this call);
 * without it the lower tiles are read-modify-written too.
 */
enum { LLMC_HESSIAN_ASSUME_SYMMETRIC = 1 };
int llmc_hessian_accumulate(float* H, int64_t ldh, const void* X, int64_t ldx,
                            int64_t T, int64_t K, int32_t x_dtype, float alpha,
                            int32_t flags, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMC_AMD_H */
