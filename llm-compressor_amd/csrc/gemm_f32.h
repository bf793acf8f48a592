// Internal fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32), used for the
// trailing-matrix updates of the Cholesky chain and of the GPTQ block loop.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

struct GemmF32 {
  // C[M,N] = alpha * A' * B' + beta * C,   all row-major
  //   trans_b = 0: B' = B,  B stored [Kc,N];   trans_b = 1: B' = B^T, B stored [N,Kc]
  //   trans_a = 0: A' = A,  A stored [M,Kc];   trans_a = 1: A' = A^T, A stored [Kc,M] (only with
  //   trans_b = 0 and without the a_lower_tri hint)
  const float* A;
  int64_t lda;
  const float* B;
  int64_t ldb;
  float* C;
  int64_t ldc;
  int M, N, Kc;
  float alpha, beta;
  int trans_b;
  int trans_a;
  // structure hints (tile-granular; operands must hold exact zeros where the structure says so)
  int c_lower;      // only tiles that touch the lower triangle of C are computed
  int a_lower_tri;  // A[m,k] = 0 for k > m : contraction stops at the tile's last row
  int b_lower_tri;  // B'[k,n] = 0 for k < n : contraction starts at the tile's first column
  // batching over blockIdx.z
  int batch;
  int64_t stride_a, stride_b, stride_c;
  // contraction length of the last block of the batch when it differs from Kc (a contraction cut into
  // `batch` pieces whose last one is shorter); 0 = Kc like the others
  int kc_last;
  // second batch level (independent problems, each with `batch` blocks): blockIdx.z = b + batch * b2;
  // 0 or 1 = none
  int batch2;
  int64_t stride2_a, stride2_b, stride2_c;
};

// enqueue on `st`; returns 0 or 1000 + hipError_t
int llmc_gemm_f32(const GemmF32& g, hipStream_t st);

// The same product on the 16-bit matrix cores (every operand split into three bf16 planes, six partial
// products; see gemm_x3.hip): taken when the shape is a whole number of 128- or 256-wide tiles and big enough
// to fill the chip.  Returns -1 when the product is left to the fp32 matrix instruction.
int llmc_gemm_x3(const GemmF32& g, hipStream_t st);
// 0 = never use the split product, 1 = whenever it applies (default)
void llmc_gemm_x3_set_mode(int mode);
