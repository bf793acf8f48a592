// Shared device helpers for the gfx950 kernels (64-wide wavefronts).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmc_amd.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define LLMC_CHECK_ARG(cond, n) \
  do {                          \
    if (!(cond)) return -(n);   \
  } while (0)

// hipGetLastError() after a launch: >0 return = 1000 + hipError_t
#define LLMC_LAUNCH_STATUS()                      \
  do {                                            \
    hipError_t e__ = hipGetLastError();           \
    if (e__ != hipSuccess) return 1000 + (int)e__; \
  } while (0)

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet), same as torch's cast
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// value of f after a round trip through bf16
__device__ __forceinline__ float round_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // RNE
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// load one element of a {bf16,f16,f32} buffer as fp32
template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i) {
  if (DT == LLMC_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  if (DT == LLMC_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// round an fp32 value to element type DT and return it as fp32
template <int DT>
__device__ __forceinline__ float round_to(float f) {
  if (DT == LLMC_BF16) return round_bf16(f);
  if (DT == LLMC_F16) return (float)(_Float16)f;
  return f;
}

template <int DT>
__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float f) {
  if (DT == LLMC_BF16)
    ((uint16_t*)p)[i] = f32_to_bf16_bits(f);
  else if (DT == LLMC_F16)
    ((uint16_t*)p)[i] = f32_to_f16_bits(f);
  else
    ((float*)p)[i] = f;
}

__host__ __device__ __forceinline__ int dtype_size(int dt) { return dt == LLMC_F32 ? 4 : 2; }

// wave-wide reductions over 64 lanes
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Host tables of per-problem pointers reach the device as kernel arguments (copied when the launch is
// enqueued), 32 entries per launch: the host array may be released as soon as the call returns, nothing
// depends on how the runtime stages copies from pageable memory, and the upload is an ordinary kernel
// node for a caller that captures the stream.
template <typename T>
struct ItemChunk {
  T v[32];
};
template <typename T>
__global__ void upload_items_kernel(ItemChunk<T> c, int count, T* __restrict__ dst) {
  const int i = threadIdx.x;
  if (i < count) dst[i] = c.v[i];
}
template <typename T>
inline int upload_items(const T* host, int n, T* dev, hipStream_t st) {
  static_assert(sizeof(ItemChunk<T>) <= 3072, "chunk must fit the kernel argument buffer");
  for (int at = 0; at < n; at += 32) {
    ItemChunk<T> c = {};
    const int count = n - at < 32 ? n - at : 32;
    for (int i = 0; i < count; ++i) c.v[i] = host[at + i];
    hipLaunchKernelGGL((upload_items_kernel<T>), dim3(1), dim3(32), 0, st, c, count, dev + at);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return 1000 + (int)e;
  }
  return 0;
}
