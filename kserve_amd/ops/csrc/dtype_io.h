// Element load/store helpers for kernels instantiated for both activation
// dtypes: `short` carries bf16 bits (the convention of common.h), `float`
// is true fp32. All arithmetic happens in fp32 after the load.
#pragma once

#include "common.h"

template <typename T>
__device__ __forceinline__ float ld_f32(const T* p, long i);
template <>
__device__ __forceinline__ float ld_f32<float>(const float* p, long i) {
  return p[i];
}
template <>
__device__ __forceinline__ float ld_f32<short>(const short* p, long i) {
  return bf16_bits_to_float(p[i]);
}

template <typename T>
__device__ __forceinline__ void st_f32(T* p, long i, float v);
template <>
__device__ __forceinline__ void st_f32<float>(float* p, long i, float v) {
  p[i] = v;
}
template <>
__device__ __forceinline__ void st_f32<short>(short* p, long i, float v) {
  p[i] = float_to_bf16_bits(v);
}

// block-wide sum for blockDim.x == 64 * NWAVES; `scratch` holds NWAVES floats
// and may be reused after the call returns (trailing barrier).
template <int NWAVES>
__device__ __forceinline__ float block_sum_sync(float v, float* scratch) {
  float r = block_reduce_sum<NWAVES>(v, scratch);
  __syncthreads();
  return r;
}
