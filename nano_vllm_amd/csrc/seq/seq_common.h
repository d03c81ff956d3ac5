// Shared helpers of libnvl_seq.so (gfx950 only: 64-wide wavefronts are assumed throughout).
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include "../../../include/nvl_seq.h"

typedef __bf16 bf16_t;

void nvs_set_error(const char* fmt, ...);
int nvs_check_launch(const char* what);

#define NVS_REQUIRE(cond, ...)       \
  do {                               \
    if (!(cond)) {                   \
      nvs_set_error(__VA_ARGS__);    \
      return NVS_EINVAL;             \
    }                                \
  } while (0)

// element access in 32-bit whatever the storage type
__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t* p) { return (float)*p; }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t* p, float v) { *p = (bf16_t)v; }   // round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// sum over a workgroup of up to 1024 threads; `red` is LDS for 16 floats; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();                       // `red` may still be read from a previous call
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

#define NVS_DISPATCH(dtype, ...)                       \
  do {                                                 \
    if ((dtype) == NVS_BF16) {                         \
      typedef bf16_t T;                                \
      __VA_ARGS__;                                     \
    } else {                                           \
      typedef float T;                                 \
      __VA_ARGS__;                                     \
    }                                                  \
  } while (0)
