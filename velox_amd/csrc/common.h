// Shared helpers of the gfx950 kernels: element types, conversions, reductions, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Element type codes used across the C interface.
#define VELOX_F32 0
#define VELOX_BF16 1

typedef __bf16 bf16_t;
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));

#define VELOX_WAVE 64

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ short bf16_bits(float v) { return __builtin_bit_cast(short, (bf16_t)v); }

// Sum over the 64 lanes of a wave; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, VELOX_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, VELOX_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds one float per wave (16 at most).
// Every thread gets the result.  The order of the additions is fixed, so the result does not
// depend on anything but the values.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (VELOX_WAVE - 1);
  const int wave = threadIdx.x / VELOX_WAVE;
  const int waves = (blockDim.x + VELOX_WAVE - 1) / VELOX_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

#define VELOX_RETURN_LAUNCH_STATUS() return (int)hipGetLastError()
