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

// 16 bytes per lane from global memory straight into LDS: lane l's piece lands at dst + 16 l, so one instruction fills a
// contiguous kilobyte.  `dst` must be the same for the whole wave.  Written as assembly on purpose: of a load that the
// compiler knows to write LDS it assumes that any later LDS read may touch what is still in flight, and waits for ALL
// outstanding loads before the first read, which undoes a load issued ahead into another buffer.  The caller orders
// things itself: `wait_for_loads<N>()` (at most N of the wave's loads still in flight) and a barrier before the reads.
__device__ __forceinline__ void load_to_lds_16(const void* src, void* dst) {
  const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(at), "v"(src) : "memory", "m0");
}
// The same with the address as a base that is the same for the whole wave (it travels in scalar registers) plus 32 bits of
// byte offset per lane: no 64-bit vector arithmetic per load.
__device__ __forceinline__ void load_to_lds_16(const void* wave_base, uint32_t lane_bytes, void* dst) {
  const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(at), "v"(lane_bytes), "s"(wave_base) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_for_loads() {
  static_assert(N >= 0 && N < 64, "the counter of loads in flight has six bits");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

#define VELOX_RETURN_LAUNCH_STATUS() return (int)hipGetLastError()
