// Probes of what the card delivers, to set measured step times against: a streaming read of device memory, a loop of
// independent bfloat16 matrix instructions, and a barrier across the workgroups of a resident grid.  None is on the
// path of a model step.
#include "common.h"

typedef __bf16 probe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float probe_float16_t __attribute__((ext_vector_type(16)));
typedef unsigned int probe_uint4_t __attribute__((ext_vector_type(4)));

// Every thread reads 16-byte pieces with a grid stride, four in flight, and adds them up; the sums are stored only
// where they are "impossible" values, so that the loads stay and the stores cost nothing.
__global__ __launch_bounds__(256) void probe_read_kernel(const probe_uint4_t* __restrict__ data, long long vectors, unsigned int* __restrict__ sink) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned int sum = 0;
  for (; i + 3 * stride < vectors; i += 4 * stride) {
    const probe_uint4_t a = __builtin_nontemporal_load(data + i);
    const probe_uint4_t b = __builtin_nontemporal_load(data + i + stride);
    const probe_uint4_t c = __builtin_nontemporal_load(data + i + 2 * stride);
    const probe_uint4_t d = __builtin_nontemporal_load(data + i + 3 * stride);
    sum += (a.x ^ a.y ^ a.z ^ a.w) + (b.x ^ b.y ^ b.z ^ b.w) + (c.x ^ c.y ^ c.z ^ c.w) + (d.x ^ d.y ^ d.z ^ d.w);
  }
  for (; i < vectors; i += stride) {
    const probe_uint4_t a = __builtin_nontemporal_load(data + i);
    sum += a.x ^ a.y ^ a.z ^ a.w;
  }
  if (sum == 0x9e3779b9u) sink[0] = sum;
}

// bytes must be a multiple of 16 and data 16-byte aligned; `sink` is one 32-bit word.
extern "C" int velox_probe_read(const void* data, long long bytes, void* sink, int blocks, hipStream_t stream) {
  if (bytes <= 0 || bytes % 16 != 0 || blocks <= 0) return (int)hipErrorInvalidValue;
  probe_read_kernel<<<blocks, 256, 0, stream>>>((const probe_uint4_t*)data, bytes / 16, (unsigned int*)sink);
  VELOX_RETURN_LAUNCH_STATUS();
}

// Every wave issues `iterations` rounds of four independent 32x32x16 bfloat16 matrix instructions (2*32*32*16 flops
// each) on operands made from its lane number; the accumulators are stored where they are not finite.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iterations, float* __restrict__ sink) {
  probe_bf16x8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(1.0f / (float)(threadIdx.x + i + 1));
    b[i] = (__bf16)(1.0f / (float)(threadIdx.x + 2 * i + 3));
  }
  probe_float16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iterations; ++it) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  float total = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) total += c0[i] + c1[i] + c2[i] + c3[i];
  if (!(total == total) || total < 0.0f) sink[0] = total;
}

// Flops of a launch: blocks * 4 waves * iterations * 4 * 32768.
extern "C" int velox_probe_mfma(int blocks, int iterations, void* sink, hipStream_t stream) {
  if (blocks <= 0 || iterations <= 0) return (int)hipErrorInvalidValue;
  probe_mfma_kernel<<<blocks, 256, 0, stream>>>(iterations, (float*)sink);
  VELOX_RETURN_LAUNCH_STATUS();
}

// `rounds` barriers in a row across all workgroups of a grid that is resident as a whole (at most one workgroup per
// compute unit is asked for): the price of replacing a kernel boundary by a barrier inside one kernel.
// fenced = 0: a tree of relaxed agent-scope counters (16 groups a cache line apart add up their arrivals, the last of a
//   group adds to the master that everybody polls); data that crosses the barrier would have to move through agent-scope
//   atomic stores and loads, since nothing writes the caches back or invalidates them;
// fenced = 1: one counter with release on arrival and acquire on the poll and behind the barrier, which is what ordinary
//   stores and loads on either side need (the L2 write-back and the invalidation are the price).
// A workgroup that polls more than a bounded number of times gives up, raises `failed` and returns; whoever sees the flag
// returns too, so the kernel ends whatever happens.  counters: 17 * 32 words, zero before the launch.
constexpr int BARRIER_GROUPS = 16;
constexpr unsigned BARRIER_POLLS = 1u << 21;

__global__ __launch_bounds__(256) void probe_grid_barrier_kernel(unsigned* __restrict__ counters, int* __restrict__ failed, int rounds, int fenced) {
  const int g = blockIdx.x % BARRIER_GROUPS;
  const unsigned members = (gridDim.x - g + BARRIER_GROUPS - 1) / BARRIER_GROUPS;
  __shared__ int gave_up;
  for (int r = 0; r < rounds; ++r) {
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned polls = 0;
      int bad = 0;
      if (fenced) {
        __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        while (__hip_atomic_load(counters, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)(r + 1) * gridDim.x) {
          if (++polls > BARRIER_POLLS || __hip_atomic_load(failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { bad = 1; break; }
          __builtin_amdgcn_s_sleep(1);
        }
      } else {
        const unsigned before = __hip_atomic_fetch_add(counters + 32 * (1 + g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == members * (unsigned)(r + 1)) __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        while (__hip_atomic_load(counters, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)(r + 1) * BARRIER_GROUPS) {
          if (++polls > BARRIER_POLLS || __hip_atomic_load(failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { bad = 1; break; }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      if (bad) __hip_atomic_store(failed, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      gave_up = bad;
    }
    __syncthreads();
    if (gave_up) return;
    if (fenced) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
}

// blocks: at least BARRIER_GROUPS and at most the number of compute units (every workgroup has to be resident while the
// others wait for it).
extern "C" int velox_probe_grid_barrier(int blocks, int rounds, int fenced, void* counters, void* failed, hipStream_t stream) {
  int device = 0, units = 0;
  if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
    return (int)hipErrorInvalidValue;
  if (blocks < BARRIER_GROUPS || blocks > units || rounds <= 0) return (int)hipErrorInvalidValue;
  probe_grid_barrier_kernel<<<blocks, 256, 0, stream>>>((unsigned*)counters, (int*)failed, rounds, fenced);
  VELOX_RETURN_LAUNCH_STATUS();
}
