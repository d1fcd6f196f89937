// Sampling kernels for gfx950: row argmax, the per-row sampler (temperature, top-k, top-p, exponential
// race with a counter-based generator) and the repetition / presence / frequency penalties.
// One workgroup per row; every reduction runs in a fixed order, so a row's result depends on that
// row alone.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

#define SAMPLE_THREADS 1024

struct Best { float value; int index; };

__device__ __forceinline__ Best better(Best a, Best b) {
  // larger value wins; equal values: the smaller index
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

__device__ __forceinline__ Best block_best(Best v, Best* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int waves = (blockDim.x + 63) / 64;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    Best other;
    other.value = __shfl_xor(v.value, offset, VELOX_WAVE);
    other.index = __shfl_xor(v.index, offset, VELOX_WAVE);
    v = better(v, other);
  }
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  Best total = scratch[0];
  for (int w = 1; w < waves; ++w) total = better(total, scratch[w]);
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int waves = (blockDim.x + 63) / 64;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// the best of row[lo .. hi), indices counted from the start of the row
__device__ __forceinline__ Best best_of_range(const float* __restrict__ row, int lo, int hi, Best* scratch) {
  Best best{-INFINITY, 0x7fffffff};
  // 16-byte loads over the aligned middle of the range, single elements at its ends
  const float* start = row + lo;
  const int count = hi - lo;
  const int head = (int)((16 - ((uintptr_t)start & 15)) & 15) / 4;
  const int first = head < count ? head : count;
  const int quads = (count - first) / 4;
  for (int i = threadIdx.x; i < first; i += blockDim.x) best = better(best, Best{start[i], lo + i});
  const float4_t* body = reinterpret_cast<const float4_t*>(start + first);
  for (int q = threadIdx.x; q < quads; q += blockDim.x) {
    const float4_t v = body[q];
#pragma unroll
    for (int j = 0; j < 4; ++j) best = better(best, Best{v[j], lo + first + 4 * q + j});
  }
  for (int i = first + 4 * quads + threadIdx.x; i < count; i += blockDim.x) best = better(best, Best{start[i], lo + i});
  return block_best(best, scratch);
}

// One workgroup per (row, chunk of the vocabulary).  With one chunk the index goes straight to `out`; with several, each
// chunk's best goes to `partial[row][chunk]` and argmax_merge_kernel picks among them (few rows alone would leave most
// of the GPU idle while 600 KB per row are read).
__global__ void __launch_bounds__(SAMPLE_THREADS) argmax_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                               Best* __restrict__ partial, int vocab, int chunk) {
  __shared__ Best scratch[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  const int lo = blockIdx.y * chunk;
  const int hi = lo + chunk < vocab ? lo + chunk : vocab;
  const Best best = best_of_range(row, lo, hi, scratch);
  if (threadIdx.x != 0) return;
  if (gridDim.y == 1) out[blockIdx.x] = best.index;
  else partial[blockIdx.x * gridDim.y + blockIdx.y] = best;
}

__global__ void __launch_bounds__(64) argmax_merge_kernel(const Best* __restrict__ partial, int* __restrict__ out, int chunks) {
  Best best{-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < chunks; c += 64) best = better(best, partial[blockIdx.x * chunks + c]);
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    Best other;
    other.value = __shfl_xor(best.value, offset, VELOX_WAVE);
    other.index = __shfl_xor(best.index, offset, VELOX_WAVE);
    best = better(best, other);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best.index;
}

// partial: room for rows * chunks (value, index) pairs of 8 bytes, used when chunks > 1.
extern "C" int velox_argmax(const float* logits, int* out, void* partial, int rows, int vocab, int chunks, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (chunks < 1 || (chunks > 1 && partial == nullptr)) return -1;
  const int chunk = (vocab + chunks - 1) / chunks;
  argmax_kernel<<<dim3(rows, chunks), SAMPLE_THREADS, 0, stream>>>(logits, out, (Best*)partial, vocab, chunk);
  if (chunks > 1) argmax_merge_kernel<<<rows, 64, 0, stream>>>((const Best*)partial, out, chunks);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---- the entry point that allocates nothing (declared in no_alloc.h) ----------------------------------------------
// The chunks' best pairs of velox_argmax_static.  In host code this name is only a stand-in for the symbol: each GPU
// holds its own copy at its own address, which hipGetSymbolAddress gives with that GPU current; host code passes
// that address on, never the name.
static __device__ __align__(256) unsigned char argmax_static_scratch[VELOX_ARGMAX_STATIC_BYTES];

#define VELOX_MAX_DEVICES 64
static void* argmax_scratch_of_device[VELOX_MAX_DEVICES];  // the address of each GPU's copy, looked up once
static std::mutex argmax_scratch_lock;

static int argmax_scratch_of_current_device(void** address) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return (int)status;
  if (device < 0 || device >= VELOX_MAX_DEVICES) return VELOX_NO_ALLOC_NO_SCRATCH;
  std::lock_guard<std::mutex> guard(argmax_scratch_lock);
  if (argmax_scratch_of_device[device] == nullptr) {
    void* found = nullptr;
    status = hipGetSymbolAddress(&found, HIP_SYMBOL(argmax_static_scratch));
    if (status != hipSuccess) return (int)status;
    if (found == nullptr) return VELOX_NO_ALLOC_NO_SCRATCH;
    argmax_scratch_of_device[device] = found;
  }
  *address = argmax_scratch_of_device[device];
  return 0;
}

extern "C" int velox_argmax_static_init(void) {
  void* address = nullptr;
  return argmax_scratch_of_current_device(&address);
}

extern "C" int velox_argmax_static(const float* logits, int* out, int rows, int vocab, int chunks, hipStream_t stream) {
  if (rows < 0 || vocab < 1 || chunks < 1 || chunks > vocab || logits == nullptr || out == nullptr) return VELOX_NO_ALLOC_BAD_ARGUMENT;
  if (rows == 0) return 0;
  if (rows > 65535 || chunks > 65535 || (long long)rows * chunks > VELOX_ARGMAX_STATIC_MAX_PAIRS) return VELOX_NO_ALLOC_TOO_LARGE;
  void* scratch = nullptr;
  const int found = argmax_scratch_of_current_device(&scratch);
  if (found != 0) return found;
  const int chunk = (vocab + chunks - 1) / chunks;
  // every pair that the merge reads is written by this launch first: what an earlier call left is never read
  argmax_kernel<<<dim3(rows, chunks), SAMPLE_THREADS, 0, stream>>>(logits, out, (Best*)scratch, vocab, chunk);
  if (chunks > 1) argmax_merge_kernel<<<rows, 64, 0, stream>>>((const Best*)scratch, out, chunks);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" const char* velox_no_alloc_error_text(int code) {
  switch (code) {
    case 0: return "success";
    case VELOX_NO_ALLOC_BAD_ARGUMENT: return "bad argument: rows >= 0, vocab >= 1, 1 <= chunks <= vocab and non-null pointers are required";
    case VELOX_NO_ALLOC_TOO_LARGE: return "rows * chunks exceeds VELOX_ARGMAX_STATIC_MAX_PAIRS (65536), the size of the static scratch array";
    case VELOX_NO_ALLOC_NO_SCRATCH: return "the static scratch array of this GPU could not be found";
    default: return hipGetErrorString((hipError_t)code);
  }
}

// Philox 4x32 with 10 rounds.
__device__ __forceinline__ void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// order-preserving map from float to unsigned
__device__ __forceinline__ uint32_t sort_key(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

// options per row, int32[6]: temperature (float bits), top_p (float bits), top_k, seed low 31 bits, seed high 31 bits, counter
//   temperature == 0: argmax.
//   otherwise x = logit / max(T, 1e-5); p = softmax(x); token i is kept iff fewer than top_k tokens have a larger x
//   (top_k > 0) and the tokens with a larger x hold less than top_p of the probability; among the kept tokens the
//   draw is argmax(x - max - log(e)), e = max(-log(u), 1e-10), u uniform from Philox(key = seed, counter = (i / 4, counter)).
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_kernel(const float* __restrict__ logits, const int* __restrict__ options,
                                                                int* __restrict__ out, int vocab) {
  __shared__ Best best_scratch[16];
  __shared__ float scratch[16];
  __shared__ float scratch2[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  const int* opt = options + (size_t)blockIdx.x * 6;
  const float temperature = __int_as_float(opt[0]);
  const float top_p = __int_as_float(opt[1]);
  const int top_k = opt[2];
  const uint32_t seed_lo = (uint32_t)opt[3], seed_hi = (uint32_t)opt[4], counter = (uint32_t)opt[5];
  const int tid = threadIdx.x;

  if (temperature == 0.f) {
    Best best{-INFINITY, 0x7fffffff};
    for (int i = tid; i < vocab; i += blockDim.x) {
      const float v = row[i];
      if (v > best.value || best.index == 0x7fffffff) best = Best{v, i};
    }
    best = block_best(best, best_scratch);
    if (tid == 0) out[blockIdx.x] = best.index;
    return;
  }
  const float inv_t = 1.f / fmaxf(temperature, 1e-5f);
  float mx = -INFINITY;
  for (int i = tid; i < vocab; i += blockDim.x) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, scratch);
  float z = 0.f;
  for (int i = tid; i < vocab; i += blockDim.x) z += expf(row[i] * inv_t - mx);
  z = block_sum(z, scratch);

  // smallest key whose tokens are kept
  uint32_t threshold = 0u;
  const bool filter = (top_k > 0 && top_k < vocab) || top_p < 1.f;
  if (filter) {
    const float mass_limit = top_p * z;
    uint32_t lo = 0u, hi = 0xffffffffu;  // predicate(hi) holds (nothing is larger); find the smallest key where it holds
    while (lo < hi) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      float count = 0.f, mass = 0.f;
      for (int i = tid; i < vocab; i += blockDim.x) {
        const float x = row[i] * inv_t;
        if (sort_key(x) > mid) { count += 1.f; mass += expf(x - mx); }
      }
      count = block_sum(count, scratch);
      mass = block_sum(mass, scratch2);
      const bool ok = (top_k <= 0 || count < (float)top_k) && (mass < mass_limit);
      if (ok) hi = mid; else lo = mid + 1u;
    }
    threshold = lo;
  }

  Best best{-INFINITY, 0x7fffffff};
  const int quads = (vocab + 3) / 4;
  for (int q = tid; q < quads; q += blockDim.x) {
    uint32_t bits[4];
    philox4x32((uint32_t)q, counter, 0u, 0u, seed_lo, seed_hi, bits);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 4 * q + e;
      if (i >= vocab) break;
      const float x = row[i] * inv_t;
      if (filter && sort_key(x) < threshold) continue;
      const float u = ((float)(bits[e] >> 8) + 0.5f) * (1.0f / 16777216.0f);
      const float noise = fmaxf(-logf(u), 1e-10f);
      const float score = (x - mx) - logf(noise);
      if (score > best.value || best.index == 0x7fffffff) best = Best{score, i};
    }
  }
  best = block_best(best, best_scratch);
  if (tid == 0) out[blockIdx.x] = best.index;
}

extern "C" int velox_sample(const float* logits, const int* options, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, options, out, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}

// Penalties over the tokens a request has seen (prompt and output), each distinct token once:
//   v = logit - frequency * count;  v = v > 0 ? v / repetition : v * repetition;  v -= presence
__global__ void penalties_kernel(float* __restrict__ logits, const int* __restrict__ tokens, const int* __restrict__ lengths,
                                 const float* __restrict__ coeffs, int vocab, int width) {
  const int r = blockIdx.x;
  const int n = lengths[r];
  const int* seen = tokens + (size_t)r * width;
  const float repetition = coeffs[3 * r], presence = coeffs[3 * r + 1], frequency = coeffs[3 * r + 2];
  float* row = logits + (size_t)r * vocab;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int token = seen[i];
    if (token < 0 || token >= vocab) continue;
    int count = 0;
    bool first = true;
    for (int j = 0; j < n; ++j) {
      const bool same = seen[j] == token;
      count += same ? 1 : 0;
      if (same && j < i) first = false;
    }
    if (!first) continue;
    float v = row[token] - frequency * (float)count;
    v = v > 0.f ? v / repetition : v * repetition;
    row[token] = v - presence;
  }
}

extern "C" int velox_apply_penalties(float* logits, const int* tokens, const int* lengths, const float* coeffs, int rows, int vocab,
                                     int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  penalties_kernel<<<rows, 256, 0, stream>>>(logits, tokens, lengths, coeffs, vocab, width);
  VELOX_RETURN_LAUNCH_STATUS();
}
