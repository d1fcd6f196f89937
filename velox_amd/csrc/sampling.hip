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

// ---- the threshold of top-k / top-p: a radix search over the ordered keys ------------------------------------------
// A token is kept iff fewer than top_k tokens have a larger x and the tokens with a larger x hold less than top_p of the
// probability.  Both conditions only get harder to meet as x falls, so the kept tokens are those whose key is at least
// some threshold.  The threshold is found digit by digit (11, 11 and 10 bits of the 32-bit key): one pass over the row
// fills, for the tokens that match the digits found so far, a table per value of the next digit (how many tokens, how
// much probability); a walk down the table from the largest digit finds the last digit whose largest member is still
// kept.  Probabilities are summed as 40-bit fixed-point integers, so a sum does not depend on the order in which the
// threads add and a row's threshold is the same in every run and every batch.
#define SELECT_BINS 2048
__device__ __forceinline__ unsigned long long fixed_point_mass(float p) { return (unsigned long long)(p * 1099511627776.f); }  // p in [0, 1], 2^40

struct Above { unsigned int count; unsigned long long mass; };

// Visits the elements of quads [q_lo, q_hi) of a row (quad q = elements 4q .. 4q + 3, those below vocab): f(index, value).
// Whole quads come as 16-byte loads when the row starts at a 16-byte boundary, four loads in flight per thread (with one
// load at a time a pass would take as many trips to the caches as a thread has quads).
template <typename F> __device__ __forceinline__ void for_each_in_quads(const float* __restrict__ row, int vocab, int q_lo, int q_hi, F f) {
  const bool aligned = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  int whole = aligned ? vocab / 4 : q_lo;  // quads below `whole` are complete and can be loaded as one
  whole = whole < q_hi ? whole : q_hi;
  whole = whole > q_lo ? whole : q_lo;
  const float4_t* body = reinterpret_cast<const float4_t*>(row);
  const int stride = blockDim.x;
  int q = q_lo + threadIdx.x;
  for (; q + 3 * stride < whole; q += 4 * stride) {
    const float4_t v0 = body[q], v1 = body[q + stride], v2 = body[q + 2 * stride], v3 = body[q + 3 * stride];
#pragma unroll
    for (int e = 0; e < 4; ++e) f(4 * q + e, v0[e]);
#pragma unroll
    for (int e = 0; e < 4; ++e) f(4 * (q + stride) + e, v1[e]);
#pragma unroll
    for (int e = 0; e < 4; ++e) f(4 * (q + 2 * stride) + e, v2[e]);
#pragma unroll
    for (int e = 0; e < 4; ++e) f(4 * (q + 3 * stride) + e, v3[e]);
  }
  for (; q < whole; q += stride) {
    const float4_t v = body[q];
#pragma unroll
    for (int e = 0; e < 4; ++e) f(4 * q + e, v[e]);
  }
  const int end = 4 * q_hi < vocab ? 4 * q_hi : vocab;
  for (int i = 4 * whole + threadIdx.x; i < end; i += stride) f(i, row[i]);
}

// One digit of the search.  `counts` and `masses` hold the table of this digit (SELECT_BINS entries, filled by the whole
// workgroup, barrier behind it); `above` is what lies above every token that matches the digits found so far.  Wave 0 walks
// the table; every thread gets the digit found, and `above` grows by what lies above that digit's tokens.
__device__ __forceinline__ int select_digit(const unsigned int* counts, const unsigned long long* masses, int bins, int top_k, bool use_mass,
                                            unsigned long long mass_limit, Above& above, int* found_digit, Above* found_above) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    const int per_lane = bins / 64;  // lane 0 holds the largest digits
    const int hi = bins - 1 - lane * per_lane;  // this lane's digits: hi, hi - 1, ..., hi - per_lane + 1
    unsigned int c = 0;
    unsigned long long m = 0;
    for (int j = 0; j < per_lane; ++j) { c += counts[hi - j]; m += masses[hi - j]; }
    // what lies above this lane's first digit: the sums of the lanes before it
    unsigned int c_before = c;
    unsigned long long m_before = m;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const unsigned int oc = __shfl_up(c_before, offset, VELOX_WAVE);
      const unsigned long long om = __shfl_up(m_before, offset, VELOX_WAVE);
      if (lane >= offset) { c_before += oc; m_before += om; }
    }
    c_before = above.count + c_before - c;
    m_before = above.mass + m_before - m;
    // the smallest digit of this lane whose members' top is still kept
    int lowest = 0x7fffffff;
    unsigned int lowest_c = 0;
    unsigned long long lowest_m = 0;
    for (int j = 0; j < per_lane; ++j) {
      const bool kept = (top_k <= 0 || c_before < (unsigned int)top_k) && (!use_mass || m_before < mass_limit);
      if (kept) { lowest = hi - j; lowest_c = c_before; lowest_m = m_before; }
      c_before += counts[hi - j];
      m_before += masses[hi - j];
    }
    // over the wave: kept digits form a run from the top, so the smallest one overall is the answer
    int best = lowest;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
      const int other = __shfl_xor(best, offset, VELOX_WAVE);
      best = other < best ? other : best;
    }
    if (best == lowest && lowest != 0x7fffffff) {
      *found_digit = lowest;
      found_above->count = lowest_c;
      found_above->mass = lowest_m;
    }
    if (best == 0x7fffffff && lane == 0) {  // (cannot happen: the largest digit's top is always kept)
      *found_digit = bins - 1;
      *found_above = above;
    }
  }
  __syncthreads();
  above = *found_above;
  return *found_digit;
}

// options per row, int32[6]: temperature (float bits), top_p (float bits), top_k, seed low 31 bits, seed high 31 bits, counter
//   temperature == 0: argmax.
//   otherwise x = logit / max(T, 1e-5); p = softmax(x); token i is kept iff fewer than top_k tokens have a larger x
//   (top_k > 0) and the tokens with a larger x hold less than top_p of the probability; among the kept tokens the
//   draw is argmax(x - max - log(e)), e = max(-log(u), 1e-10), u uniform from Philox(key = seed, counter = (i / 4, counter)).
// Passes over the row (from the caches: a row is a few hundred kilobytes): the maximum; with a filter, the sum and three
// digits of the threshold; the draw.  Either one workgroup walks the whole row (sample_kernel), or, when the rows are
// too few to fill the GPU that way, the row is cut into chunks of quads with a workgroup each and every pass is a
// kernel (the sample_chunk_* kernels): the same functions over a range of quads, the tables added up in global memory
// as integers, so both ways give the same token.
struct RowOptions {
  float temperature, top_p, inv_t;
  int top_k;
  uint32_t seed_lo, seed_hi, counter;
  bool use_mass, filter;
};

__device__ __forceinline__ RowOptions read_options(const int* __restrict__ opt, int vocab) {
  RowOptions o;
  o.temperature = __int_as_float(opt[0]);
  o.top_p = __int_as_float(opt[1]);
  o.top_k = opt[2];
  o.seed_lo = (uint32_t)opt[3];
  o.seed_hi = (uint32_t)opt[4];
  o.counter = (uint32_t)opt[5];
  o.inv_t = 1.f / fmaxf(o.temperature, 1e-5f);
  o.use_mass = o.top_p < 1.f;
  o.filter = (o.top_k > 0 && o.top_k < vocab) || o.use_mass;
  return o;
}

// digits of the threshold: bits 31..21, 20..10, 9..0
__device__ __forceinline__ int level_shift(int level) { return level == 0 ? 21 : level == 1 ? 10 : 0; }
__device__ __forceinline__ int level_bins(int level) { return level == 2 ? 1024 : 2048; }

// Adds the tokens of quads [q_lo, q_hi) that match the digits found so far (`prefix`) to the tables of digit `level`
// (`counts`, `masses`: LDS, cleared by the caller, barrier behind the clearing).  At level 0 every token's mass also goes
// into the returned sum.
__device__ __forceinline__ unsigned long long add_to_tables(const float* __restrict__ row, int vocab, int q_lo, int q_hi, const RowOptions& o, float mx,
                                                            int level, uint32_t prefix, unsigned int* counts, unsigned long long* masses) {
  const int shift = level_shift(level);
  const int bins = level_bins(level);
  const uint32_t known = level == 0 ? 0u : ~((1u << (shift + (level == 2 ? 10 : 11))) - 1u);  // mask of the digits found so far
  unsigned long long my_total = 0ull;
  const bool use_mass = o.use_mass;
  const float inv_t = o.inv_t;
  for_each_in_quads(row, vocab, q_lo, q_hi, [&](int, float v) {
    const float x = v * inv_t;
    const uint32_t key = sort_key(x);
    const bool match = (key & known) == prefix;
    if (level == 0 || match) {
      const unsigned long long mass = use_mass ? fixed_point_mass(expf(x - mx)) : 0ull;
      if (level == 0) my_total += mass;
      if (match) {
        const int digit = (int)((key >> shift) & (uint32_t)(bins - 1));
        atomicAdd(&counts[digit], 1u);
        if (use_mass && mass != 0ull) atomicAdd(&masses[digit], mass);
      }
    }
  });
  return my_total;
}

// The draw among the kept tokens of quads [q_lo, q_hi): this thread's best (score, index).
__device__ __forceinline__ Best draw_in_quads(const float* __restrict__ row, int vocab, int q_lo, int q_hi, const RowOptions& o, float mx, uint32_t threshold) {
  Best best{-INFINITY, 0x7fffffff};
  const bool aligned = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  const bool filter = o.filter;
  const float inv_t = o.inv_t;
  auto load_quad = [&](int q, float (&v)[4]) {
    if (aligned && 4 * q + 3 < vocab) {
      const float4_t loaded = *reinterpret_cast<const float4_t*>(row + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = loaded[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = 4 * q + e < vocab ? row[4 * q + e] : -INFINITY;
    }
  };
  constexpr int AHEAD = 4;  // quads in flight per thread
  for (int q0 = q_lo + threadIdx.x; q0 < q_hi; q0 += AHEAD * blockDim.x) {
    float ahead[AHEAD][4];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      const int qa = q0 + a * blockDim.x;
      load_quad(qa < q_hi ? qa : q0, ahead[a]);
    }
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      const int q = q0 + a * blockDim.x;
      if (q >= q_hi) break;
      float (&v)[4] = ahead[a];
      bool any = false;
#pragma unroll
      for (int e = 0; e < 4; ++e) any = any || (4 * q + e < vocab && !(filter && sort_key(v[e] * inv_t) < threshold));
      if (!any) continue;  // (the noise of a quad is only worked out where a token of it is kept)
      uint32_t bits[4];
      philox4x32((uint32_t)q, o.counter, 0u, 0u, o.seed_lo, o.seed_hi, bits);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * q + e;
        if (i >= vocab) break;
        const float x = v[e] * inv_t;
        if (filter && sort_key(x) < threshold) continue;
        const float u = ((float)(bits[e] >> 8) + 0.5f) * (1.0f / 16777216.0f);
        const float noise = fmaxf(-logf(u), 1e-10f);
        const float score = (x - mx) - logf(noise);
        if (score > best.value || best.index == 0x7fffffff) best = Best{score, i};
      }
    }
  }
  return best;
}

// One workgroup per row.
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_kernel(const float* __restrict__ logits, const int* __restrict__ options,
                                                                int* __restrict__ out, int vocab) {
  __shared__ Best best_scratch[16];
  __shared__ float scratch[16];
  __shared__ unsigned int counts[SELECT_BINS];
  __shared__ unsigned long long masses[SELECT_BINS];
  __shared__ unsigned long long total_mass;
  __shared__ int found_digit;
  __shared__ Above found_above;
  const float* row = logits + (size_t)blockIdx.x * vocab;
  const RowOptions o = read_options(options + (size_t)blockIdx.x * 6, vocab);
  const int tid = threadIdx.x;
  const int quads = (vocab + 3) / 4;

  if (o.temperature == 0.f) {
    Best best{-INFINITY, 0x7fffffff};
    for_each_in_quads(row, vocab, 0, quads, [&](int i, float v) { best = better(best, Best{v, i}); });
    best = block_best(best, best_scratch);
    if (tid == 0) out[blockIdx.x] = best.index;
    return;
  }
  float mx = -INFINITY;
  for_each_in_quads(row, vocab, 0, quads, [&](int, float v) { mx = fmaxf(mx, v * o.inv_t); });
  mx = block_max(mx, scratch);

  // smallest key whose tokens are kept
  uint32_t threshold = 0u;
  if (o.filter) {
    Above above{0u, 0ull};
    unsigned long long mass_limit = 0ull;
    uint32_t prefix = 0u;  // the digits found so far, in place
#pragma unroll 1
    for (int level = 0; level < 3; ++level) {
      const int bins = level_bins(level);
      for (int b = tid; b < bins; b += blockDim.x) { counts[b] = 0u; masses[b] = 0ull; }
      if (tid == 0 && level == 0) total_mass = 0ull;
      __syncthreads();
      const unsigned long long my_total = add_to_tables(row, vocab, 0, quads, o, mx, level, prefix, counts, masses);
      if (level == 0 && o.use_mass) atomicAdd(&total_mass, my_total);
      __syncthreads();
      // (at least 1: the largest token is kept however small top_p is)
      if (level == 0) mass_limit = max(1ull, (unsigned long long)((double)o.top_p * (double)total_mass));
      const int digit = select_digit(counts, masses, bins, o.top_k, o.use_mass, mass_limit, above, &found_digit, &found_above);
      prefix |= (uint32_t)digit << level_shift(level);
      __syncthreads();  // the tables are free again
    }
    threshold = prefix;
  }

  Best best = draw_in_quads(row, vocab, 0, quads, o, mx, threshold);
  best = block_best(best, best_scratch);
  if (tid == 0) out[blockIdx.x] = best.index;
}

extern "C" int velox_sample(const float* logits, const int* options, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, options, out, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---- a row cut into chunks: one kernel per pass ---------------------------------------------------------------------
// What the chunks of a row share, in global memory: each chunk's maximum and best pair, the tables of the three digits
// (cleared by the first kernel, added to with integer atomics by the kernels of the digits) and what the search has
// found so far.  Every workgroup of a kernel reads what the kernel before left and works out the digit before its own
// once more for itself (a walk down 2,048 entries); the workgroup of chunk 0 writes it down for the kernels after.
struct RowSearch {
  unsigned long long total_mass;
  unsigned long long above_mass[2];
  unsigned int above_count[2];
  unsigned int prefix[2];  // the digits found after level 0 and after level 1, in place
};

struct ChunkedScratch {
  float* chunk_max;            // [rows, chunks]
  Best* chunk_best;            // [rows, chunks]
  RowSearch* search;           // [rows]
  unsigned int* counts;        // [rows, 3, SELECT_BINS]
  unsigned long long* masses;  // [rows, 3, SELECT_BINS]
};

static size_t chunked_scratch_layout(int rows, int chunks, void* base, ChunkedScratch* scratch) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  size_t at = 0;
  char* p = (char*)base;
  auto take = [&](size_t bytes) { char* here = p + at; at += up(bytes); return here; };
  ChunkedScratch s;
  s.masses = (unsigned long long*)take((size_t)rows * 3 * SELECT_BINS * sizeof(unsigned long long));
  s.counts = (unsigned int*)take((size_t)rows * 3 * SELECT_BINS * sizeof(unsigned int));
  s.search = (RowSearch*)take((size_t)rows * sizeof(RowSearch));
  s.chunk_best = (Best*)take((size_t)rows * chunks * sizeof(Best));
  s.chunk_max = (float*)take((size_t)rows * chunks * sizeof(float));
  if (scratch != nullptr) *scratch = s;
  return at;
}

__device__ __forceinline__ void chunk_quads(int vocab, int& q_lo, int& q_hi) {
  const int quads = (vocab + 3) / 4;
  const int per_chunk = (quads + gridDim.y - 1) / gridDim.y;
  q_lo = blockIdx.y * per_chunk;
  q_hi = q_lo + per_chunk < quads ? q_lo + per_chunk : quads;
  if (q_lo > quads) q_lo = quads;
}

// pass 1: clears the row's tables, leaves the chunk's maximum (or, for a greedy row, its best pair)
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_chunk_max_kernel(const float* __restrict__ logits, const int* __restrict__ options,
                                                                          ChunkedScratch s, int vocab) {
  __shared__ Best best_scratch[16];
  __shared__ float scratch[16];
  const int r = blockIdx.x, c = blockIdx.y, chunks = gridDim.y;
  const float* row = logits + (size_t)r * vocab;
  const RowOptions o = read_options(options + (size_t)r * 6, vocab);
  int q_lo, q_hi;
  chunk_quads(vocab, q_lo, q_hi);
  if (o.temperature == 0.f) {
    Best best{-INFINITY, 0x7fffffff};
    for_each_in_quads(row, vocab, q_lo, q_hi, [&](int i, float v) { best = better(best, Best{v, i}); });
    best = block_best(best, best_scratch);
    if (threadIdx.x == 0) s.chunk_best[r * chunks + c] = best;
    return;
  }
  if (o.filter) {
    const int entries = 3 * SELECT_BINS;
    for (int e = c * blockDim.x + threadIdx.x; e < entries; e += chunks * blockDim.x) {
      s.counts[(size_t)r * entries + e] = 0u;
      s.masses[(size_t)r * entries + e] = 0ull;
    }
    if (c == 0 && threadIdx.x == 0) s.search[r].total_mass = 0ull;
  }
  float mx = -INFINITY;
  for_each_in_quads(row, vocab, q_lo, q_hi, [&](int, float v) { mx = fmaxf(mx, v * o.inv_t); });
  mx = block_max(mx, scratch);
  if (threadIdx.x == 0) s.chunk_max[r * chunks + c] = mx;
}

__device__ __forceinline__ float row_max_of_chunks(const float* __restrict__ chunk_max, int chunks) {
  float mx = -INFINITY;
  for (int c = 0; c < chunks; ++c) mx = fmaxf(mx, chunk_max[c]);
  return mx;
}

// The digit of `level` from the row's finished tables (global), given what was found before; `counts`, `masses`: LDS.
__device__ __forceinline__ uint32_t finished_digit(const ChunkedScratch& s, int r, int level, const RowOptions& o, uint32_t prefix_before, Above& above,
                                                   unsigned int* counts, unsigned long long* masses, int* found_digit, Above* found_above) {
  const int bins = level_bins(level);
  const size_t base = ((size_t)r * 3 + level) * SELECT_BINS;
  for (int b = threadIdx.x; b < bins; b += blockDim.x) { counts[b] = s.counts[base + b]; masses[b] = s.masses[base + b]; }
  __syncthreads();
  const unsigned long long mass_limit = max(1ull, (unsigned long long)((double)o.top_p * (double)s.search[r].total_mass));
  const int digit = select_digit(counts, masses, bins, o.top_k, o.use_mass, mass_limit, above, found_digit, found_above);
  __syncthreads();  // the tables are free again
  return prefix_before | ((uint32_t)digit << level_shift(level));
}

// passes 2..4: the tables of digit LEVEL
template <int LEVEL>
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_chunk_tables_kernel(const float* __restrict__ logits, const int* __restrict__ options,
                                                                             ChunkedScratch s, int vocab) {
  __shared__ unsigned int counts[SELECT_BINS];
  __shared__ unsigned long long masses[SELECT_BINS];
  __shared__ unsigned long long total_mass;
  __shared__ int found_digit;
  __shared__ Above found_above;
  const int r = blockIdx.x, c = blockIdx.y, chunks = gridDim.y;
  const float* row = logits + (size_t)r * vocab;
  const RowOptions o = read_options(options + (size_t)r * 6, vocab);
  if (o.temperature == 0.f || !o.filter) return;
  const int tid = threadIdx.x;
  int q_lo, q_hi;
  chunk_quads(vocab, q_lo, q_hi);
  const float mx = row_max_of_chunks(s.chunk_max + r * chunks, chunks);
  uint32_t prefix = 0u;
  if (LEVEL >= 1) {
    Above above{0u, 0ull};
    if (LEVEL == 2) { prefix = s.search[r].prefix[0]; above.count = s.search[r].above_count[0]; above.mass = s.search[r].above_mass[0]; }
    prefix = finished_digit(s, r, LEVEL - 1, o, prefix, above, counts, masses, &found_digit, &found_above);
    if (c == 0 && tid == 0) {
      s.search[r].prefix[LEVEL - 1] = prefix;
      s.search[r].above_count[LEVEL - 1] = above.count;
      s.search[r].above_mass[LEVEL - 1] = above.mass;
    }
  }
  const int bins = level_bins(LEVEL);
  for (int b = tid; b < bins; b += blockDim.x) { counts[b] = 0u; masses[b] = 0ull; }
  if (tid == 0) total_mass = 0ull;
  __syncthreads();
  const unsigned long long my_total = add_to_tables(row, vocab, q_lo, q_hi, o, mx, LEVEL, prefix, counts, masses);
  if (LEVEL == 0 && o.use_mass && my_total != 0ull) atomicAdd(&total_mass, my_total);
  __syncthreads();
  const size_t base = ((size_t)r * 3 + LEVEL) * SELECT_BINS;
  for (int b = tid; b < bins; b += blockDim.x) {
    if (counts[b] != 0u) atomicAdd(&s.counts[base + b], counts[b]);
    if (masses[b] != 0ull) atomicAdd(&s.masses[base + b], masses[b]);
  }
  if (LEVEL == 0 && tid == 0 && total_mass != 0ull) atomicAdd(&s.search[r].total_mass, total_mass);
}

// pass 5: the last digit, then the draw among the chunk's kept tokens
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_chunk_draw_kernel(const float* __restrict__ logits, const int* __restrict__ options,
                                                                           ChunkedScratch s, int vocab, int with_filter) {
  __shared__ Best best_scratch[16];
  __shared__ unsigned int counts[SELECT_BINS];
  __shared__ unsigned long long masses[SELECT_BINS];
  __shared__ int found_digit;
  __shared__ Above found_above;
  const int r = blockIdx.x, c = blockIdx.y, chunks = gridDim.y;
  const float* row = logits + (size_t)r * vocab;
  const RowOptions o = read_options(options + (size_t)r * 6, vocab);
  if (o.temperature == 0.f) return;  // (its chunks' best pairs are there since the first pass)
  int q_lo, q_hi;
  chunk_quads(vocab, q_lo, q_hi);
  const float mx = row_max_of_chunks(s.chunk_max + r * chunks, chunks);
  uint32_t threshold = 0u;
  if (o.filter && !with_filter) {
    // the caller promised that no row has a filter, and this one has: the kernels of the digits did not run.  No token
    // rather than one drawn from the wrong set: the row's result is -1.
    if (threadIdx.x == 0) s.chunk_best[r * chunks + c] = Best{INFINITY, -1};
    return;
  }
  if (o.filter) {
    Above above{s.search[r].above_count[1], s.search[r].above_mass[1]};
    threshold = finished_digit(s, r, 2, o, s.search[r].prefix[1], above, counts, masses, &found_digit, &found_above);
  }
  Best best = draw_in_quads(row, vocab, q_lo, q_hi, o, mx, threshold);
  best = block_best(best, best_scratch);
  if (threadIdx.x == 0) s.chunk_best[r * chunks + c] = best;
}

extern "C" long long velox_sample_chunked_scratch_bytes(int rows, int chunks) {
  if (rows < 1 || chunks < 1) return 0;
  return (long long)chunked_scratch_layout(rows, chunks, nullptr, nullptr);
}

// The same tokens as velox_sample, every row cut into `chunks` chunks.  scratch: velox_sample_chunked_scratch_bytes(rows,
// chunks) bytes at a 256-byte boundary, contents arbitrary.  with_filter = 0 promises that no row has top-k or top-p (the
// three kernels of the digits are then left out; a row that has one all the same gets the token -1).
extern "C" int velox_sample_chunked(const float* logits, const int* options, int* out, int rows, int vocab, int chunks, void* scratch,
                                    long long scratch_bytes, int with_filter, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (chunks < 2 || chunks > 1024 || rows > 65535 || scratch == nullptr || ((uintptr_t)scratch & 255) != 0) return -1;
  ChunkedScratch s;
  if ((long long)chunked_scratch_layout(rows, chunks, scratch, &s) > scratch_bytes) return -1;
  const dim3 grid(rows, chunks);
  sample_chunk_max_kernel<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, options, s, vocab);
  if (with_filter) {
    sample_chunk_tables_kernel<0><<<grid, SAMPLE_THREADS, 0, stream>>>(logits, options, s, vocab);
    sample_chunk_tables_kernel<1><<<grid, SAMPLE_THREADS, 0, stream>>>(logits, options, s, vocab);
    sample_chunk_tables_kernel<2><<<grid, SAMPLE_THREADS, 0, stream>>>(logits, options, s, vocab);
  }
  sample_chunk_draw_kernel<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, options, s, vocab, with_filter);
  argmax_merge_kernel<<<rows, 64, 0, stream>>>(s.chunk_best, out, chunks);
  VELOX_RETURN_LAUNCH_STATUS();
}

// Penalties over the tokens a request has seen (prompt and output), each distinct token once:
//   v = logit - frequency * count;  v = v > 0 ? v / repetition : v * repetition;  v -= presence
// One workgroup per row.  The vocabulary is taken a range of PENALTY_RANGE token ids at a time: the history's tokens
// inside the range are counted into a table in LDS, then the history is walked again and whoever takes a token's count
// out of the table (leaving zero behind, so the table is clean for the next range) applies it.  Work grows with the
// history's length times the number of ranges, never with its square.
#define PENALTY_RANGE 8192
__global__ void __launch_bounds__(256) penalties_kernel(float* __restrict__ logits, const int* __restrict__ tokens, const int* __restrict__ lengths,
                                                        const float* __restrict__ coeffs, int vocab, int width) {
  __shared__ int table[PENALTY_RANGE];
  __shared__ unsigned int touched[(1 << 20) / PENALTY_RANGE / 32 + 1];  // one bit per range (vocabularies up to 2^20 ids and beyond: see below)
  const int r = blockIdx.x;
  const int n = lengths[r] < width ? lengths[r] : width;
  const int* seen = tokens + (size_t)r * width;
  const float repetition = coeffs[3 * r], presence = coeffs[3 * r + 1], frequency = coeffs[3 * r + 2];
  float* row = logits + (size_t)r * vocab;
  const int ranges = (vocab + PENALTY_RANGE - 1) / PENALTY_RANGE;
  const bool track = ranges <= (1 << 20) / PENALTY_RANGE;  // (a larger vocabulary visits every range)
  for (int i = threadIdx.x; i < PENALTY_RANGE; i += blockDim.x) table[i] = 0;
  for (int i = threadIdx.x; i < (int)(sizeof(touched) / sizeof(touched[0])); i += blockDim.x) touched[i] = 0u;
  __syncthreads();
  if (track) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int token = seen[i];
      if (token >= 0 && token < vocab) atomicOr(&touched[(token / PENALTY_RANGE) >> 5], 1u << ((token / PENALTY_RANGE) & 31));
    }
    __syncthreads();
  }
  for (int range = 0; range < ranges; ++range) {
    if (track && !((touched[range >> 5] >> (range & 31)) & 1u)) continue;  // (the same for every thread)
    const int lo = range * PENALTY_RANGE;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int token = seen[i];
      if (token >= lo && token < lo + PENALTY_RANGE && token < vocab) atomicAdd(&table[token - lo], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int token = seen[i];
      if (token < lo || token >= lo + PENALTY_RANGE || token >= vocab) continue;
      const int count = atomicExch(&table[token - lo], 0);
      if (count == 0) continue;  // another occurrence of the token took the count
      float v = row[token] - frequency * (float)count;
      v = v > 0.f ? v / repetition : v * repetition;
      row[token] = v - presence;
    }
    __syncthreads();
  }
}

extern "C" int velox_apply_penalties(float* logits, const int* tokens, const int* lengths, const float* coeffs, int rows, int vocab,
                                     int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  penalties_kernel<<<rows, 256, 0, stream>>>(logits, tokens, lengths, coeffs, vocab, width);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---- penalties from a table of counts that lives on the device -------------------------------------------------------
// counts: int32 [table rows, vocab], one row per request with penalties: how often the request has seen each token
// (prompt and output).  The row is built once from the request's tokens and then kept up to date from the sampler's
// output, on the device: a step's penalties need neither the history nor the value of the token before it on the host.
__global__ void __launch_bounds__(256) count_tokens_kernel(int* __restrict__ counts_row, const int* __restrict__ tokens, int n, int vocab) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const int token = tokens[i];
    if (token >= 0 && token < vocab) atomicAdd(&counts_row[token], 1);
  }
}

// row_of[r]: the table row of batch row r, or -1 (no penalties)
__global__ void __launch_bounds__(64) count_sampled_kernel(int* __restrict__ counts, const int* __restrict__ row_of, const int* __restrict__ tokens, int rows,
                                                           int vocab) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows || row_of[r] < 0) return;
  const int token = tokens[r];
  if (token >= 0 && token < vocab) atomicAdd(&counts[(size_t)row_of[r] * vocab + token], 1);  // (one request may not sit in two rows; atomic all the same)
}

// v = logit - frequency * count;  v = v > 0 ? v / repetition : v * repetition;  v -= presence, where count > 0
__global__ void __launch_bounds__(256) penalties_from_counts_kernel(float* __restrict__ logits, const int* __restrict__ counts, const int* __restrict__ row_of,
                                                                    const float* __restrict__ coeffs, int vocab) {
  const int r = blockIdx.x;
  const int table_row = row_of[r];
  if (table_row < 0) return;
  const float repetition = coeffs[3 * r], presence = coeffs[3 * r + 1], frequency = coeffs[3 * r + 2];
  float* row = logits + (size_t)r * vocab;
  const int* seen = counts + (size_t)table_row * vocab;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < vocab; i += gridDim.y * blockDim.x) {
    const int count = seen[i];
    if (count == 0) continue;
    float v = row[i] - frequency * (float)count;
    v = v > 0.f ? v / repetition : v * repetition;
    row[i] = v - presence;
  }
}

extern "C" int velox_count_tokens(int* counts_row, const int* tokens, int n, int vocab, hipStream_t stream) {
  if (n <= 0) return 0;
  const int blocks = (n + 255) / 256 < 256 ? (n + 255) / 256 : 256;
  count_tokens_kernel<<<blocks, 256, 0, stream>>>(counts_row, tokens, n, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" int velox_count_sampled(int* counts, const int* row_of, const int* tokens, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  count_sampled_kernel<<<(rows + 63) / 64, 64, 0, stream>>>(counts, row_of, tokens, rows, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" int velox_penalties_from_counts(float* logits, const int* counts, const int* row_of, const float* coeffs, int rows, int vocab, int chunks,
                                           hipStream_t stream) {
  if (rows <= 0) return 0;
  if (chunks < 1 || chunks > 65535 || rows > 65535) return -1;
  penalties_from_counts_kernel<<<dim3(rows, chunks), 256, 0, stream>>>(logits, counts, row_of, coeffs, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}
