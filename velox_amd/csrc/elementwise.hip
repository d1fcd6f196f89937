// Memory-bound kernels of the decoder step for gfx950: embedding gather, residual-add + RMSNorm,
// SiLU(gate) * up, and the fused bias + rotary + cache write.  All arithmetic is float32; values
// are rounded once, at the store.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// embedding: out[t, :] = float(table[ids[t], :]); an id outside the table yields NaN rows.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* dst = out + (size_t)t * hidden;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = __builtin_nanf("");
    return;
  }
  const T* src = table + (size_t)id * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(src[i]);
}

extern "C" int velox_embed(const int* ids, const void* table, float* out, int tokens, int hidden, int vocab, int table_dtype, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (table_dtype == VELOX_BF16)
    embed_kernel<bf16_t><<<tokens, 256, 0, stream>>>(ids, (const bf16_t*)table, out, hidden, vocab);
  else
    embed_kernel<float><<<tokens, 256, 0, stream>>>(ids, (const float*)table, out, hidden, vocab);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ids[dest[k]] = tokens[source[k]] for k < n: token ids that were sampled by the step before this one and have not been
// to the host, put where this step's rows expect them.  (Pairs outside either array are skipped: the host has checked.)
__global__ void __launch_bounds__(64) place_tokens_kernel(int* __restrict__ ids, const int* __restrict__ dest, const int* __restrict__ source,
                                                          const int* __restrict__ tokens, int n, int num_ids, int num_tokens) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n) return;
  const int to = dest[k], from = source[k];
  if (to >= 0 && to < num_ids && from >= 0 && from < num_tokens) ids[to] = tokens[from];
}

extern "C" int velox_place_tokens(int* ids, const int* dest, const int* source, const int* tokens, int n, int num_ids, int num_tokens,
                                  hipStream_t stream) {
  if (n <= 0) return 0;
  place_tokens_kernel<<<(n + 63) / 64, 64, 0, stream>>>(ids, dest, source, tokens, n, num_ids, num_tokens);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// residual add + RMSNorm.  One block per output row.
//   rows == nullptr: r = residual[row] (+ delta[row]); residual[row] = r; out[row] = norm(r)
//   rows != nullptr: r = residual[rows[row]] (+ delta[rows[row]]); out[row] = norm(r); nothing else is written
//   norm(r) = r * rsqrt(sum(r^2) / H + eps) * w
// ---------------------------------------------------------------------------------------------
//   delta may be `partials` stacked tensors (partial sums of a split product), `partial_stride` elements apart: they are
//   added in order, first to last.
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta, const int* __restrict__ rows,
                                   const float* __restrict__ weight, TO* __restrict__ out, int hidden, float eps,
                                   int partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const size_t src_row = rows ? (size_t)rows[row] : (size_t)row;
  float* res = residual + src_row * hidden;
  const TD* del = delta ? delta + src_row * hidden : nullptr;
  const bool write_back = (rows == nullptr) && (delta != nullptr);
  float sumsq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float r = res[i];
    if (del)
      for (int p = 0; p < partials; ++p) r += to_f32(del[p * partial_stride + i]);
    if (write_back) res[i] = r;
    sumsq += r * r;
  }
  const float total = block_sum(sumsq, scratch);
  const float inv = rsqrtf(total / (float)hidden + eps);
  TO* dst = out + (size_t)row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float r = res[i];
    if (del && !write_back)
      for (int p = 0; p < partials; ++p) r += to_f32(del[p * partial_stride + i]);
    dst[i] = from_f32<TO>(r * inv * weight[i]);
  }
}

// Same arithmetic with the row held in registers: one read of residual and delta, 16-byte accesses.  Needs
// hidden % 4 == 0 and hidden <= 4 * threads * CHUNKS.
template <typename T> struct Quad;
template <> struct Quad<float> {
  float4_t v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, float x) { v[i] = x; }
};
template <> struct Quad<bf16_t> {
  short4_t v;
  __device__ __forceinline__ float get(int i) const { return __uint_as_float(((uint32_t)(uint16_t)v[i]) << 16); }
  __device__ __forceinline__ void set(int i, float x) { v[i] = bf16_bits(x); }
};

template <typename TD, typename TO, int CHUNKS>
__global__ void add_rmsnorm_rows_in_registers_kernel(float* __restrict__ residual, const TD* __restrict__ delta, const int* __restrict__ rows,
                                                     const float* __restrict__ weight, TO* __restrict__ out, int hidden, float eps,
                                                     int partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const size_t src_row = rows ? (size_t)rows[row] : (size_t)row;
  float* res = residual + src_row * hidden;
  const TD* del = delta ? delta + src_row * hidden : nullptr;
  const bool write_back = (rows == nullptr) && (delta != nullptr);
  float4_t r[CHUNKS];
  float sumsq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int at = (threadIdx.x + c * blockDim.x) * 4;
    r[c] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (at < hidden) {
      r[c] = *reinterpret_cast<const float4_t*>(res + at);
      if (del) {
        // four partial sums are asked for together (the last one again where fewer are left) and added in order
        for (int p = 0; p < partials; p += 4) {
          Quad<TD> d[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int pu = p + u < partials ? p + u : partials - 1;
            d[u] = *reinterpret_cast<const Quad<TD>*>(del + pu * partial_stride + at);
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            if (p + u < partials) {
#pragma unroll
              for (int j = 0; j < 4; ++j) r[c][j] += d[u].get(j);
            }
          }
        }
      }
      if (write_back) *reinterpret_cast<float4_t*>(res + at) = r[c];
#pragma unroll
      for (int j = 0; j < 4; ++j) sumsq += r[c][j] * r[c][j];
    }
  }
  const float total = block_sum(sumsq, scratch);
  const float inv = rsqrtf(total / (float)hidden + eps);
  TO* dst = out + (size_t)row * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int at = (threadIdx.x + c * blockDim.x) * 4;
    if (at < hidden) {
      const float4_t w = *reinterpret_cast<const float4_t*>(weight + at);
      Quad<TO> o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o.set(j, r[c][j] * inv * w[j]);
      *reinterpret_cast<Quad<TO>*>(dst + at) = o;
    }
  }
}

extern "C" int velox_add_rmsnorm(float* residual, const void* delta, const int* rows, const float* weight, void* out,
                                 int num_rows, int hidden, float eps, int delta_dtype, int out_dtype, int partials,
                                 long long partial_stride, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (partials < 1 || (partials > 1 && partial_stride % 4 != 0)) return -1;
  const int threads = hidden >= 2048 ? 512 : 256;
  const bool aligned = (((uintptr_t)residual | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out) & 15) == 0;
  const bool in_registers = aligned && hidden % 4 == 0 && hidden <= 4 * threads * 4;
#define LAUNCH(TD, TO)                                                                                                                  \
  do {                                                                                                                                  \
    if (in_registers)                                                                                                                   \
      add_rmsnorm_rows_in_registers_kernel<TD, TO, 4><<<num_rows, threads, 0, stream>>>(residual, (const TD*)delta, rows, weight, (TO*)out, hidden, eps, partials, (size_t)partial_stride); \
    else                                                                                                                                \
      add_rmsnorm_kernel<TD, TO><<<num_rows, threads, 0, stream>>>(residual, (const TD*)delta, rows, weight, (TO*)out, hidden, eps, partials, (size_t)partial_stride); \
  } while (0)
  if (delta_dtype == VELOX_BF16 && out_dtype == VELOX_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == VELOX_F32 && out_dtype == VELOX_F32) LAUNCH(float, float);
  else if (delta_dtype == VELOX_BF16 && out_dtype == VELOX_F32) LAUNCH(bf16_t, float);
  else LAUNCH(float, bf16_t);
#undef LAUNCH
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// out[t, i] = silu(gate_up[t, i]) * gate_up[t, inter + i], silu(x) = x / (1 + exp(-x))
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter) {
  const int t = blockIdx.y;
  const T* row = gate_up + (size_t)t * 2 * inter;
  T* dst = out + (size_t)t * inter;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += gridDim.x * blockDim.x) {
    const float g = to_f32(row[i]);
    const float u = to_f32(row[inter + i]);
    dst[i] = from_f32<T>(g / (1.f + expf(-g)) * u);
  }
}

// 16-byte accesses; needs inter % (16 / sizeof(T)) == 0.
template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter) {
  constexpr int N = 16 / sizeof(T);
  const int t = blockIdx.y;
  const T* row = gate_up + (size_t)t * 2 * inter;
  T* dst = out + (size_t)t * inter;
  for (int at = (blockIdx.x * blockDim.x + threadIdx.x) * N; at < inter; at += gridDim.x * blockDim.x * N) {
    const float4_t gv = *reinterpret_cast<const float4_t*>(row + at);
    const float4_t uv = *reinterpret_cast<const float4_t*>(row + inter + at);
    float4_t ov;
    const T* ge = reinterpret_cast<const T*>(&gv);
    const T* ue = reinterpret_cast<const T*>(&uv);
    T* oe = reinterpret_cast<T*>(&ov);
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float g = to_f32(ge[j]);
      oe[j] = from_f32<T>(g / (1.f + expf(-g)) * to_f32(ue[j]));
    }
    *reinterpret_cast<float4_t*>(dst + at) = ov;
  }
}

extern "C" int velox_silu_mul(const void* gate_up, void* out, int tokens, int inter, int dtype, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const int per = dtype == VELOX_BF16 ? 8 : 4;
  if (inter % per == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    int bx = (inter / per + 255) / 256;
    if (bx > 32) bx = 32;
    dim3 grid(bx, tokens);
    if (dtype == VELOX_BF16) silu_mul_vec_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter);
    else silu_mul_vec_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter);
    VELOX_RETURN_LAUNCH_STATUS();
  }
  int bx = (inter + 255) / 256;
  if (bx > 64) bx = 64;
  dim3 grid(bx, tokens);
  if (dtype == VELOX_BF16) silu_mul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter);
  else silu_mul_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// bias + rotary + cache write, one block per token.
//   qkv[t] = [q (nh*d) | k (nkv*d) | v (nkv*d)], optional float32 bias of the same width.
//   q: q += bias; rotate; stored back in place.
//   k: k += bias; rotate; stored to k_cache[page, kv_head, offset, :]
//   v: v += bias;          stored to v_cache[page, kv_head, :, offset]
//   rotation of the first 2*half channels of a head, halves paired (i, i + half):
//     lo' = lo*cos - hi*sin, hi' = lo*sin + hi*cos, cos/sin = table[position[t], i]
//   slot = page * page_size + offset.  With write_kv == 0 only q is touched.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ positions,
                                     const float* __restrict__ cos_table, const float* __restrict__ sin_table, int half,
                                     const int* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     int nh, int nkv, int d, int page_size, int write_kv) {
  const int t = blockIdx.x;
  const int width = (nh + 2 * nkv) * d;
  T* row = qkv + (size_t)t * width;
  const int pos = positions[t];
  const float* cs = cos_table ? cos_table + (size_t)pos * half : nullptr;
  const float* sn = sin_table ? sin_table + (size_t)pos * half : nullptr;
  const int slot = slots[t];
  const size_t page = (size_t)(slot / page_size);
  const int offset = slot % page_size;
  const int half_d = d / 2;  // work items per head: pairs (i, i + d/2) so every channel is visited once

  const int q_items = nh * half_d;
  const int k_items = write_kv ? nkv * half_d : 0;
  for (int item = threadIdx.x; item < q_items + k_items; item += blockDim.x) {
    const bool is_k = item >= q_items;
    const int local = is_k ? item - q_items : item;
    const int head = local / half_d;
    const int i = local % half_d;
    const int base = (is_k ? nh * d : 0) + head * d;
    // the two channels this item owns
    int c0, c1;
    bool rotate;
    if (cs != nullptr && i < half) { c0 = i; c1 = i + half; rotate = true; }
    else {
      // channels outside the rotated span are handled in pairs of their own so that all d are covered
      // rotated span is [0, 2*half); the remaining d - 2*half channels are split over items i >= half
      const int rest = (cs != nullptr) ? 2 * half : 0;
      const int j = (cs != nullptr) ? i - half : i;
      c0 = rest + 2 * j; c1 = c0 + 1; rotate = false;
    }
    float x0 = to_f32(row[base + c0]);
    float x1 = to_f32(row[base + c1]);
    if (bias) { x0 += bias[base + c0]; x1 += bias[base + c1]; }
    float y0 = x0, y1 = x1;
    if (rotate) {
      const float c = cs[i], s = sn[i];
      y0 = x0 * c - x1 * s;
      y1 = x0 * s + x1 * c;
    }
    if (!is_k) {
      row[base + c0] = from_f32<T>(y0);
      row[base + c1] = from_f32<T>(y1);
    } else {
      T* dst = k_cache + ((page * nkv + head) * page_size + offset) * d;
      dst[c0] = from_f32<T>(y0);
      dst[c1] = from_f32<T>(y1);
    }
  }
  if (write_kv) {
    const int v_base = (nh + nkv) * d;
    for (int item = threadIdx.x; item < nkv * d; item += blockDim.x) {
      const int head = item / d;
      const int c = item % d;
      float x = to_f32(row[v_base + item]);
      if (bias) x += bias[v_base + item];
      v_cache[((page * nkv + head) * d + c) * page_size + offset] = from_f32<T>(x);
    }
  }
}

// The same with 16-byte accesses, for the usual case that the whole head rotates (2 * half == d) or nothing does.
// An item is a run of N = 16 / sizeof(T) channels of the low half of a head together with the matching run of the high half.
// PARTIAL = true: the rows come as `parts` float32 partial sums, partial[s][token][column] (what the split-K product
// leaves), added here in the order s = 0, 1, ...; qkv is then only written.  Otherwise qkv is read and written in place.
template <typename T, bool PARTIAL>
struct RowSource {
  const T* qkv;
  const float* partial;
  int parts;
  size_t part_stride;  // elements between two partial sums
  __device__ __forceinline__ float at(size_t index) const {
    if constexpr (PARTIAL) {
      float sum = partial[index];
      for (int s = 1; s < parts; ++s) sum += partial[s * part_stride + index];
      return sum;
    } else {
      return to_f32(qkv[index]);
    }
  }
  // N consecutive elements from a 16-byte aligned index
  template <int N> __device__ __forceinline__ void run(size_t index, float* out) const {
    if constexpr (PARTIAL) {
#pragma unroll
      for (int j = 0; j < N; ++j) out[j] = 0.f;
      // three partial sums are asked for together (the last one again where fewer are left) and added in order
      for (int s = 0; s < parts; s += 3) {
        float4_t more[3][N / 4];
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          const int su = s + u < parts ? s + u : parts - 1;
#pragma unroll
          for (int piece = 0; piece < N / 4; ++piece) more[u][piece] = reinterpret_cast<const float4_t*>(partial + su * part_stride + index)[piece];
        }
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          if (s + u < parts) {
#pragma unroll
            for (int piece = 0; piece < N / 4; ++piece)
#pragma unroll
              for (int j = 0; j < 4; ++j) out[4 * piece + j] += more[u][piece][j];
          }
        }
      }
    } else {
      const float4_t raw = *reinterpret_cast<const float4_t*>(qkv + index);
      const T* values = reinterpret_cast<const T*>(&raw);
#pragma unroll
      for (int j = 0; j < N; ++j) out[j] = to_f32(values[j]);
    }
  }
};

template <typename T, bool PARTIAL>
__global__ void rope_kv_write_vec_kernel(T* __restrict__ qkv, const float* __restrict__ partial, int parts, const float* __restrict__ bias,
                                         const int* __restrict__ positions, const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                         const int* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                         int nh, int nkv, int d, int page_size, int write_kv) {
  constexpr int N = 16 / sizeof(T);
  const int t = blockIdx.x;
  const int half = d / 2;
  const int width = (nh + 2 * nkv) * d;
  const RowSource<T, PARTIAL> source{qkv, partial, parts, (size_t)gridDim.x * width};
  const size_t row_at = (size_t)t * width;
  T* row = qkv + row_at;
  const int pos = positions[t];
  const float* cs = cos_table ? cos_table + (size_t)pos * half : nullptr;
  const float* sn = sin_table ? sin_table + (size_t)pos * half : nullptr;
  const int slot = slots[t];
  const size_t page = (size_t)(slot / page_size);
  const int offset = slot % page_size;
  const int runs = half / N;
  const int q_items = nh * runs;
  const int k_items = write_kv ? nkv * runs : 0;
  for (int item = threadIdx.x; item < q_items + k_items; item += blockDim.x) {
    const bool is_k = item >= q_items;
    const int local = is_k ? item - q_items : item;
    const int head = local / runs;
    const int c0 = (local % runs) * N;
    const int base = (is_k ? nh * d : 0) + head * d;
    __attribute__((aligned(16))) float x_lo[N], x_hi[N];
    source.template run<N>(row_at + base + c0, x_lo);
    source.template run<N>(row_at + base + half + c0, x_hi);
    // bias and angles of the run, as 16-byte loads (c0 and half are multiples of N, the tables' rows of half)
    __attribute__((aligned(16))) float b_lo[N], b_hi[N], cos_run[N], sin_run[N];
#pragma unroll
    for (int piece = 0; piece < N / 4; ++piece) {
      const float4_t zero = {0.f, 0.f, 0.f, 0.f};
      reinterpret_cast<float4_t*>(b_lo)[piece] = bias ? reinterpret_cast<const float4_t*>(bias + base + c0)[piece] : zero;
      reinterpret_cast<float4_t*>(b_hi)[piece] = bias ? reinterpret_cast<const float4_t*>(bias + base + half + c0)[piece] : zero;
      reinterpret_cast<float4_t*>(cos_run)[piece] = cs ? reinterpret_cast<const float4_t*>(cs + c0)[piece] : zero;
      reinterpret_cast<float4_t*>(sin_run)[piece] = sn ? reinterpret_cast<const float4_t*>(sn + c0)[piece] : zero;
    }
    float4_t lo_v, hi_v;
    T* lo = reinterpret_cast<T*>(&lo_v);
    T* hi = reinterpret_cast<T*>(&hi_v);
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float x0 = x_lo[j] + b_lo[j], x1 = x_hi[j] + b_hi[j];
      float y0 = x0, y1 = x1;
      if (cs) {
        y0 = x0 * cos_run[j] - x1 * sin_run[j];
        y1 = x0 * sin_run[j] + x1 * cos_run[j];
      }
      lo[j] = from_f32<T>(y0);
      hi[j] = from_f32<T>(y1);
    }
    T* dst = is_k ? k_cache + ((page * nkv + head) * page_size + offset) * d : row + base;
    *reinterpret_cast<float4_t*>(dst + c0) = lo_v;
    *reinterpret_cast<float4_t*>(dst + half + c0) = hi_v;
  }
  if (write_kv) {
    // Values go to [channel][offset].  Eight consecutive tokens of a prompt fill eight consecutive offsets of a page:
    // where this token sits in such a run (slots s .. s + 7 with s a multiple of 8, held by tokens t' .. t' + 7), the
    // run's first token writes all eight as whole 16- or 32-byte pieces and the other seven write nothing; every
    // token's workgroup finds the same answer from the slots alone.  (Single 2-byte stores from eight workgroups, on
    // different parts of the GPU, to one cache line are what made this kernel slow for prompts.)
    constexpr int RUN = 8;
    const int v_base = (nh + nkv) * d;
    const int lead = t - offset % RUN;  // the token that would hold the run's first slot
    bool in_run = page_size >= RUN && lead >= 0 && lead + RUN <= (int)gridDim.x;
    if (in_run) {
      const int first_slot = slot - offset % RUN;
      for (int j = 0; j < RUN; ++j) in_run = in_run && slots[lead + j] == first_slot + j;
    }
    if (!in_run) {
      // neighbouring lanes take neighbouring channels, so that a store instruction touches as few cache lines as the layout allows
      for (int item = threadIdx.x; item < nkv * d; item += blockDim.x) {
        const int head = item / d, c = item % d;
        float x = source.at(row_at + v_base + item);
        if (bias) x += bias[v_base + item];
        v_cache[((page * nkv + head) * d + c) * page_size + offset] = from_f32<T>(x);
      }
    } else if (lead == t) {
      for (int item = threadIdx.x; item < nkv * d; item += blockDim.x) {
        const int head = item / d, c = item % d;
        const float b = bias ? bias[v_base + item] : 0.f;
        __attribute__((aligned(16))) T run[RUN];
#pragma unroll
        for (int j = 0; j < RUN; ++j) run[j] = from_f32<T>(source.at((size_t)(t + j) * width + v_base + item) + b);
        T* dst = v_cache + ((page * nkv + head) * d + c) * page_size + offset;
#pragma unroll
        for (int piece = 0; piece < (int)(RUN * sizeof(T) / 16); ++piece)
          reinterpret_cast<float4_t*>(dst)[piece] = reinterpret_cast<const float4_t*>(run)[piece];
      }
    }
  }
}

// Rows that come as float32 partial sums partial[parts][tokens][(nh + 2 nkv) d] (bfloat16 only): their sum, plus bias, is
// rotated; queries go to qkv[tokens][(nh + 2 nkv) d] (only the query columns are written), keys and values to the cache.
// Needs a rotation of the whole head or none, d / 2 a multiple of 8, and 16-byte aligned operands.
extern "C" int velox_rope_kv_write_partial_bf16(void* qkv, const float* partial, int parts, const float* bias, const int* positions,
                                                const float* cos_table, const float* sin_table, int half, const int* slots, void* k_cache,
                                                void* v_cache, int tokens, int nh, int nkv, int d, int page_size, int write_kv, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const bool whole_head = (cos_table == nullptr || 2 * half == d) && (d / 2) % 8 == 0;
  const bool aligned = (((uintptr_t)qkv | (uintptr_t)partial | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)bias | (uintptr_t)cos_table | (uintptr_t)sin_table) & 15) == 0;
  if (!whole_head || !aligned || parts < 1) return (int)hipErrorInvalidValue;
  rope_kv_write_vec_kernel<bf16_t, true><<<tokens, 256, 0, stream>>>((bf16_t*)qkv, partial, parts, bias, positions, cos_table, sin_table, slots,
                                                                    (bf16_t*)k_cache, (bf16_t*)v_cache, nh, nkv, d, page_size, write_kv);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" int velox_rope_kv_write(void* qkv, const float* bias, const int* positions, const float* cos_table, const float* sin_table,
                                   int half, const int* slots, void* k_cache, void* v_cache, int tokens, int nh, int nkv, int d,
                                   int page_size, int write_kv, int dtype, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const int per = dtype == VELOX_BF16 ? 8 : 4;
  const bool whole_head = (cos_table == nullptr || 2 * half == d) && (d / 2) % per == 0;
  const bool aligned = (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)bias | (uintptr_t)cos_table | (uintptr_t)sin_table) & 15) == 0;
  if (whole_head && aligned) {
    if (dtype == VELOX_BF16)
      rope_kv_write_vec_kernel<bf16_t, false><<<tokens, 256, 0, stream>>>((bf16_t*)qkv, nullptr, 0, bias, positions, cos_table, sin_table, slots,
                                                                  (bf16_t*)k_cache, (bf16_t*)v_cache, nh, nkv, d, page_size, write_kv);
    else
      rope_kv_write_vec_kernel<float, false><<<tokens, 256, 0, stream>>>((float*)qkv, nullptr, 0, bias, positions, cos_table, sin_table, slots,
                                                                 (float*)k_cache, (float*)v_cache, nh, nkv, d, page_size, write_kv);
    VELOX_RETURN_LAUNCH_STATUS();
  }
  if (dtype == VELOX_BF16)
    rope_kv_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>((bf16_t*)qkv, bias, positions, cos_table, sin_table, half, slots,
                                                            (bf16_t*)k_cache, (bf16_t*)v_cache, nh, nkv, d, page_size, write_kv);
  else
    rope_kv_write_kernel<float><<<tokens, 256, 0, stream>>>((float*)qkv, bias, positions, cos_table, sin_table, half, slots,
                                                           (float*)k_cache, (float*)v_cache, nh, nkv, d, page_size, write_kv);
  VELOX_RETURN_LAUNCH_STATUS();
}


// out[m, :] = x[m, :] * rsqrt(sum_b sums[m][b] / width + eps): the second half of a norm whose first half (the weight)
// a product's epilogue has applied already; for consumers that cannot scale their own result rows.  m <= 16 rows.
__global__ void row_scale_apply_kernel(const bf16_t* __restrict__ x, const float* __restrict__ sums, int blocks, float inv_width,
                                       float eps, bf16_t* __restrict__ out, int n) {
  __shared__ float scale;
  const int row = blockIdx.x;
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int b = 0; b < blocks; ++b) total += sums[(size_t)row * blocks + b];
    scale = rsqrtf(total * inv_width + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) out[(size_t)row * n + i] = from_f32<bf16_t>(to_f32(x[(size_t)row * n + i]) * scale);
}

extern "C" int velox_row_scale_apply(const void* x, const float* sums, int blocks, float inv_width, float eps, void* out, int m, int n,
                                     hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (m > 16) return -1;
  row_scale_apply_kernel<<<m, 256, 0, stream>>>((const bf16_t*)x, sums, blocks, inv_width, eps, (bf16_t*)out, n);
  VELOX_RETURN_LAUNCH_STATUS();
}
