// Paged attention for gfx950, one head size per build (-DVELOX_HEAD_DIM=<multiple of 16>), float32 and bfloat16.
//
// One kernel serves portions of prompts, single decoded tokens and any mix of them.  A sequence
// b brings q_len = cu_q[b+1] - cu_q[b] new tokens; its keys 0 .. kv_len-1 are in the cache already
// (the step wrote this portion's keys before calling).  The query of token m sits at position
// kv_len - q_len + m and reads key n iff n <= position (and n > position - window when a window is
// set).  Scores are (q . k) * scale in float32, softmax in float32 with a running maximum, the
// probabilities are rounded to the value type for the second product (nothing is rounded in a
// float32 run), the sum of the unrounded probabilities normalises.
//
// Work split.  The G = heads / kv_heads query heads that share a KV head are stacked under their
// token: row r of a sequence = (token r / G, head kv_head * G + r % G).  A workgroup of 4 waves
// owns 64 consecutive rows of one (sequence, KV head): each wave 16 rows, all waves share the K/V
// tiles staged in LDS.  A decode step is the case q_len = 1 (rows = the G heads); its keys can be
// split over `splits` workgroups whose partial results a second kernel merges.
//
// Matrix cores.  Both products run on 16x16 MFMA tiles in the transposed form, so no register
// shuffles are needed between them:  S^T[key, row] = K Q^T,  O^T[channel, row] = V^T P^T.
// Operand convention (`Frag`): for a block of 16 contraction indices, lane (g = lane / 16,
// i = lane % 16) holds indices 4g .. 4g+3 of matrix row/column i.  bfloat16 feeds one
// v_mfma_f32_16x16x16_bf16 per block, float32 four v_mfma_f32_16x16x4_f32 (true float32 inputs).
// The accumulator of a tile is, per lane, rows 4g .. 4g+3 of column i: exactly the Frag of the next
// product's right operand.  Values are cached transposed inside a page ([channel][offset]) so the
// V^T tile is filled by contiguous copies.
#include "common.h"

#ifndef VELOX_HEAD_DIM
#error "build with -DVELOX_HEAD_DIM=<head size>"
#endif

constexpr int D = VELOX_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 between 16 and 256");
constexpr int ROWS_PER_BLOCK = 64;

template <typename T> struct Frag;
template <> struct Frag<float> { float4_t v; };
template <> struct Frag<bf16_t> { short4_t v; };

template <typename T> __device__ __forceinline__ Frag<T> load_frag(const T* p) {
  Frag<T> f;
  if constexpr (sizeof(T) == 4) f.v = *reinterpret_cast<const float4_t*>(p);
  else f.v = *reinterpret_cast<const short4_t*>(p);
  return f;
}
template <typename T> __device__ __forceinline__ Frag<T> zero_frag() {
  Frag<T> f;
  f.v[0] = 0; f.v[1] = 0; f.v[2] = 0; f.v[3] = 0;
  return f;
}

__device__ __forceinline__ float4_t mma16(const Frag<float>& a, const Frag<float>& b, float4_t c) {
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[0], b.v[0], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[1], b.v[1], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[2], b.v[2], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[3], b.v[3], c, 0, 0, 0);
  return c;
}
__device__ __forceinline__ float4_t mma16(const Frag<bf16_t>& a, const Frag<bf16_t>& b, float4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, b.v, c, 0, 0, 0);
}

__device__ __forceinline__ void set_prob(Frag<float>& f, int j, float p) { f.v[j] = p; }
__device__ __forceinline__ void set_prob(Frag<bf16_t>& f, int j, float p) { f.v[j] = bf16_bits(p); }

// exp for the softmax: the library's accurate expf in a float32 run, the hardware exp2 otherwise
template <typename T> __device__ __forceinline__ float softmax_exp(float x) {
  if constexpr (sizeof(T) == 4) return expf(x);
  else return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}

template <typename T> struct Vec16;  // 16 bytes of T
template <> struct Vec16<float> { float4_t v; static constexpr int N = 4; };
template <> struct Vec16<bf16_t> { float4_t v; static constexpr int N = 8; };

// keeps the first `valid` elements of a 16-byte vector, zeroes the rest
__device__ __forceinline__ void mask_tail(Vec16<float>& x, int valid) {
#pragma unroll
  for (int i = 0; i < 4; ++i) x.v[i] = i < valid ? x.v[i] : 0.f;
}
__device__ __forceinline__ void mask_tail(Vec16<bf16_t>& x, int valid) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t keep = (2 * w < valid ? 0x0000ffffu : 0u) | (2 * w + 1 < valid ? 0xffff0000u : 0u);
    x.v[w] = __uint_as_float(__float_as_uint(x.v[w]) & keep);
  }
}

template <typename T, int BN>
__global__ void __launch_bounds__(256) paged_attention_kernel(
    const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ cu_q, const int* __restrict__ kv_lens,
    T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_lse,
    int nh, int nkv, int page_shift, float scale, int window, int splits, int total_tokens) {
  constexpr int PAD = 16 / sizeof(T);
  constexpr int KS = D + PAD;   // row stride of the K tile   [BN][D]
  constexpr int VS = BN + PAD;  // row stride of the V^T tile [D][BN]
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NT = BN / 16;
  constexpr int NC = D / 16;
  __shared__ __attribute__((aligned(16))) T k_tile[BN * KS];
  __shared__ __attribute__((aligned(16))) T v_tile[D * VS];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i = lane & 15;
  const int group = nh / nkv;
  const int kvh = blockIdx.y;
  const int b = blockIdx.z / splits, split = blockIdx.z % splits;
  const int page_size = 1 << page_shift;

  const int q_start = cu_q[b];
  const int q_len = cu_q[b + 1] - q_start;
  const int kv_len = kv_lens[b];
  const int ctx = kv_len - q_len;
  const int rows_total = q_len * group;
  const int r0 = blockIdx.x * ROWS_PER_BLOCK;
  if (r0 >= rows_total) return;

  const int r = r0 + wave * 16 + i;
  const bool row_ok = r < rows_total;
  const int tok = row_ok ? r / group : 0;
  const int head = kvh * group + (row_ok ? r % group : 0);
  const int pos = ctx + tok;

  // keys this workgroup has to visit
  const int first_tok = r0 / group;
  const int last_row = (r0 + ROWS_PER_BLOCK - 1 < rows_total - 1) ? r0 + ROWS_PER_BLOCK - 1 : rows_total - 1;
  const int last_tok = last_row / group;
  int n_end = ctx + last_tok + 1;
  if (n_end > kv_len) n_end = kv_len;
  int n_begin = 0;
  if (window > 0) {
    n_begin = ctx + first_tok - window + 1;
    if (n_begin < 0) n_begin = 0;
    n_begin = n_begin / BN * BN;
  }
  const int tiles_total = (n_end - n_begin + BN - 1) / BN;
  const int tiles_per_split = (tiles_total + splits - 1) / splits;
  const int tile_lo = split * tiles_per_split;
  int tile_hi = tile_lo + tiles_per_split;
  if (tile_hi > tiles_total) tile_hi = tiles_total;

  // what this wave can skip: tiles wholly after its last row's position
  int wave_last_pos = row_ok ? pos : -1;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const int other = __shfl_xor(wave_last_pos, offset, VELOX_WAVE);
    wave_last_pos = other > wave_last_pos ? other : wave_last_pos;
  }

  Frag<T> qf[NC];
  {
    const T* qp = qkv + (size_t)(q_start + tok) * qkv_stride + (size_t)head * D + 4 * g;
#pragma unroll
    for (int c = 0; c < NC; ++c) qf[c] = row_ok ? load_frag<T>(qp + 16 * c) : zero_frag<T>();
  }

  float m_i = -INFINITY, l_i = 0.f;
  float4_t acc_o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) acc_o[c] = float4_t{0.f, 0.f, 0.f, 0.f};

  const int* table = block_tables + (size_t)b * table_width;

  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int n0 = n_begin + tile * BN;
    __syncthreads();
    // ---- stage K[n0 .. n0+BN) as [key][channel] -------------------------------------------
    {
      constexpr int VPR = D / VEC;
      for (int v = tid; v < BN * VPR; v += 256) {
        const int key = v / VPR, vec = v % VPR;
        const int n = n0 + key;
        Vec16<T> x;
        x.v = float4_t{0.f, 0.f, 0.f, 0.f};
        if (n < kv_len) {
          const size_t page = (size_t)table[n >> page_shift];
          const int off = n & (page_size - 1);
          x.v = *reinterpret_cast<const float4_t*>(k_cache + ((page * nkv + kvh) * page_size + off) * D + vec * VEC);
        }
        *reinterpret_cast<float4_t*>(k_tile + key * KS + vec * VEC) = x.v;
      }
    }
    // ---- stage V^T[n0 .. n0+BN) as [channel][key] -----------------------------------------
    {
      const int run = page_size < BN ? page_size : BN;  // consecutive keys that are contiguous in a page
      if (run >= VEC) {
        const int vpr = run / VEC;
        const int per_run = D * vpr;
        for (int v = tid; v < BN * D / VEC; v += 256) {
          const int rn = v / per_run, rem = v % per_run;
          const int dd = rem / vpr, vec = rem % vpr;
          const int nl = rn * run + vec * VEC;
          const int n = n0 + nl;
          Vec16<T> x;
          x.v = float4_t{0.f, 0.f, 0.f, 0.f};
          if (n < kv_len) {
            const size_t page = (size_t)table[n >> page_shift];
            const int off = n & (page_size - 1);
            x.v = *reinterpret_cast<const float4_t*>(v_cache + ((page * nkv + kvh) * D + dd) * page_size + off);
            if (n + VEC > kv_len) mask_tail(x, kv_len - n);
          }
          *reinterpret_cast<float4_t*>(v_tile + dd * VS + nl) = x.v;
        }
      } else {
        const int per_run = D * run;
        for (int v = tid; v < BN * D; v += 256) {
          const int rn = v / per_run, rem = v % per_run;
          const int dd = rem / run, e = rem % run;
          const int nl = rn * run + e;
          const int n = n0 + nl;
          T x = from_f32<T>(0.f);
          if (n < kv_len) {
            const size_t page = (size_t)table[n >> page_shift];
            const int off = n & (page_size - 1);
            x = v_cache[((page * nkv + kvh) * D + dd) * page_size + off];
          }
          v_tile[dd * VS + nl] = x;
        }
      }
    }
    __syncthreads();
    if (n0 > wave_last_pos) continue;  // nothing this wave may read; it still took part in the staging

    // ---- S^T = K Q^T ----------------------------------------------------------------------
    float4_t s[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      s[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const Frag<T> a = load_frag<T>(k_tile + (16 * t + i) * KS + 16 * c + 4 * g);
        s[t] = mma16(a, qf[c], s[t]);
      }
    }
    // ---- mask, running maximum ------------------------------------------------------------
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + 16 * t + 4 * g + j;
        const bool keep = row_ok && n < kv_len && n <= pos && (window <= 0 || n > pos - window);
        const float val = keep ? s[t][j] * scale : -INFINITY;
        s[t][j] = val;
        mx = fmaxf(mx, val);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, VELOX_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, VELOX_WAVE));
    const float m_new = fmaxf(m_i, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m_i == -INFINITY) ? 0.f : softmax_exp<T>(m_i - m_safe);
    float psum = 0.f;
    Frag<T> pf[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = (s[t][j] == -INFINITY) ? 0.f : softmax_exp<T>(s[t][j] - m_safe);
        psum += p;
        set_prob(pf[t], j, p);
      }
    l_i = l_i * alpha + psum;  // partial over this lane's keys; the four lane groups are summed at the end
    m_i = m_new;
    // ---- O^T = O^T * alpha + V^T P^T ------------------------------------------------------
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      acc_o[c] = acc_o[c] * alpha;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const Frag<T> a = load_frag<T>(v_tile + (16 * c + i) * VS + 16 * t + 4 * g);
        acc_o[c] = mma16(a, pf[t], acc_o[c]);
      }
    }
  }

  l_i += __shfl_xor(l_i, 16, VELOX_WAVE);
  l_i += __shfl_xor(l_i, 32, VELOX_WAVE);
  if (!row_ok) return;
  const float inv = l_i > 0.f ? 1.f / l_i : 1.f;
  const size_t token = (size_t)(q_start + tok);
  if (splits == 1) {
    T* dst = out + (token * nh + head) * D + 4 * g;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[16 * c + j] = from_f32<T>(acc_o[c][j] * inv);
    }
  } else {
    const size_t slot = ((size_t)split * total_tokens + token) * nh + head;
    float* dst = part_o + slot * D + 4 * g;
#pragma unroll
    for (int c = 0; c < NC; ++c) *reinterpret_cast<float4_t*>(dst + 16 * c) = acc_o[c] * inv;
    if (g == 0) part_lse[slot] = l_i > 0.f ? m_i + logf(l_i) : -INFINITY;
  }
}

// out[token, head, :] = sum_s w_s * o_s / sum_s w_s,  w_s = exp(lse_s - max_s lse_s)
template <typename T>
__global__ void merge_splits_kernel(const float* __restrict__ part_o, const float* __restrict__ part_lse, T* __restrict__ out,
                                    int nh, int splits, int total_tokens) {
  const size_t token = blockIdx.x;
  const int head = blockIdx.y;
  float mx = -INFINITY;
  for (int s = 0; s < splits; ++s) mx = fmaxf(mx, part_lse[((size_t)s * total_tokens + token) * nh + head]);
  const float m_safe = (mx == -INFINITY) ? 0.f : mx;
  for (int dd = threadIdx.x; dd < D; dd += blockDim.x) {
    float acc = 0.f, denom = 0.f;
    for (int s = 0; s < splits; ++s) {
      const size_t slot = ((size_t)s * total_tokens + token) * nh + head;
      const float lse = part_lse[slot];
      const float w = (lse == -INFINITY) ? 0.f : expf(lse - m_safe);
      acc += w * part_o[slot * D + dd];
      denom += w;
    }
    out[(token * nh + head) * D + dd] = from_f32<T>(acc / (denom > 0.f ? denom : 1.f));
  }
}

template <typename T> constexpr int tile_keys() { return (sizeof(T) * D > 512) ? 32 : 64; }

template <typename T>
static int launch(const void* qkv, int qkv_stride, const void* k_cache, const void* v_cache, const int* block_tables, int table_width,
                  const int* cu_q, const int* kv_lens, void* out, float* part_o, float* part_lse, int num_seqs, int total_tokens,
                  int max_q_len, int nh, int nkv, int page_shift, float scale, int window, int splits, hipStream_t stream) {
  constexpr int BN = tile_keys<T>();
  const int group = nh / nkv;
  const int row_tiles = (max_q_len * group + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  dim3 grid(row_tiles, nkv, num_seqs * splits);
  paged_attention_kernel<T, BN><<<grid, 256, 0, stream>>>(
      (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
      part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
  int status = (int)hipGetLastError();
  if (status != 0 || splits == 1) return status;
  merge_splits_kernel<T><<<dim3(total_tokens, nh), D < 64 ? 64 : D, 0, stream>>>(part_o, part_lse, (T*)out, nh, splits, total_tokens);
  return (int)hipGetLastError();
}

extern "C" int velox_attention_head_dim() { return D; }

// part_o: float32 [splits, total_tokens, nh, D]; part_lse: float32 [splits, total_tokens, nh]; both unused when splits == 1.
extern "C" int velox_paged_attention(const void* qkv, int qkv_stride, const void* k_cache, const void* v_cache,
                                     const int* block_tables, int table_width, const int* cu_q, const int* kv_lens, void* out,
                                     float* part_o, float* part_lse, int num_seqs, int total_tokens, int max_q_len, int nh, int nkv,
                                     int page_shift, float scale, int window, int splits, int dtype, hipStream_t stream) {
  if (num_seqs <= 0 || total_tokens <= 0) return 0;
  if (nh % nkv != 0 || splits < 1 || page_shift < 0) return -1;
  if (dtype == VELOX_BF16)
    return launch<bf16_t>(qkv, qkv_stride, k_cache, v_cache, block_tables, table_width, cu_q, kv_lens, out, part_o, part_lse, num_seqs,
                          total_tokens, max_q_len, nh, nkv, page_shift, scale, window, splits, stream);
  return launch<float>(qkv, qkv_stride, k_cache, v_cache, block_tables, table_width, cu_q, kv_lens, out, part_o, part_lse, num_seqs,
                       total_tokens, max_q_len, nh, nkv, page_shift, scale, window, splits, stream);
}
