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
#include <type_traits>

#include "common.h"

#ifndef VELOX_HEAD_DIM
#error "build with -DVELOX_HEAD_DIM=<head size>"
#endif

constexpr int D = VELOX_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 between 16 and 256");

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

// ---- the general kernel: portions of prompts, any mix -------------------------------------------------------------
// Contraction blocks.  A lane always holds 16 bytes of a block: bfloat16 blocks have 32 indices (lane (g, i) holds
// 8g .. 8g+7, one v_mfma_f32_16x16x32_bf16 per block), float32 blocks 16 (lane holds 4g .. 4g+3, four
// v_mfma_f32_16x16x4_f32 per block).  Both kinds of operand are one 16-byte LDS read.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

template <typename T> struct Block;
template <> struct Block<bf16_t> {
  static constexpr int KB = 32;
  typedef bf16x8_t Operand;
  static __device__ __forceinline__ float4_t mma(Operand a, Operand b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Block<float> {
  static constexpr int KB = 16;
  typedef float4_t Operand;
  static __device__ __forceinline__ float4_t mma(Operand a, Operand b, float4_t c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
    return c;
  }
};

template <typename T> __device__ __forceinline__ typename Block<T>::Operand load_operand(const T* p) {
  return __builtin_bit_cast(typename Block<T>::Operand, *reinterpret_cast<const float4_t*>(p));
}

// exponent and its unit: a float32 run uses the accurate expf on natural-log scores; a bfloat16 run folds log2(e)
// into the scale and uses the hardware exp2
template <typename T> struct Softmax;
template <> struct Softmax<float> {
  static constexpr float SCALE = 1.f, LN_UNIT = 1.f;
  static __device__ __forceinline__ float exp_of(float x) { return expf(x); }
};
template <> struct Softmax<bf16_t> {
  static constexpr float SCALE = 1.44269504088896340736f, LN_UNIT = 0.69314718055994530942f;
  static __device__ __forceinline__ float exp_of(float x) { return __builtin_amdgcn_exp2f(x); }
};

constexpr int PREFILL_PAGE_IDS = 2048;
// two waves per SIMD hide each other's waits; up to head size 128 the registers allow it without spilling, and the
// compiler is held to it (left alone it takes more registers than one wave per SIMD's worth buys back)
constexpr int GENERAL_MIN_WAVES = D <= 128 ? 2 : 1;

// CT = 16-row tiles per wave, WAVES = waves of a set: a workgroup owns 16 * WAVES * CT rows.  With CT = 2 every K and V^T
// operand read from LDS feeds two matrix instructions, which is what long streams of keys need; a row's arithmetic
// is the same for every CT and WAVES.
// KSPLIT = 2: the workgroup has two sets of 4 waves that own the same rows and take the key tiles alternately, each
// set staging its own tiles; at the end the second set hands its running (maximum, sum, output) to the first
// through LDS.  The longest workgroups of a causal step, which decide how long the step takes, finish in half the time.
template <typename T, int BN, int CT, int KSPLIT, int WAVES = 4>
__global__ void __launch_bounds__(64 * WAVES * KSPLIT) __attribute__((amdgpu_waves_per_eu(GENERAL_MIN_WAVES, WAVES > 4 ? 4 : 2))) paged_attention_kernel(
    const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ cu_q, const int* __restrict__ kv_lens,
    T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_lse,
    int nh, int nkv, int page_shift, float scale, int window, int splits, int total_tokens) {
  typedef Block<T> B;
  typedef typename B::Operand Operand;
  constexpr int KB = B::KB;
  constexpr int VEC = 16 / sizeof(T);           // elements per 16 bytes = indices of a block a lane holds
  constexpr int DP = (D + KB - 1) / KB * KB;    // head size padded to whole blocks (zero columns)
  constexpr int PAD = 16 / sizeof(T);
  constexpr int KS = DP + PAD;                  // row stride of the K tile   [BN][DP]
  constexpr int VS = BN + PAD;                  // row stride of the V^T tile [D][BN]
  constexpr int NT = BN / 16;                   // 16-key tiles of S^T per staged tile
  constexpr int NQB = DP / KB;                  // contraction blocks of Q K^T
  constexpr int NKB = BN / KB;                  // contraction blocks of P V
  constexpr int TPB = KB / 16;                  // S^T tiles per key block
  constexpr int NC = D / 16;                    // 16-channel tiles of the output
  constexpr int SETW = 64 * WAVES;              // threads of a set of waves
  static_assert(KSPLIT == 1 || WAVES == 4, "two sets of waves are sets of four");
  constexpr int ROWS_PER_BLOCK = 16 * WAVES * CT;
  constexpr int TILE_ELEMS = BN * KS + D * VS;                      // one set's K tile and V^T tile
  constexpr int MERGE_FLOATS = KSPLIT > 1 ? 256 * CT * (4 * NC + 2) : 0;  // what the second set hands over at the end
  constexpr int TILE_BYTES = KSPLIT * TILE_ELEMS * (int)sizeof(T);
  constexpr int SMEM_BYTES = TILE_BYTES > 4 * MERGE_FLOATS ? TILE_BYTES : 4 * MERGE_FLOATS;
  __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];
  __shared__ int page_ids[PREFILL_PAGE_IDS];

  const int set = KSPLIT > 1 ? threadIdx.x / 256 : 0;  // which set of 4 waves
  const int tid = KSPLIT > 1 ? threadIdx.x % 256 : threadIdx.x;  // thread within the set
  T* const k_tile = reinterpret_cast<T*>(smem) + set * TILE_ELEMS;
  T* const v_tile = k_tile + BN * KS;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i = lane & 15;
  const int group = nh / nkv;
  // The grid is (sequence and split, KV head, row block), and blockIdx.z counts a sequence's row blocks from its LAST
  // rows, which read the most keys.  Workgroups are handed out in launch order, x fastest, each to the first compute
  // unit with room: the longest of every sequence go first and the short ones fill in as compute units come free.
  // (Measured on MI355X against an order that paired long with short per compute unit, head size 96, 28 heads over 4:
  // 4,096 tokens 179 -> 152 us, 8,192 tokens 594 -> 557, 1,024 tokens 28.9 -> 25.4; 2,048 tokens, whose 448 workgroups are
  // all resident at once, 59.5 -> 62.3.)
  const int b = blockIdx.x / splits, split = blockIdx.x % splits;
  const int kvh = blockIdx.y;
  const int page_size = 1 << page_shift;

  const int q_start = cu_q[b];
  const int q_len = cu_q[b + 1] - q_start;
  const int kv_len = kv_lens[b];
  const int ctx = kv_len - q_len;
  const int rows_total = q_len * group;
  const int blocks_here = (rows_total + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  if ((int)blockIdx.z >= blocks_here) return;
  const int r0 = (blocks_here - 1 - (int)blockIdx.z) * ROWS_PER_BLOCK;

  bool row_ok[CT];
  int tok[CT], head[CT], pos[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int r = r0 + (wave * CT + ct) * 16 + i;
    row_ok[ct] = r < rows_total;
    tok[ct] = row_ok[ct] ? r / group : 0;
    head[ct] = kvh * group + (row_ok[ct] ? r % group : 0);
    pos[ct] = ctx + tok[ct];
  }

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

  // positions of this wave's rows: tiles after the last one are skipped, tiles before the first one need no mask
  int wave_last_pos = -1, wave_first_pos = 0x7fffffff;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (row_ok[ct] && pos[ct] > wave_last_pos) wave_last_pos = pos[ct];
    if (row_ok[ct] && pos[ct] < wave_first_pos) wave_first_pos = pos[ct];
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const int hi = __shfl_xor(wave_last_pos, offset, VELOX_WAVE);
    const int lo = __shfl_xor(wave_first_pos, offset, VELOX_WAVE);
    wave_last_pos = hi > wave_last_pos ? hi : wave_last_pos;
    wave_first_pos = lo < wave_first_pos ? lo : wave_first_pos;
  }

  // Page ids of the keys this workgroup visits are kept in LDS, a window of PREFILL_PAGE_IDS pages at a time (the tile
  // loop moves the window on when the next tile would leave it); zeros go to the padding columns of the K tile.
  const int* table = block_tables + (size_t)b * table_width;
  const int last_key = n_begin + tile_hi * BN < kv_len ? n_begin + tile_hi * BN : kv_len;
  const int last_page = tile_hi > tile_lo ? (last_key - 1) >> page_shift : -1;
  int first_page = (n_begin + tile_lo * BN) >> page_shift;  // first page of the window
  auto load_page_ids = [&]() {
    const int num_pages = last_page - first_page + 1;
    for (int p = threadIdx.x; p < num_pages && p < PREFILL_PAGE_IDS; p += SETW * KSPLIT) page_ids[p] = table[first_page + p];
  };
  load_page_ids();
  if constexpr (DP > D) {
    for (int e = tid; e < BN * (DP - D); e += SETW) k_tile[(e / (DP - D)) * KS + D + e % (DP - D)] = from_f32<T>(0.f);
  }
  auto page_of = [&](int n) -> size_t { return (size_t)page_ids[(n >> page_shift) - first_page]; };

  Operand qf[CT][NQB];
  float m_i[CT], l_i[CT];
  float4_t acc_o[CT][NC];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const T* qp = qkv + (size_t)(q_start + tok[ct]) * qkv_stride + (size_t)head[ct] * D + VEC * g;
#pragma unroll
    for (int cb = 0; cb < NQB; ++cb) {
      const bool inside = row_ok[ct] && (KB * cb + VEC * g < D);
      qf[ct][cb] = inside ? load_operand<T>(qp + KB * cb) : __builtin_bit_cast(Operand, float4_t{0.f, 0.f, 0.f, 0.f});
    }
    m_i[ct] = -INFINITY;
    l_i[ct] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc_o[ct][c] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  const float scale_eff = scale * Softmax<T>::SCALE;

  // ---- staging: global -> registers (issued a tile ahead) -> LDS; what does not change from tile to tile is computed once
  constexpr int VPR = D / VEC;              // vectors per key row of K
  constexpr int VECS = BN * D / VEC;        // vectors per tile (K and V^T alike)
  constexpr int ITERS = (VECS + SETW - 1) / SETW;
  const int run = page_size < BN ? page_size : BN;  // consecutive keys that are contiguous in a page of V
  const bool v_by_vectors = run >= VEC;
  const int run_shift = v_by_vectors ? __builtin_ctz(run / VEC) : 0;  // log2(vectors per run and channel)
  int k_key[ITERS], k_col[ITERS], v_dd[ITERS], v_key[ITERS], v_lds[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int v = tid + it * SETW < VECS ? tid + it * SETW : VECS - 1;  // (the spare threads of a last pass repeat its last vector)
    k_key[it] = v / VPR;
    k_col[it] = (v % VPR) * VEC;
    const int rn = (v >> run_shift) / D;            // run index within the tile
    const int rem = v - ((rn * D) << run_shift);
    v_dd[it] = rem >> run_shift;
    v_key[it] = rn * run + (rem & ((1 << run_shift) - 1)) * VEC;  // first key of the vector, local to the tile
    // column of that key in the V^T tile: inside a block of 32 keys the 8 runs of 4 are interleaved so that lane group g
    // finds the keys of its two S^T tiles side by side (bfloat16 only; float32 blocks hold one tile)
    v_lds[it] = v_dd[it] * VS + v_key[it];
  }
  float4_t k_regs[ITERS], v_regs[ITERS];

  // Every load is issued without a branch around it (a key beyond the sequence is read from the last valid place and
  // zeroed when the tile is written to LDS): a branch per load would make each wait for the one before.
  auto fetch = [&](int n0) {
    const T* k_src[ITERS];
    const T* v_src[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      int nk = n0 + k_key[it];
      nk = nk < kv_len ? nk : kv_len - 1;
      k_src[it] = k_cache + (((page_of(nk) * nkv + kvh) << page_shift) + (nk & (page_size - 1))) * D + k_col[it];
      int nv = n0 + v_key[it];
      nv = nv < kv_len ? nv : (kv_len - 1) & ~(VEC - 1);
      v_src[it] = v_cache + (((page_of(nv) * nkv + kvh) * D + v_dd[it]) << page_shift) + (nv & (page_size - 1));
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) k_regs[it] = *reinterpret_cast<const float4_t*>(k_src[it]);
    if (v_by_vectors) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) v_regs[it] = *reinterpret_cast<const float4_t*>(v_src[it]);
    }
  };
  auto commit = [&](int n0) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      if constexpr (VECS % SETW != 0) {
        if (tid + it * SETW >= VECS) continue;
      }
      if (n0 + k_key[it] >= kv_len) k_regs[it] = float4_t{0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<float4_t*>(k_tile + k_key[it] * KS + k_col[it]) = k_regs[it];
      if (v_by_vectors) {
        if (n0 + v_key[it] + VEC > kv_len) {
          Vec16<T> x;
          x.v = v_regs[it];
          mask_tail(x, kv_len - n0 - v_key[it]);
          v_regs[it] = x.v;
        }
        if constexpr (KB == 32) {
          // keys 8m .. 8m+7 of a 32-key block: the first four belong to lane group (2m) % 4 of S^T tile (2m) / 4, the
          // next four to lane group (2m+1) % 4 of tile (2m+1) / 4; lane group g's column run is 8g + 4 * tile
          const int base = v_dd[it] * VS + (v_key[it] & ~31);
          const int m = (v_key[it] & 31) >> 3;
          const int q0 = 2 * m, q1 = 2 * m + 1;  // quads of 4 keys
          typedef float float2_t __attribute__((ext_vector_type(2)));
          *reinterpret_cast<float2_t*>(v_tile + base + 8 * (q0 & 3) + 4 * (q0 >> 2)) = float2_t{v_regs[it][0], v_regs[it][1]};
          *reinterpret_cast<float2_t*>(v_tile + base + 8 * (q1 & 3) + 4 * (q1 >> 2)) = float2_t{v_regs[it][2], v_regs[it][3]};
        } else {
          *reinterpret_cast<float4_t*>(v_tile + v_lds[it]) = v_regs[it];
        }
      }
    }
    if (!v_by_vectors) {  // pages shorter than a vector: element by element, straight from global memory
      const int per = D * run;
      for (int v = tid; v < BN * D; v += SETW) {
        const int rn = v / per, rem = v % per;
        const int dd = rem / run, e = rem % run;
        const int nl = rn * run + e;
        const int n = n0 + nl;
        T x = from_f32<T>(0.f);
        if (n < kv_len) x = v_cache[((page_of(n) * nkv + kvh) * D + dd) * page_size + (n & (page_size - 1))];
        int col = nl;
        if constexpr (KB == 32) {
          const int quad = (nl & 31) >> 2;
          col = (nl & ~31) + 8 * (quad & 3) + 4 * (quad >> 2) + (nl & 3);
        }
        v_tile[dd * VS + col] = x;
      }
    }
  };

  __syncthreads();  // page ids are in place
  // iteration `it` covers tiles tile_lo + it * KSPLIT .. + KSPLIT - 1, one per set (the last iteration may leave a set without one)
  const int iterations = tile_hi > tile_lo ? (tile_hi - tile_lo + KSPLIT - 1) / KSPLIT : 0;
  if (tile_lo + set < tile_hi) fetch(n_begin + (tile_lo + set) * BN);
  for (int it = 0; it < iterations; ++it) {
    const int tile = tile_lo + it * KSPLIT + set;
    const bool have_tile = KSPLIT == 1 || tile < tile_hi;
    const int n0 = n_begin + tile * BN;
    __syncthreads();  // the previous tile has been read by every wave
    if (have_tile) commit(n0);
    __syncthreads();
    if (it + 1 < iterations) {
      const int next_first = n_begin + (tile_lo + (it + 1) * KSPLIT) * BN;  // first key of the next iteration's tiles
      if (((next_first + KSPLIT * BN - 1) >> page_shift) - first_page >= PREFILL_PAGE_IDS) {  // the same for every thread
        first_page = next_first >> page_shift;
        load_page_ids();
        __syncthreads();
      }
      if (tile + KSPLIT < tile_hi) fetch(n0 + KSPLIT * BN);  // in flight while this tile is computed
    }
    if (!have_tile || n0 > wave_last_pos) continue;  // nothing this wave may read; it still took part in the staging

    // ---- S^T = K Q^T ----------------------------------------------------------------------
    // bfloat16: the operands of the next 16 keys are asked for before this 16 keys' matrix instructions are issued, and
    // the compiler is kept from moving each read down to just before its use (a read from LDS takes longer than the
    // matrix instructions it feeds: 2,048 to 8,192 tokens 2-4% faster).  float32 operands and heads beyond 128 channels
    // are too many registers for it.
    constexpr int KEYS_AHEAD = (sizeof(T) == 2 && D <= 128) ? 1 : 0;
    float4_t s[CT][NT];
    Operand kf[KEYS_AHEAD + 1][NQB];
    if constexpr (KEYS_AHEAD > 0) {
#pragma unroll
      for (int cb = 0; cb < NQB; ++cb) kf[0][cb] = load_operand<T>(k_tile + i * KS + KB * cb + VEC * g);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (KEYS_AHEAD > 0) {
        if (t + 1 < NT) {
#pragma unroll
          for (int cb = 0; cb < NQB; ++cb) kf[(t + 1) & 1][cb] = load_operand<T>(k_tile + (16 * (t + 1) + i) * KS + KB * cb + VEC * g);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) s[ct][t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int cb = 0; cb < NQB; ++cb) {
        if constexpr (KEYS_AHEAD == 0) kf[0][cb] = load_operand<T>(k_tile + (16 * t + i) * KS + KB * cb + VEC * g);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) s[ct][t] = B::mma(kf[t & KEYS_AHEAD][cb], qf[ct][cb], s[ct][t]);
      }
    }
    // ---- scale, mask (only where the tile crosses a row's limits), running maximum ----------
    const bool whole = n0 + BN <= kv_len && n0 + BN - 1 <= wave_first_pos && (window <= 0 || n0 > wave_last_pos - window);
    float alpha[CT];
    Operand pf[CT][NKB];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      // the scale (positive) is applied inside the exponent's argument: the maximum is taken over the raw scores
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[ct][t][j]);
      } else {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = n0 + 16 * t + 4 * g + j;
            const bool keep = row_ok[ct] && n < kv_len && n <= pos[ct] && (window <= 0 || n > pos[ct] - window);
            s[ct][t][j] = keep ? s[ct][t][j] : -INFINITY;
            mx = fmaxf(mx, s[ct][t][j]);
          }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, VELOX_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, VELOX_WAVE));
      const float m_new = fmaxf(m_i[ct], mx * scale_eff);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      alpha[ct] = (m_i[ct] == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_i[ct] - m_safe);
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        Vec16<T> packed;
        T* e = reinterpret_cast<T*>(&packed.v);
#pragma unroll
        for (int u = 0; u < TPB; ++u)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // a masked score is -inf and gives exp(-inf) = 0; m_safe is finite
            const float p = Softmax<T>::exp_of(fmaf(s[ct][kb * TPB + u][j], scale_eff, -m_safe));
            psum += p;
            e[4 * u + j] = from_f32<T>(p);
          }
        pf[ct][kb] = __builtin_bit_cast(Operand, packed.v);
      }
      l_i[ct] = l_i[ct] * alpha[ct] + psum;  // partial over this lane's keys; the four lane groups are summed at the end
      m_i[ct] = m_new;
    }
    // ---- O^T = O^T * alpha + V^T P^T ------------------------------------------------------
    constexpr int TILES_AHEAD = (sizeof(T) == 2 && D <= 128 && NC > 2) ? 2 : 0;  // channel tiles whose operands are in flight ahead of the one being multiplied
    Operand vf[TILES_AHEAD + 1][NKB];
#pragma unroll
    for (int a = 0; a < TILES_AHEAD; ++a)
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) vf[a][kb] = load_operand<T>(v_tile + (16 * a + i) * VS + KB * kb + VEC * g);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if constexpr (TILES_AHEAD > 0) {
        if (c + TILES_AHEAD < NC) {
#pragma unroll
          for (int kb = 0; kb < NKB; ++kb) vf[(c + TILES_AHEAD) % (TILES_AHEAD + 1)][kb] = load_operand<T>(v_tile + (16 * (c + TILES_AHEAD) + i) * VS + KB * kb + VEC * g);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) acc_o[ct][c] = acc_o[ct][c] * alpha[ct];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        if constexpr (TILES_AHEAD == 0) vf[0][kb] = load_operand<T>(v_tile + (16 * c + i) * VS + KB * kb + VEC * g);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc_o[ct][c] = B::mma(vf[c % (TILES_AHEAD + 1)][kb], pf[ct][kb], acc_o[ct][c]);
      }
    }
  }

  if constexpr (KSPLIT > 1) {
    // the second set's state goes through LDS (the tiles are no longer needed) and is folded into the first set's
    __syncthreads();
    float4_t* const hand_acc = reinterpret_cast<float4_t*>(smem);
    float* const hand_ml = reinterpret_cast<float*>(smem) + 256 * CT * NC * 4;
    if (set == 1) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
        for (int c = 0; c < NC; ++c) hand_acc[(ct * NC + c) * 256 + tid] = acc_o[ct][c];
        hand_ml[ct * 256 + tid] = m_i[ct];
        hand_ml[(CT + ct) * 256 + tid] = l_i[ct];
      }
    }
    __syncthreads();
    if (set == 1) return;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float m_other = hand_ml[ct * 256 + tid], l_other = hand_ml[(CT + ct) * 256 + tid];
      const float m_new = fmaxf(m_i[ct], m_other);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float mine = (m_i[ct] == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_i[ct] - m_safe);
      const float theirs = (m_other == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_other - m_safe);
      l_i[ct] = l_i[ct] * mine + l_other * theirs;
      m_i[ct] = m_new;
#pragma unroll
      for (int c = 0; c < NC; ++c) acc_o[ct][c] = acc_o[ct][c] * mine + hand_acc[(ct * NC + c) * 256 + tid] * theirs;
    }
  }

#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float l = l_i[ct];
    l += __shfl_xor(l, 16, VELOX_WAVE);
    l += __shfl_xor(l, 32, VELOX_WAVE);
    if (!row_ok[ct]) continue;
    const float inv = l > 0.f ? 1.f / l : 1.f;
    const size_t token = (size_t)(q_start + tok[ct]);
    if (splits == 1) {
      T* dst = out + (token * nh + head[ct]) * D + 4 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[16 * c + j] = from_f32<T>(acc_o[ct][c][j] * inv);
      }
    } else {
      const size_t slot = ((size_t)split * total_tokens + token) * nh + head[ct];
      float* dst = part_o + slot * D + 4 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) *reinterpret_cast<float4_t*>(dst + 16 * c) = acc_o[ct][c] * inv;
      if (g == 0) part_lse[slot] = l > 0.f ? m_i[ct] * Softmax<T>::LN_UNIT + logf(l) : -INFINITY;
    }
  }
}

// ---- portions of prompts, bfloat16, tiles brought into LDS by the memory system itself ---------------------------------
// The same arithmetic as the general kernel with CT row tiles per wave, for head sizes of 64 and 128 channels and pages
// of at least 8 tokens.  What differs is how a tile of 64 keys gets into LDS: every lane asks for 16 bytes of the
// cache with a load that writes LDS directly (no registers, no LDS write instructions, no address arithmetic on the
// way back), a whole tile AHEAD of the one being multiplied, into the other of two tile buffers.  One barrier per tile
// is left: behind it every wave has read the buffer that the next loads overwrite and this tile has landed.
//
// Such a load puts lane l's 16 bytes at (wave-uniform base) + 16 l, so an instruction fills one contiguous kilobyte
// and what lies where in LDS is decided by which piece of the cache each lane asks for.  Pieces are placed so that
// the operand reads are free of bank conflicts without padding: a K row (2 D bytes) keeps its place and its 16-byte
// pieces are exchanged among themselves, piece c of key k sits at place c ^ f(k) with f(k) = (k & 3) | ((k >> 3) & 1) << 2;
// a V^T row (128 bytes: 64 keys of one channel) likewise, piece c of channel d sits at place c ^ (d & 7).  Any eight
// lanes that read together (consecutive rows, the same piece) then touch eight different places.
//
// S^T tiles take their keys in another order than the general kernel: tile u of key block b (32 keys), row 4 q + j
// (q = 0..3, j = 0..3) is key 32 b + 8 q + 4 u + j.  Lane group g then holds, over the block's two tiles, the scores
// of keys 8 g .. 8 g + 7 of the block: eight consecutive keys, which is one 16-byte piece of a V^T row in its natural
// order.  (The general kernel reorders V^T instead, in pieces of 8 bytes; a direct load cannot.)  For such a row of K
// f(k) is i & 7 for lane i: a constant of the lane.
__device__ __attribute__((aligned(16))) const unsigned int zero_piece[4] = {0u, 0u, 0u, 0u};

// KSPLIT = 2: two sets of WAVES waves own the same rows and take the key tiles alternately, each set with tile buffers of
// its own; at the end the second set hands its running (maximum, sum, output) to the first through LDS.  The longest
// workgroups of a causal step, the rows at the end of a prompt, which decide how long the step takes, then walk half
// as many tiles one after the other.
template <int CT, int WAVES, int KSPLIT = 1>
__global__ void __launch_bounds__(64 * WAVES * KSPLIT) __attribute__((amdgpu_waves_per_eu(2, 2))) direct_attention_kernel(
    const bf16_t* __restrict__ qkv, int qkv_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ cu_q, const int* __restrict__ kv_lens,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_lse,
    int nh, int nkv, int page_shift, float scale, int window, int splits, int total_tokens) {
  typedef bf16_t T;
  typedef Block<T> B;
  typedef typename B::Operand Operand;
  static_assert(CT > 0 && (D == 64 || D == 128), "head sizes whose rows are a power of two of 16-byte pieces, at least eight");
  constexpr int BN = 64, KB = 32, VEC = 8;
  constexpr int NT = BN / 16, NQB = D / KB, NKB = BN / KB, NC = D / 16;
  constexpr int CPR = D / 8;                        // 16-byte pieces of a K row
  constexpr int TILE_BYTES = BN * D * 2;            // K tile and V^T tile alike
  constexpr int LOADS = TILE_BYTES / 1024;          // load instructions per tile and operand
  static_assert(LOADS % WAVES == 0, "every wave issues the same number of loads");
  constexpr int LPW = LOADS / WAVES;
  constexpr int ROWS_PER_BLOCK = 16 * WAVES * CT;
  constexpr int SETW = 64 * WAVES;                  // threads of a set of waves
  constexpr int MERGE_BYTES = KSPLIT > 1 ? 4 * SETW * CT * (4 * NC + 2) : 0;  // what the second set hands over at the end
  static_assert(MERGE_BYTES <= KSPLIT * 4 * TILE_BYTES, "the hand-over fits into the tile buffers");
  __shared__ __attribute__((aligned(1024))) char smem_all[KSPLIT][2][2 * TILE_BYTES];
  __shared__ int page_ids[PREFILL_PAGE_IDS];

  const int set = KSPLIT > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x / SETW) : 0;  // which set of waves
  const int tid = KSPLIT > 1 ? threadIdx.x % SETW : threadIdx.x;                         // thread within the set
  char (*const smem)[2 * TILE_BYTES] = smem_all[set];
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int group = nh / nkv;
  // The grid is (sequence and split, KV head, row block), and blockIdx.z counts a sequence's row blocks from its LAST
  // rows, which read the most keys.  Workgroups are handed out in launch order, x fastest, each to the first compute
  // unit with room: the longest of every sequence go first and the short ones fill in as compute units come free
  // (against an order that paired long with short per compute unit, measured on MI355X: 2,048 tokens 62.4 -> 52.8 us,
  // 4,096 tokens 169 -> 146, 8,192 tokens 559 -> 528).
  const int b = blockIdx.x / splits, split = blockIdx.x % splits;
  const int kvh = blockIdx.y;
  const int page_size = 1 << page_shift;

  const int q_start = cu_q[b];
  const int q_len = cu_q[b + 1] - q_start;
  const int kv_len = kv_lens[b];
  const int ctx = kv_len - q_len;
  const int rows_total = q_len * group;
  const int blocks_here = (rows_total + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  if ((int)blockIdx.z >= blocks_here) return;
  const int r0 = (blocks_here - 1 - (int)blockIdx.z) * ROWS_PER_BLOCK;

  bool row_ok[CT];
  int tok[CT], head[CT], pos[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int r = r0 + (wave * CT + ct) * 16 + i;
    row_ok[ct] = r < rows_total;
    tok[ct] = row_ok[ct] ? r / group : 0;
    head[ct] = kvh * group + (row_ok[ct] ? r % group : 0);
    pos[ct] = ctx + tok[ct];
  }
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

  int wave_last_pos = -1, wave_first_pos = 0x7fffffff;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (row_ok[ct] && pos[ct] > wave_last_pos) wave_last_pos = pos[ct];
    if (row_ok[ct] && pos[ct] < wave_first_pos) wave_first_pos = pos[ct];
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const int hi = __shfl_xor(wave_last_pos, offset, VELOX_WAVE);
    const int lo = __shfl_xor(wave_first_pos, offset, VELOX_WAVE);
    wave_last_pos = hi > wave_last_pos ? hi : wave_last_pos;
    wave_first_pos = lo < wave_first_pos ? lo : wave_first_pos;
  }

  // page ids of the keys this workgroup visits, a window of PREFILL_PAGE_IDS pages at a time
  const int* table = block_tables + (size_t)b * table_width;
  const int last_key = n_begin + tile_hi * BN < kv_len ? n_begin + tile_hi * BN : kv_len;
  const int last_page = tile_hi > tile_lo ? (last_key - 1) >> page_shift : -1;
  int first_page = (n_begin + tile_lo * BN) >> page_shift;
  auto load_page_ids = [&]() {
    const int num_pages = last_page - first_page + 1;
    for (int p = threadIdx.x; p < num_pages && p < PREFILL_PAGE_IDS; p += SETW * KSPLIT) page_ids[p] = table[first_page + p];
  };
  load_page_ids();
  auto page_of = [&](int n) -> size_t { return (size_t)page_ids[(n >> page_shift) - first_page]; };

  Operand qf[CT][NQB];
  float m_i[CT], l_i[CT];
  float4_t acc_o[CT][NC];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const T* qp = qkv + (size_t)(q_start + tok[ct]) * qkv_stride + (size_t)head[ct] * D + VEC * g;
#pragma unroll
    for (int cb = 0; cb < NQB; ++cb)
      qf[ct][cb] = row_ok[ct] ? load_operand<T>(qp + KB * cb) : __builtin_bit_cast(Operand, float4_t{0.f, 0.f, 0.f, 0.f});
    m_i[ct] = -INFINITY;
    l_i[ct] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc_o[ct][c] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  const float scale_eff = scale * Softmax<T>::SCALE;

  // ---- what each lane asks for: load instruction q = wave + WAVES * m of a tile fills bytes [1024 q, 1024 q + 1024) of
  // the K part (or the V^T part) of a buffer; lane l's 16 bytes are piece s = 64 q + l of the tile
  int k_key[LPW], k_col[LPW], v_chan[LPW];
  int v_key;
#pragma unroll
  for (int m = 0; m < LPW; ++m) {
    const int s = 64 * (wave + WAVES * m) + lane;
    const int key = s / CPR, place = s % CPR;
    k_key[m] = key;
    k_col[m] = 8 * (place ^ ((key & 3) | (((key >> 3) & 1) << 2)));
    v_chan[m] = s / 8;
  }
  v_key = 8 * ((lane & 7) ^ ((lane >> 3) & 7));  // (the channel's low bits are the lane's: 64 q is a multiple of 8 channels)
  // A tile that lies wholly inside the sequence, which is every tile but a sequence's last, takes the short way.  The
  // keys of one load instruction (64 / CPR consecutive ones, at a multiple of as many) lie in one page, since a page
  // holds at least 8: their page's address is the same for the whole wave and is worked out in scalar registers, and a
  // lane's offset from it never changes.  A lane's eight values of a channel lie in one page too; its page differs
  // from other lanes', but is the same for all of the wave's loads of a tile, which are 8 WAVES channels apart.
  constexpr int KEYS_PER_LOAD = 64 / CPR;
  const uint32_t k_lane_bytes = (uint32_t)(((lane / CPR) * D + k_col[0]) * 2);
  const size_t v_page_elems = ((size_t)nkv * D) << page_shift;
  const uint32_t v_lane_elems = ((uint32_t)(kvh * D + 8 * wave + (lane >> 3))) << page_shift;
  auto issue = [&](int tile_n0, int tile_buffer) {
    // (both are the same for the whole wave; said so, or the compiler keeps them and all that follows from them in
    // vector registers)
    const int n0 = __builtin_amdgcn_readfirstlane(tile_n0), buffer = __builtin_amdgcn_readfirstlane(tile_buffer);
    char* const k_dst = smem[buffer];
    char* const v_dst = smem[buffer] + TILE_BYTES;
    if (n0 + BN <= kv_len) {  // (the same for every thread)
      // (all page ids first: the loads below are barriers to the compiler's reordering, and each id is a trip to LDS)
      const int window_first = __builtin_amdgcn_readfirstlane(first_page);
      const int nv = n0 + v_key;
      const size_t v_page = page_of(nv);
      size_t k_page[LPW];
#pragma unroll
      for (int m = 0; m < LPW; ++m)
        k_page[m] = (size_t)__builtin_amdgcn_readfirstlane(page_ids[((n0 + KEYS_PER_LOAD * (wave + WAVES * m)) >> page_shift) - window_first]);
#pragma unroll
      for (int m = 0; m < LPW; ++m) {
        const int key0 = n0 + KEYS_PER_LOAD * (wave + WAVES * m);
        const T* base = k_cache + (((k_page[m] * nkv + kvh) << page_shift) + (key0 & (page_size - 1))) * D;
        load_to_lds_16(base, k_lane_bytes, k_dst + 1024 * (wave + WAVES * m));
      }
      const T* v_src = v_cache + v_page * v_page_elems + (v_lane_elems + (uint32_t)(nv & (page_size - 1)));
#pragma unroll
      for (int m = 0; m < LPW; ++m) load_to_lds_16(v_src + ((size_t)(8 * WAVES * m) << page_shift), v_dst + 1024 * (wave + WAVES * m));
      return;
    }
#pragma unroll
    for (int m = 0; m < LPW; ++m) {
      int nk = n0 + k_key[m];
      nk = nk < kv_len ? nk : kv_len - 1;  // (a key beyond the sequence: any valid address; its scores are masked)
      const T* src = k_cache + (((page_of(nk) * nkv + kvh) << page_shift) + (nk & (page_size - 1))) * D + k_col[m];
      load_to_lds_16(src, k_dst + 1024 * (wave + WAVES * m));
    }
#pragma unroll
    for (int m = 0; m < LPW; ++m) {
      // Values beyond the sequence are whatever the page holds, and even a probability of zero times an infinity is
      // no zero: a piece that lies wholly beyond the sequence is taken from a piece of zeros instead (the piece that the
      // sequence ends in is cleaned up in LDS, below)
      const int nv = n0 + v_key;
      const bool beyond = nv >= kv_len;
      const int nc = beyond ? (kv_len - 1) & ~7 : nv;
      const T* src = v_cache + (((page_of(nc) * nkv + kvh) * D + v_chan[m]) << page_shift) + (nc & (page_size - 1));
      load_to_lds_16(beyond ? reinterpret_cast<const T*>(zero_piece) : src, v_dst + 1024 * (wave + WAVES * m));
    }
  };

  // ---- where each lane reads its operands.  K: row 8 (i / 4) + (i % 4) of a key block (+ 4 u for tile u, + 32 b for
  // block b), piece (4 cb + g) ^ (i & 7) = 4 (cb ^ h) + (g ^ (i & 3)) with h = (i / 4) & 1.  V^T: row i of a channel
  // tile, piece (4 kb + g) ^ (i & 7) likewise.
  const int h = (i >> 2) & 1;
  const int k_row_bytes = (8 * (i >> 2) + (i & 3)) * (2 * D) + 16 * (g ^ (i & 3));
  const int k_even = k_row_bytes + 64 * h, k_odd = k_row_bytes + 64 * (1 - h);           // cb even / odd: + 128 (cb / 2)
  const int v_row_bytes = TILE_BYTES + i * 128 + 16 * (g ^ (i & 3));
  const int v_first = v_row_bytes + 64 * h, v_second = v_row_bytes + 64 * (1 - h);       // kb = 0 / 1

  // (the queries have arrived before the loop, said in a way the compiler sees: it would otherwise wait for them, and with
  // them for every load in flight, at their first use in every round of the loop)
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();  // page ids are in place
  // round `it` covers tiles tile_lo + it * KSPLIT .. + KSPLIT - 1, one per set (the last round may leave a set without one)
  const int rounds = tile_hi > tile_lo ? (tile_hi - tile_lo + KSPLIT - 1) / KSPLIT : 0;
  if (tile_lo + set < tile_hi) issue(n_begin + (tile_lo + set) * BN, 0);
  int buffer = 0;
  for (int it = 0; it < rounds; ++it, buffer ^= 1) {
    const int tile = tile_lo + it * KSPLIT + set;
    const bool have_tile = KSPLIT == 1 || tile < tile_hi;
    const int n0 = n_begin + tile * BN;
    wait_for_loads<0>();                  // this wave's pieces of the tile have landed
    __syncthreads();                      // everybody's have, and everybody is done with the other buffer
    if (it + 1 < rounds) {
      const int next_first = n_begin + (tile_lo + (it + 1) * KSPLIT) * BN;  // first key of the next round's tiles
      if (((next_first + KSPLIT * BN - 1) >> page_shift) - first_page >= PREFILL_PAGE_IDS) {  // the same for every thread
        first_page = next_first >> page_shift;
        __syncthreads();
        load_page_ids();
        __syncthreads();
      }
      if (tile + KSPLIT < tile_hi) issue(n0 + KSPLIT * BN, buffer ^ 1);
    }
    // the sequence's last tile, if it is one of this round's and the sequence ends inside a piece of eight keys (the same
    // answer for every thread; once per sequence and workgroup): what follows the last key in that piece is zeroed in LDS
    const int last_tile = (kv_len - 1 - n_begin) / BN;
    if ((kv_len & 7) != 0 && last_tile >= tile_lo + it * KSPLIT && last_tile < tile_lo + (it + 1) * KSPLIT && last_tile < tile_hi) {
      if (tile == last_tile) {
        const int piece = (kv_len - n0) >> 3, valid = (kv_len - n0) & 7;
        for (int channel = tid; channel < D; channel += SETW) {
          float4_t* const at = reinterpret_cast<float4_t*>(smem[buffer] + TILE_BYTES + channel * 128 + 16 * (piece ^ (channel & 7)));
          Vec16<T> x;
          x.v = *at;
          mask_tail(x, valid);
          *at = x.v;
        }
      }
      __syncthreads();
    }
    if (!have_tile) continue;
    if (n0 > wave_last_pos) continue;  // nothing this wave may read
    const char* const tile_base = smem[buffer];

    // ---- S^T = K Q^T: tile t = 2 b + u of the 64 keys ----------------------------------------
    float4_t s[CT][NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      Operand kf[NQB > 0 ? NQB : 1];  // (the template is parsed for every head size, run for 64 and 128)
      const int tile_bytes = (32 * (t >> 1) + 4 * (t & 1)) * (2 * D);
#pragma unroll
      for (int cb = 0; cb < NQB; ++cb)
        kf[cb] = __builtin_bit_cast(Operand, *reinterpret_cast<const float4_t*>(tile_base + ((cb & 1) ? k_odd : k_even) + 128 * (cb >> 1) + tile_bytes));
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) s[ct][t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int cb = 0; cb < NQB; ++cb)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) s[ct][t] = B::mma(kf[cb], qf[ct][cb], s[ct][t]);
    }
    // ---- scale, mask (only where the tile crosses a row's limits), running maximum ----------
    const bool whole = n0 + BN <= kv_len && n0 + BN - 1 <= wave_first_pos && (window <= 0 || n0 > wave_last_pos - window);
    float alpha[CT];
    Operand pf[CT][NKB];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[ct][t][j]);
      } else {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = n0 + 32 * (t >> 1) + 8 * g + 4 * (t & 1) + j;
            const bool keep = row_ok[ct] && n < kv_len && n <= pos[ct] && (window <= 0 || n > pos[ct] - window);
            s[ct][t][j] = keep ? s[ct][t][j] : -INFINITY;
            mx = fmaxf(mx, s[ct][t][j]);
          }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, VELOX_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, VELOX_WAVE));
      // The reference of a row's exponents need not be its maximum: any number the scores do not exceed by much will do,
      // the sums and the output are relative to it all the same and the final division takes it out.  It is moved (and
      // everything gathered so far rescaled) only when a score lies more than REFERENCE_SLACK above it, in units of the
      // exponent (powers of two): probabilities then stay below 2^REFERENCE_SLACK, far inside the range of both number
      // formats, and after a row's first tile the rescaling is the exception.
      constexpr float REFERENCE_SLACK = 8.f;
      const float top = mx * scale_eff;
      const bool stays = top - m_i[ct] <= REFERENCE_SLACK;  // (false while the row has seen no key: -inf)
      const float m_new = stays ? m_i[ct] : top;
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      alpha[ct] = stays ? 1.f : ((m_i[ct] == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_i[ct] - m_safe));
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        Vec16<T> packed;
        T* e = reinterpret_cast<T*>(&packed.v);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p = Softmax<T>::exp_of(fmaf(s[ct][kb * 2 + u][j], scale_eff, -m_safe));
            psum += p;
            e[4 * u + j] = from_f32<T>(p);
          }
        pf[ct][kb] = __builtin_bit_cast(Operand, packed.v);
      }
      l_i[ct] = l_i[ct] * alpha[ct] + psum;
      m_i[ct] = m_new;
    }
    // ---- O^T = O^T * alpha + V^T P^T --------------------------------------------------------
    constexpr int AHEAD = 1;  // channel tiles whose operands are in flight ahead of the one being multiplied
    Operand vf[AHEAD + 1][NKB];
    auto read_values = [&](int c, Operand (&into)[NKB]) {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) into[kb] = __builtin_bit_cast(Operand, *reinterpret_cast<const float4_t*>(tile_base + (kb ? v_second : v_first) + 2048 * c));
    };
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) read_values(a, vf[a]);
    // The kernel is bound by the vector instructions it issues, and the output's rescaling is 64 of a tile's 400: it is
    // left out when no row of the wave saw its maximum move (nearly always, a few tiles into a row's keys).
    bool moved = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) moved = moved || alpha[ct] != 1.f;
    if (__ballot(moved) != 0ull) {
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc_o[ct][c] = acc_o[ct][c] * alpha[ct];
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (c + AHEAD < NC) read_values(c + AHEAD, vf[(c + AHEAD) % (AHEAD + 1)]);
      if constexpr (AHEAD > 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc_o[ct][c] = B::mma(vf[c % (AHEAD + 1)][kb], pf[ct][kb], acc_o[ct][c]);
    }
  }

  if constexpr (KSPLIT > 1) {
    // the second set's state goes through LDS (the tiles are no longer needed) and is folded into the first set's
    __syncthreads();
    float4_t* const hand_acc = reinterpret_cast<float4_t*>(&smem_all[0][0][0]);
    float* const hand_ml = reinterpret_cast<float*>(&smem_all[0][0][0]) + SETW * CT * NC * 4;
    if (set == 1) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
        for (int c = 0; c < NC; ++c) hand_acc[(ct * NC + c) * SETW + tid] = acc_o[ct][c];
        hand_ml[ct * SETW + tid] = m_i[ct];
        hand_ml[(CT + ct) * SETW + tid] = l_i[ct];
      }
    }
    __syncthreads();
    if (set == 1) return;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float m_other = hand_ml[ct * SETW + tid], l_other = hand_ml[(CT + ct) * SETW + tid];
      const float m_new = fmaxf(m_i[ct], m_other);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float mine = (m_i[ct] == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_i[ct] - m_safe);
      const float theirs = (m_other == -INFINITY) ? 0.f : Softmax<T>::exp_of(m_other - m_safe);
      l_i[ct] = l_i[ct] * mine + l_other * theirs;
      m_i[ct] = m_new;
#pragma unroll
      for (int c = 0; c < NC; ++c) acc_o[ct][c] = acc_o[ct][c] * mine + hand_acc[(ct * NC + c) * SETW + tid] * theirs;
    }
  }

#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float l = l_i[ct];
    l += __shfl_xor(l, 16, VELOX_WAVE);
    l += __shfl_xor(l, 32, VELOX_WAVE);
    if (!row_ok[ct]) continue;
    const float inv = l > 0.f ? 1.f / l : 1.f;
    const size_t token = (size_t)(q_start + tok[ct]);
    if (splits == 1) {
      T* dst = out + (token * nh + head[ct]) * D + 4 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[16 * c + j] = from_f32<T>(acc_o[ct][c][j] * inv);
      }
    } else {
      const size_t slot = ((size_t)split * total_tokens + token) * nh + head[ct];
      float* dst = part_o + slot * D + 4 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) *reinterpret_cast<float4_t*>(dst + 16 * c) = acc_o[ct][c] * inv;
      if (g == 0) part_lse[slot] = l > 0.f ? m_i[ct] * Softmax<T>::LN_UNIT + logf(l) : -INFINITY;
    }
  }
}

// Zeroes the elements of a 4-key fragment whose key index is not below `valid`.
__device__ __forceinline__ void mask_frag(Frag<float>& f, int valid) {
#pragma unroll
  for (int j = 0; j < 4; ++j) f.v[j] = j < valid ? f.v[j] : 0.f;
}
__device__ __forceinline__ void mask_frag(Frag<bf16_t>& f, int valid) {
#pragma unroll
  for (int j = 0; j < 4; ++j) f.v[j] = j < valid ? f.v[j] : (short)0;
}

// Decode: every sequence brings one token, and the G <= 16 query heads of a KV head are the 16 columns of the
// MFMA tiles.  The step is bound by reading the cache once, so nothing is staged: each wave streams its own
// 16-key tiles straight from global memory into MFMA operands (K rows as [key i][channels 16c + 4g ..], or
// [channels 32c + 8g ..] where KeyOps below allows, V^T rows as [channel 16c + i][keys 4g ..], 8- or 16-byte loads of
// contiguous cache lines), two tiles ahead of the
// arithmetic, with no barrier in the loop.  The page ids of the workgroup's key range are copied into LDS first, so
// that a tile's addresses do not wait for a second trip to memory.  The WAVES waves of a workgroup interleave the
// tiles of one (sequence, KV head, split) and merge their running (max, sum, output) through LDS at the end.
constexpr int DECODE_PAGE_IDS = 2048;

// Operands of S^T = K Q^T in the decode kernel.  For bfloat16 heads of a multiple of 32 channels a lane reads 16 bytes of
// its key's row (channels 32c + 8g ..) and one v_mfma_f32_16x16x32_bf16 takes them: half as many loads, each touching
// half as many cache lines, as with the 16-channel fragments that every other case uses.
template <typename T, bool WIDE> struct KeyOps {
  static constexpr int STEPS = D / 16, SPAN = 16, LANE = 4;
  typedef Frag<T> Operand;
  static __device__ __forceinline__ Operand load(const T* p) { return load_frag<T>(p); }
  static __device__ __forceinline__ Operand zero() { return zero_frag<T>(); }
  static __device__ __forceinline__ float4_t mma(const Operand& a, const Operand& b, float4_t c) { return mma16(a, b, c); }
};
template <> struct KeyOps<bf16_t, true> {
  static constexpr int STEPS = D / 32, SPAN = 32, LANE = 8;
  typedef bf16x8_t Operand;
  static __device__ __forceinline__ Operand load(const bf16_t* p) { return *reinterpret_cast<const bf16x8_t*>(p); }
  static __device__ __forceinline__ Operand zero() { return __builtin_bit_cast(bf16x8_t, float4_t{0.f, 0.f, 0.f, 0.f}); }
  static __device__ __forceinline__ float4_t mma(const Operand& a, const Operand& b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

template <typename T, int DEPTH, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) decode_attention_kernel(
    const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ kv_lens,
    T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_lse,
    int nh, int nkv, int page_shift, float scale, int window, int splits, int total_tokens) {
  constexpr int NC = D / 16;
  constexpr int NCW = (NC + WAVES - 1) / WAVES;
  typedef KeyOps<T, sizeof(T) == 2 && D % 32 == 0> KO;
  __shared__ __attribute__((aligned(16))) float4_t acc_all[WAVES * NC * 64];
  __shared__ float m_all[WAVES * 16];
  __shared__ float l_all[WAVES * 16];
  __shared__ int page_ids[DECODE_PAGE_IDS];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i = lane & 15;
  const int group = nh / nkv;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int page_size = 1 << page_shift;
  const int kv_len = kv_lens[b];
  const int pos = kv_len - 1;
  const bool row_ok = i < group;
  const int head = kvh * group + (row_ok ? i : 0);

  int n_begin = 0;
  if (window > 0) {
    n_begin = pos - window + 1;
    if (n_begin < 0) n_begin = 0;
    n_begin &= ~15;
  }
  const int tiles_total = (kv_len - n_begin + 15) / 16;
  const int per_split = (tiles_total + splits - 1) / splits;
  const int t_lo = split * per_split;
  int t_hi = t_lo + per_split;
  if (t_hi > tiles_total) t_hi = tiles_total;

  const int* table = block_tables + (size_t)b * table_width;
  // page ids of keys [n_begin + 16 t_lo, n_begin + 16 t_hi)
  const int first_page = (n_begin + 16 * t_lo) >> page_shift;
  const int last_key = n_begin + 16 * t_hi < kv_len ? n_begin + 16 * t_hi : kv_len;
  const int num_pages = t_hi > t_lo ? ((last_key - 1) >> page_shift) - first_page + 1 : 0;
  {
    // (each thread's first id without a branch around the load: it is on the way of everything that follows)
    int at = first_page + (tid < num_pages ? tid : 0);
    at = at < table_width ? at : table_width - 1;
    const int id = table[at];
    if (tid < num_pages) page_ids[tid] = id;
    for (int p = tid + 64 * WAVES; p < num_pages && p < DECODE_PAGE_IDS; p += 64 * WAVES) page_ids[p] = table[first_page + p];
  }

  typename KO::Operand qf[KO::STEPS];
  {
    const T* qp = qkv + (size_t)b * qkv_stride + (size_t)head * D + KO::LANE * g;
#pragma unroll
    for (int c = 0; c < KO::STEPS; ++c) {
      qf[c] = KO::load(qp + KO::SPAN * c);
      if (!row_ok) qf[c] = KO::zero();
    }
  }
  __syncthreads();
  // (the launcher sends a step here only if a split's keys span at most DECODE_PAGE_IDS pages; the clamp keeps a
  // violated promise from reading outside the array)
  auto page_of = [&](int n) -> size_t {
    const int p = (n >> page_shift) - first_page;
    return (size_t)page_ids[p < DECODE_PAGE_IDS ? p : DECODE_PAGE_IDS - 1];
  };

  struct Tile {
    typename KO::Operand k[KO::STEPS];
    Frag<T> v[NC];
  };
  // No branch surrounds a load, so the loads of a tile do not wait for those of the tiles before it: a key beyond the
  // sequence is read from the last valid place instead; its score is masked and its values are zeroed when the
  // tile is used.
  auto load_tile = [&](Tile& tile, int t) {
    int n_k = n_begin + 16 * t + i;      // the key whose row this lane reads
    int n_v = n_begin + 16 * t + 4 * g;  // the first of the four keys whose values this lane reads
    n_k = n_k < kv_len ? n_k : kv_len - 1;
    n_v = n_v < kv_len ? n_v : (kv_len - 1) & ~3;
    const T* kp = k_cache + ((page_of(n_k) * nkv + kvh) * page_size + (n_k & (page_size - 1))) * D + KO::LANE * g;
    const T* vp = v_cache + ((page_of(n_v) * nkv + kvh) * D + i) * page_size + (n_v & (page_size - 1));
#pragma unroll
    for (int c = 0; c < KO::STEPS; ++c) tile.k[c] = KO::load(kp + KO::SPAN * c);
#pragma unroll
    // (values are read once and a load instruction covers whole cache lines of V^T where pages hold 16 tokens: the
    // non-temporal hint then streams them faster, 80 us against 96 for 537 MB on MI355X; on the half lines of a K
    // load it costs speed)
    for (int c = 0; c < NC; ++c) {
      if constexpr (sizeof(T) == 4) tile.v[c].v = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(vp + (size_t)16 * c * page_size));
      else tile.v[c].v = __builtin_nontemporal_load(reinterpret_cast<const short4_t*>(vp + (size_t)16 * c * page_size));
    }
  };

  float m_i = -INFINITY, l_i = 0.f;
  float4_t acc_o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) acc_o[c] = float4_t{0.f, 0.f, 0.f, 0.f};

  auto compute_tile = [&](Tile& tile, int t) {
    if (n_begin + 16 * t + 16 > kv_len) {  // the sequence ends inside this tile (the same for the whole wave)
      const int valid = kv_len - (n_begin + 16 * t + 4 * g);
#pragma unroll
      for (int c = 0; c < NC; ++c) mask_frag(tile.v[c], valid);
    }
    float4_t s = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KO::STEPS; ++c) s = KO::mma(tile.k[c], qf[c], s);
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n_begin + 16 * t + 4 * g + j;
      const bool keep = row_ok && n < kv_len && (window <= 0 || n > pos - window);
      s[j] = keep ? s[j] * scale : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, VELOX_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, VELOX_WAVE));
    const float m_new = fmaxf(m_i, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m_i == -INFINITY) ? 0.f : softmax_exp<T>(m_i - m_safe);
    Frag<T> pf;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float p = (s[j] == -INFINITY) ? 0.f : softmax_exp<T>(s[j] - m_safe);
      psum += p;
      set_prob(pf, j, p);
    }
    l_i = l_i * alpha + psum;
    m_i = m_new;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc_o[c] = mma16(tile.v[c], pf, acc_o[c] * alpha);
  };

  // A ring of DEPTH register sets: while a tile is computed the next DEPTH - 1 are in flight.  The loop is unrolled by
  // the ring's length (register sets are named at compile time) and no load sits behind a branch: a tile beyond the
  // wave's last one is read again from the last one and never used.
  Tile ring[DEPTH];
  const int t0 = t_lo + wave;
  if (t0 < t_hi) {
    const int t_last = t0 + (t_hi - 1 - t0) / WAVES * WAVES;  // this wave's last tile
    auto step = [&](int t, Tile& cur, Tile& far) {
      const int tn = t + WAVES * (DEPTH - 1);
      load_tile(far, tn < t_hi ? tn : t_last);
      compute_tile(cur, t);
    };
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s) load_tile(ring[s], t0 + WAVES * s < t_hi ? t0 + WAVES * s : t_last);
    // (set S is computed while set S - 1, the one computed last, is filled again)
    auto round = [&](auto self, auto set, int& t) {
      constexpr int S = decltype(set)::value;
      step(t, ring[S], ring[(S + DEPTH - 1) % DEPTH]);
      t += WAVES;
      if constexpr (S + 1 < DEPTH) {
        if (t < t_hi) self(self, std::integral_constant<int, S + 1>{}, t);
      }
    };
    for (int t = t0; t < t_hi;) round(round, std::integral_constant<int, 0>{}, t);
    // Never true.  It keeps what was asked for ahead alive on the way out of the loop: otherwise the compiler moves
    // those loads behind the loop's exit tests, to the place of their use, where nothing hides their latency.
    if (splits < 0) {
#pragma unroll
      for (int s = 0; s < DEPTH; ++s) {
#pragma unroll
        for (int c = 0; c < NC; ++c) acc_o[c] = mma16(ring[s].v[c], ring[s].v[c], acc_o[c]);
#pragma unroll
        for (int c = 0; c < KO::STEPS; ++c) acc_o[0] = KO::mma(ring[s].k[c], ring[s].k[c], acc_o[0]);
      }
    }
  }

  l_i += __shfl_xor(l_i, 16, VELOX_WAVE);
  l_i += __shfl_xor(l_i, 32, VELOX_WAVE);
#pragma unroll
  for (int c = 0; c < NC; ++c) acc_all[(wave * NC + c) * 64 + lane] = acc_o[c];
  if (g == 0) { m_all[wave * 16 + i] = m_i; l_all[wave * 16 + i] = l_i; }
  __syncthreads();
  float m_tot = -INFINITY;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) m_tot = fmaxf(m_tot, m_all[w * 16 + i]);
  const float m_ref = (m_tot == -INFINITY) ? 0.f : m_tot;
  float weight[WAVES];
  float l_tot = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const float mw = m_all[w * 16 + i];
    weight[w] = (mw == -INFINITY) ? 0.f : softmax_exp<T>(mw - m_ref);
    l_tot += weight[w] * l_all[w * 16 + i];
  }
  if (!row_ok) return;
  const float inv = l_tot > 0.f ? 1.f / l_tot : 1.f;
  const size_t slot = ((size_t)split * total_tokens + b) * nh + head;
#pragma unroll
  for (int cc = 0; cc < NCW; ++cc) {
    const int c = wave + WAVES * cc;  // this wave writes channel blocks wave, wave + WAVES, ...
    if (c >= NC) break;
    float4_t sum = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < WAVES; ++w) sum += acc_all[(w * NC + c) * 64 + lane] * weight[w];
    sum = sum * inv;
    if (splits == 1) {
      T* dst = out + ((size_t)b * nh + head) * D + 16 * c + 4 * g;
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[j] = from_f32<T>(sum[j]);
    } else {
      *reinterpret_cast<float4_t*>(part_o + slot * D + 16 * c + 4 * g) = sum;
    }
  }
  if (splits > 1 && wave == 0 && g == 0) part_lse[slot] = l_tot > 0.f ? m_tot + logf(l_tot) : -INFINITY;
}

// out[token, head, :] = sum_s w_s * o_s / sum_s w_s,  w_s = exp(lse_s - max_s lse_s)
template <typename T>
__global__ void merge_splits_kernel(const float* __restrict__ part_o, const float* __restrict__ part_lse, T* __restrict__ out,
                                    int nh, int splits, int total_tokens, int first_token) {
  const size_t token = (size_t)blockIdx.x + first_token;  // (the launch covers tokens [first_token, total_tokens))
  const int head = blockIdx.y;
  const size_t stride = (size_t)total_tokens * nh;  // slots per split
  const size_t slot0 = token * nh + head;
  float mx = -INFINITY;
#pragma unroll 8
  for (int s = 0; s < splits; ++s) mx = fmaxf(mx, part_lse[s * stride + slot0]);
  const float m_safe = (mx == -INFINITY) ? 0.f : mx;
  for (int dd = threadIdx.x; dd < D; dd += blockDim.x) {
    float acc = 0.f, denom = 0.f;
#pragma unroll 8
    for (int s = 0; s < splits; ++s) {
      const size_t slot = s * stride + slot0;
      const float lse = part_lse[slot];
      const float w = (lse == -INFINITY) ? 0.f : expf(lse - m_safe);
      acc += w * part_o[slot * D + dd];
      denom += w;
    }
    out[slot0 * D + dd] = from_f32<T>(acc / (denom > 0.f ? denom : 1.f));
  }
}

// Which kernel portions of prompts take: 0 = chosen by shape; 1 = never the kernel with direct loads; 2 = that kernel
// wherever it can run, 3 = the same with two sets of waves (for tests and measurements).
static int portion_kernel_choice = 0;
extern "C" void velox_attention_portion_kernel(int choice) { portion_kernel_choice = choice; }

static int compute_units() {
  static int cached = 0;  // (the same value whichever thread gets here first)
  if (cached == 0) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
      count = 256;
    cached = count;
  }
  return cached;
}

template <typename T> constexpr int tile_keys() { return (sizeof(T) * D > 512) ? 32 : 64; }

template <typename T>
static int launch(const void* qkv, int qkv_stride, const void* k_cache, const void* v_cache, const int* block_tables, int table_width,
                  const int* cu_q, const int* kv_lens, void* out, float* part_o, float* part_lse, int num_seqs, int total_tokens,
                  int max_q_len, int max_kv_len, int nh, int nkv, int page_shift, float scale, int window, int splits, int first_token,
                  hipStream_t stream) {
  constexpr int BN = tile_keys<T>();
  const int group = nh / nkv;
  // the streaming kernel keeps the page ids of a split's keys in LDS: they have to fit
  const int keys_per_split = (((max_kv_len + 15) / 16 + splits - 1) / splits) * 16;
  const bool ids_fit = (keys_per_split >> page_shift) + 2 <= DECODE_PAGE_IDS;
  if (max_q_len == 1 && total_tokens == num_seqs && first_token == 0 && group <= 16 && page_shift >= 2 && sizeof(T) * D <= 512 && ids_fit) {
    // every sequence decodes one token: the streaming kernel.  Register sets per wave: one being computed, the others
    // in flight.  (For steps with one workgroup per compute unit, twice as many sets and eight waves per workgroup
    // were both measured slower on MI355X.)
    constexpr int DEPTH = sizeof(T) * D <= 256 ? 3 : 2;
    decode_attention_kernel<T, DEPTH, 4><<<dim3(splits, nkv, num_seqs), 256, 0, stream>>>(
        (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, kv_lens, (T*)out, part_o, part_lse,
        nh, nkv, page_shift, scale, window, splits, total_tokens);
    int status = (int)hipGetLastError();
    if (status != 0 || splits == 1) return status;
    merge_splits_kernel<T><<<dim3(total_tokens, nh), D < 64 ? 64 : D, 0, stream>>>(part_o, part_lse, (T*)out, nh, splits, total_tokens, 0);
    return (int)hipGetLastError();
  }
  // The kernel whose tiles reach LDS by direct loads: bfloat16, head sizes 64 and 128, pages of at least 8 tokens.
  constexpr bool HAS_DIRECT = sizeof(T) == 2 && (D == 64 || D == 128);
  const bool direct_ok = HAS_DIRECT && page_shift >= 3 && portion_kernel_choice != 1;
  auto launch_direct = [&](bool two_sets = false) -> int {
    if constexpr (HAS_DIRECT) {
      dim3 grid(num_seqs * splits, nkv, (max_q_len * group + 127) / 128);
      if (grid.z > 65535u) return (int)hipErrorInvalidValue;  // (more than 8 million rows in one portion)
      if (two_sets)
        direct_attention_kernel<2, 4, 2><<<grid, 512, 0, stream>>>(
            (const bf16_t*)qkv, qkv_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, table_width, cu_q, kv_lens, (bf16_t*)out,
            part_o, part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
      else
        direct_attention_kernel<2, 4><<<grid, 256, 0, stream>>>(
            (const bf16_t*)qkv, qkv_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, table_width, cu_q, kv_lens, (bf16_t*)out,
            part_o, part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
    }
    int status = (int)hipGetLastError();
    if (status != 0 || splits == 1) return status;
    merge_splits_kernel<T><<<dim3(total_tokens - first_token, nh), D < 64 ? 64 : D, 0, stream>>>(part_o, part_lse, (T*)out, nh, splits, total_tokens,
                                                                                                 first_token);
    return (int)hipGetLastError();
  };
  if (direct_ok && portion_kernel_choice >= 2 && max_q_len * group > 64) return launch_direct(portion_kernel_choice == 3);
  if (direct_ok && max_q_len * group > 64) {
    // Measured on MI355X over prompts and portions of 128 to 8,192 tokens behind up to 30,000 keys, with 28 heads over 4,
    // 12 over 2 and 40 over 8 (us: the kernels below / direct loads / direct loads with two sets of waves).  Direct loads
    // from 0.6 workgroups of 128 rows per compute unit on, and wherever the keys are split over workgroups (few tokens
    // behind thousands of keys): 2 x 2,048 tokens 105 / 84 / 100, 8,192 tokens 641 / 535 / 575, 512 tokens behind 29,488
    // keys 397 / 355 / 375; fewer workgroups stay with the kernels below (512 tokens: 16 / 22 / 19).
    // Two sets of waves share a workgroup's keys, which fills the compute units that one set leaves half empty:
    //  * up to 1.5 workgroups per compute unit (12 heads over 2: 4 x 512 tokens behind 1,536 keys 79 / 63 / 45, 4,096 tokens
    //    158 / 122 / 81; 28 over 4: 1,024 tokens 34 / 36 / 28), up to 1.75 for one prompt from an empty cache, the step whose
    //    last rows decide its time (2,048 tokens: 72 / 67 / 53);
    //  * with split keys, when even the splits leave compute units empty (12 over 2, 512 tokens behind 3,584 keys: 57 / 48 / 41);
    //  * above that, where the workgroups are about equally long (at least as many keys in the cache as in the portions,
    //    2,048 keys or more) and the count says so: one set keeps two workgroups on a compute unit, two sets one that is
    //    done in 0.55 of the time, and whole rounds of workgroups decide (40 heads over 8, 640 workgroups on 256 compute
    //    units: 4 x 512 tokens behind 3,584 keys 299 / 238 / 226, behind 7,680 keys 598 / 477 / 438; with 448 one round of one set
    //    is quicker, 28 over 4, 4 x 512 behind 3,584: 162 / 142 / 152).
    const long long units = compute_units();
    const long long workgroups = (long long)((max_q_len * group + 127) / 128) * nkv * num_seqs * splits;
    if (splits > 1) return launch_direct(workgroups <= units);
    if (workgroups * 5 >= 3 * units) {
      const long long two_sets_up_to = (num_seqs == 1 && max_kv_len <= max_q_len) ? 7 * units / 4 : 3 * units / 2;
      bool two_sets = workgroups <= two_sets_up_to;
      if (!two_sets && max_kv_len >= 2048 && max_kv_len >= 2 * max_q_len)
        two_sets = 55 * ((workgroups + units - 1) / units) < 100 * ((workgroups + 2 * units - 1) / (2 * units));
      return launch_direct(two_sets);
    }
  }
  // Eight waves per workgroup when bfloat16 portions are long enough to fill their rows and the step brings enough rows
  // that the larger workgroups still fill the GPU.  Behind few keys (a causal step's longest workgroup decides how
  // long the step takes, and short streams of keys leave LDS idle) a wave takes one row tile, 128 rows per workgroup;
  // behind many keys two, 256 rows per workgroup: every K and V^T operand read from LDS then feeds two matrix
  // instructions.  Measured on MI355X: 2,048 tokens from an empty cache 75 us against 85, 4 x 512 tokens behind 8,192
  // keys 315 us against 426 the other way round; the two meet where an average row reads about 1,300 keys.
  constexpr int WIDE = (sizeof(T) == 2 && D <= 128) ? 2 : 1;
  const int rows = max_q_len * group;
  if ((rows + 63) / 64 > 65535) return (int)hipErrorInvalidValue;  // (row blocks are the grid's third dimension)
  if (WIDE == 2 && rows > 64 && (long long)total_tokens * group / 128 * nkv * splits >= compute_units()) {
    if (max_kv_len - max_q_len / 2 <= 1280 || rows < 192) {  // (keys an average row reads)
      dim3 grid(num_seqs * splits, nkv, (rows + 127) / 128);
      // With enough workgroups to keep two on every compute unit, the 128 rows go to four waves of two row tiles: half
      // the reads of K and V^T from LDS per row, which bound this kernel.  Measured on MI355X (us, eight waves of one
      // tile against four of two): 4 x 512 tokens behind 1,024 keys 62.7 / 54.7, 2,048 tokens from an empty cache
      // 75.0 / 71.5, two such sequences 130.9 / 108.5 (28 heads over 4); 93.8 / 77.9 and 171.9 / 147.3 with 40 heads
      // over 8.  With fewer workgroups the eight waves hide more of a short stream's latency (12 heads over 2, two
      // sequences of 2,048: 61.5 / 75.8).
      const long long workgroups = (long long)grid.x * grid.y * grid.z;
      if (rows >= 256 && workgroups * 4 >= 7LL * compute_units()) {
        paged_attention_kernel<T, BN, 2, 1, 4><<<grid, 256, 0, stream>>>(
            (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
            part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
      } else {
        paged_attention_kernel<T, BN, 1, 1, 8><<<grid, 512, 0, stream>>>(
            (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
            part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
      }
    } else {
      dim3 grid(num_seqs * splits, nkv, (rows + 255) / 256);
      paged_attention_kernel<T, BN, WIDE, 1, 8><<<grid, 512, 0, stream>>>(
          (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
          part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
    }
  } else if (WIDE == 2 && (long long)((rows + 63) / 64) * nkv * num_seqs * splits < 2 * compute_units() && max_kv_len >= 8 * BN) {
    // too few workgroups to fill the GPU and many keys each: two sets of waves share a workgroup's keys
    dim3 grid(num_seqs * splits, nkv, (rows + 63) / 64);
    paged_attention_kernel<T, BN, 1, WIDE><<<grid, 256 * WIDE, 0, stream>>>(
        (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
        part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
  } else {
    dim3 grid(num_seqs * splits, nkv, (rows + 63) / 64);
    paged_attention_kernel<T, BN, 1, 1><<<grid, 256, 0, stream>>>(
        (const T*)qkv, qkv_stride, (const T*)k_cache, (const T*)v_cache, block_tables, table_width, cu_q, kv_lens, (T*)out, part_o,
        part_lse, nh, nkv, page_shift, scale, window, splits, total_tokens);
  }
  int status = (int)hipGetLastError();
  if (status != 0 || splits == 1) return status;
  merge_splits_kernel<T><<<dim3(total_tokens - first_token, nh), D < 64 ? 64 : D, 0, stream>>>(part_o, part_lse, (T*)out, nh, splits, total_tokens,
                                                                                               first_token);
  return (int)hipGetLastError();
}

extern "C" int velox_attention_head_dim() { return D; }

// part_o: float32 [splits, total_tokens, nh, D]; part_lse: float32 [splits, total_tokens, nh]; both unused when splits == 1.
// first_token: the sequences given (cu_q holds rows of qkv and out) cover rows [first_token, total_tokens); a launch for
// the later sequences of a step passes its first row here so that only those rows are merged.
extern "C" int velox_paged_attention(const void* qkv, int qkv_stride, const void* k_cache, const void* v_cache,
                                     const int* block_tables, int table_width, const int* cu_q, const int* kv_lens, void* out,
                                     float* part_o, float* part_lse, int num_seqs, int total_tokens, int max_q_len, int max_kv_len,
                                     int nh, int nkv, int page_shift, float scale, int window, int splits, int first_token, int dtype,
                                     hipStream_t stream) {
  if (num_seqs <= 0 || total_tokens <= 0) return 0;
  if (nh % nkv != 0 || splits < 1 || page_shift < 0 || max_kv_len < 1 || first_token < 0 || first_token >= total_tokens) return -1;
  if (dtype == VELOX_BF16)
    return launch<bf16_t>(qkv, qkv_stride, k_cache, v_cache, block_tables, table_width, cu_q, kv_lens, out, part_o, part_lse, num_seqs,
                          total_tokens, max_q_len, max_kv_len, nh, nkv, page_shift, scale, window, splits, first_token, stream);
  return launch<float>(qkv, qkv_stride, k_cache, v_cache, block_tables, table_width, cu_q, kv_lens, out, part_o, part_lse, num_seqs,
                       total_tokens, max_q_len, max_kv_len, nh, nkv, page_shift, scale, window, splits, first_token, stream);
}
