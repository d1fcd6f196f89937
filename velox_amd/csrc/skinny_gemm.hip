// out[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) for few rows (M <= 64), bfloat16 operands, float32 accumulation: the
// matrix products of a decode step on gfx950.  Such a product is bound by reading W once from HBM, so the kernel is
// built around keeping many wide loads of W in flight:
//
//  * a workgroup owns 16 * RT consecutive rows of W (output columns) and ALL of K; its waves split K among
//    themselves and their partial sums are added through LDS in a fixed order (no atomics: the result is the same
//    on every run and does not depend on the launch);
//  * a lane reads W in runs of 16 consecutive bfloat16 (32 bytes): for a block of 64 contraction indices, lane
//    (g = lane / 16, i = lane % 16) holds W[row i][k0 + 16 g .. + 15], the four lane groups cover 128 contiguous
//    bytes of each row.  The two halves of the run feed two v_mfma_f32_16x16x32_bf16, W as the left operand
//    (16 rows x 32 indices) and the activations as the right one (32 indices x 16 batch rows) with the same index
//    assignment, so out^T[n, m] accumulates in the usual 16x16 layout;
//  * the activations are small (M x K) and come from L2 in the same lane layout; batch rows beyond M are zeros.
//
// Requirements checked by the caller: K % 64 == 0, M <= 16 * CT, 16-byte aligned operands.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float8_raw_t __attribute__((ext_vector_type(8)));

struct Run16 {  // 16 consecutive bfloat16 = two MFMA operands
  bf16x8_t lo, hi;
};

__device__ __forceinline__ Run16 load_run(const bf16_t* p) {
  Run16 r;
  const float4_t* q = reinterpret_cast<const float4_t*>(p);
  const float4_t a = q[0], b = q[1];
  r.lo = __builtin_bit_cast(bf16x8_t, a);
  r.hi = __builtin_bit_cast(bf16x8_t, b);
  return r;
}

// A lane's run in the packed layout: the first halves of the 64 lanes' runs are one contiguous kilobyte and the second
// halves the next, so each load instruction reads whole cache lines.  Every weight is read once per product, so the
// loads carry the non-temporal hint (measured on MI355X: a kernel that only reads whole lines streams 10-17% faster
// with it; on half lines, as in the row-major layout, the hint costs 15%).  p = block + 8 * lane.
__device__ __forceinline__ Run16 load_run_packed(const bf16_t* p) {
  Run16 r;
  const float4_t* q = reinterpret_cast<const float4_t*>(p);
  const float4_t a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 64);
  r.lo = __builtin_bit_cast(bf16x8_t, a);
  r.hi = __builtin_bit_cast(bf16x8_t, b);
  return r;
}

// the two halves `half` elements apart (8: one run of 32 bytes; 512: the packed layout, read through the caches)
__device__ __forceinline__ Run16 load_run_halves(const bf16_t* p, int half) {
  Run16 r;
  const float4_t a = *reinterpret_cast<const float4_t*>(p), b = *reinterpret_cast<const float4_t*>(p + half);
  r.lo = __builtin_bit_cast(bf16x8_t, a);
  r.hi = __builtin_bit_cast(bf16x8_t, b);
  return r;
}

__device__ __forceinline__ Run16 zero_run() {
  Run16 r;
  const float4_t z = {0.f, 0.f, 0.f, 0.f};
  r.lo = __builtin_bit_cast(bf16x8_t, z);
  r.hi = r.lo;
  return r;
}

// GLU = true: W holds two stacked matrices, gate rows [0, n) and up rows [n, 2n); the first RT / 2 row tiles of a
// workgroup are gate rows, the others the up rows of the same output columns, and what is stored is
// silu(gate) * up, computed on the float32 sums (the [M, 2n] product is never written).
// PACKED = true: W is stored tile by tile in the order the lanes read it, [row tile of 16][block of 64 indices][half of a
// run][lane][8 elements] (rows padded with zeros to a multiple of 16; for GLU gate and up are padded separately), so that
// each of a wave's two loads of a block is one contiguous kilobyte.
// Activations in the order the lanes read them (M <= 16): [block of 64 indices][half h][lane = 16 g + row][8 elements]
// holds index 16 g + 8 h + e of the block, the layout of one 16-row tile of a packed W.  A kernel that writes the
// activations of the next product can leave them like this (beside the row-major copy); the next product's two loads
// of a block are then one contiguous kilobyte each instead of sixteen pieces of sixteen rows.  Rows beyond M are never
// written and hold whatever was there: they only reach output columns that nobody stores.
__device__ __forceinline__ size_t packed_row_offset(int row, int index) {
  return (size_t)(index >> 6) * 1024 + (size_t)(((index >> 3) & 1) * 512 + ((((index >> 4) & 3) * 16 + row) << 3) + (index & 7));
}

struct NoHooks {
  __device__ __forceinline__ void after_first() const {}
  __device__ __forceinline__ void before_barrier() const {}
};

// The products of one workgroup: every wave multiplies its share of K and leaves its sums in partial[wave]; after
// the barrier at the end each tile's sum is partial[0][tile] + partial[1][tile] + ... (to be added in that order).
// hooks.after_first() runs once, behind the first round of loads and products: the place for loads that the epilogue
// needs and whose addresses depend on loads issued before this function (they then fly with the second round of
// weights).  hooks.before_barrier() runs behind the main loop, before the barrier: the place to leave further things
// in LDS for the epilogue.
// a_packed != 0: the activations come in the lanes' order (see packed_row_offset; only with CT = 1).
template <int RT, int CT, int WAVES, bool GLU, bool PACKED, typename Hooks = NoHooks>
__device__ __forceinline__ void skinny_partial_sums(const bf16_t* __restrict__ a, int a_packed, const bf16_t* __restrict__ w, int m, int n, int k,
                                                    float4_t (&partial)[WAVES][RT * CT][64], Hooks hooks = Hooks(), int tile0 = -1, int w_half = -1) {
  constexpr int UNROLL = 4;  // blocks of 64 indices whose loads are issued together
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, i = lane & 15;
  constexpr int RTO = GLU ? RT / 2 : RT;  // row tiles that become output columns
  // tile0 >= 0: the workgroup's first row tile is given (else blockIdx.x counts groups of RTO tiles); w_half = 0 or 1 with
  // a packed W: only rows 8 w_half .. 8 w_half + 7 of the tile are read, the others count as zeros (two workgroups can
  // then share a tile, each with half the bytes to fetch)
  const int n0 = (tile0 >= 0 ? tile0 : blockIdx.x * RTO) * 16;

  // this wave's share of K, in blocks of 64
  const int blocks_total = k / 64;
  const int per_wave = (blocks_total + WAVES - 1) / WAVES;
  const int kb_lo = wave * per_wave;
  int kb_hi = kb_lo + per_wave;
  if (kb_hi > blocks_total) kb_hi = blocks_total;

  const bf16_t* w_ptr[RT];
  bool w_ok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int col = n0 + 16 * (rt % RTO) + i;          // output column this row of W contributes to
    w_ok[rt] = col < n;
    if constexpr (PACKED) {
      const size_t tiles_per_matrix = (size_t)(n + 15) / 16;
      const size_t tile = (size_t)(n0 / 16 + rt % RTO) + (rt >= RTO ? tiles_per_matrix : 0);
      w_ok[rt] = n0 + 16 * (rt % RTO) < n;  // padded rows are zeros in memory
      w_ptr[rt] = w + (w_ok[rt] ? tile : 0) * (size_t)(k / 64) * 1024 + lane * 8;
      w_ok[rt] = w_ok[rt] && (w_half < 0 || (i >> 3) == w_half);
    } else {
      const size_t row = (size_t)col + (rt >= RTO ? n : 0);  // its row in W
      w_ptr[rt] = w + (w_ok[rt] ? row : 0) * k + 16 * g;
    }
  }
  const bf16_t* a_ptr[CT];
  bool a_ok[CT];
  const int a_block = a_packed ? 1024 : 64;  // elements from one block of 64 indices to the next
  const int a_half = a_packed ? 512 : 8;     // and from the first half of a lane's run to the second
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int row = 16 * ct + i;
    a_ok[ct] = a_packed ? true : row < m;
    a_ptr[ct] = a_packed ? a + lane * 8 : a + (size_t)(a_ok[ct] ? row : 0) * k + 16 * g;
  }

  float4_t acc[RT][CT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = float4_t{0.f, 0.f, 0.f, 0.f};

  for (int kb = kb_lo; kb < kb_hi; kb += UNROLL) {
    Run16 wr[UNROLL][RT];
    Run16 ar[UNROLL][CT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const bool in_range = kb + u < kb_hi;
      const size_t k0 = (size_t)(kb + u) * 64;
      const size_t w0 = PACKED ? (size_t)(kb + u) * 1024 : k0;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wr[u][rt] = (in_range && w_ok[rt]) ? (PACKED ? load_run_packed(w_ptr[rt] + w0) : load_run(w_ptr[rt] + w0)) : zero_run();
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) ar[u][ct] = (in_range && a_ok[ct]) ? load_run_halves(a_ptr[ct] + (size_t)(kb + u) * a_block, a_half) : zero_run();
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wr[u][rt].lo, ar[u][ct].lo, acc[rt][ct], 0, 0, 0);
          acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wr[u][rt].hi, ar[u][ct].hi, acc[rt][ct], 0, 0, 0);
        }
    if (kb == kb_lo) hooks.after_first();
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) partial[wave][rt * CT + ct][lane] = acc[rt][ct];
  hooks.before_barrier();
  __syncthreads();
}

// Rows of A that still have to be normalised: A holds x * norm_weight in bfloat16 and the producer (the kernel
// below that adds a product to the residual stream) left sums of squares of x, one per workgroup and row; a product with
// such an A is scaled row by row with rstd[m] = rsqrt(sum_b partial[m][b] / width + eps) in its epilogue, which is the
// same as normalising A first.  The sums are added in a fixed order.  Only for M <= 16.
struct RowScale {
  const float* partial;  // [16][blocks] (row m's sums are contiguous), or null: rows are used as they are
  int blocks;
  float inv_width, eps;
};

// How a workgroup adds a row's sums: wave v takes the blocks [v * share, (v + 1) * share), lane (g, row) of it every fourth
// of them.  The loads write LDS directly (lane's value of round t lands at stage[wave][t][lane]): issued before the
// weights stream, they hold no registers meanwhile and are back long before the main loop ends, so no trip to memory
// is left for the epilogue.  Behind the main loop a wave reads its own values back, adds them and leaves one number
// per row in LDS; whoever needs rstd[m] adds the waves' numbers in wave order.
constexpr int ROW_SCALE_ROUNDS = 16;      // loads per lane: residual widths up to 16 * 64 * WAVES
constexpr int ROW_SCALE_BLOCKS = 64 * 8;  // what the eight-wave kernels take

template <int WAVES>
struct RowScaleLoads {
  typedef float Stage[WAVES][ROW_SCALE_ROUNDS][64];
  struct Share {
    int first, end, rounds;  // this lane's first block, the end of its wave's share, loads per lane
  };
  // (computed where it is needed rather than kept: the main loop has no registers to spare)
  static __device__ __forceinline__ Share share_of(const RowScale& rs) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int share = ((rs.blocks + WAVES - 1) / WAVES + 3) & ~3;
    return Share{wave * share + (lane >> 4), (wave + 1) * share < rs.blocks ? (wave + 1) * share : rs.blocks, share / 4};
  }

  static __device__ __forceinline__ void issue(const RowScale& rs, int m, Stage& stage) {
    if (rs.partial == nullptr) return;  // (the same for every thread of the launch)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = (lane & 15) < m ? (lane & 15) : 0;  // (a row beyond M reads row 0's sums; nobody uses its scale)
    const Share sh = share_of(rs);
    const float* p = rs.partial + (size_t)row * rs.blocks;
    for (int t = 0; t < sh.rounds; ++t) {
      const int b = sh.first + 4 * t;  // (what lies beyond the share is read from the row's last block and dropped below)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p + (b < sh.end ? b : rs.blocks - 1)),
                                       (__attribute__((address_space(3))) void*)(&stage[wave][t][0]), 4, 0, 0);
    }
  }

  // behind the main loop: this wave's part of every row's sum goes to part[wave][row]
  static __device__ __forceinline__ void leave(const RowScale& rs, const Stage& stage, float (&part)[WAVES][16]) {
    if (rs.partial == nullptr) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Share sh = share_of(rs);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the wave's own loads into LDS have landed (the weights were waited for already)
    float total = 0.f;
    for (int t = 0; t < sh.rounds; ++t) total += sh.first + 4 * t < sh.end ? stage[wave][t][lane] : 0.f;
    total += __shfl_xor(total, 16, VELOX_WAVE);  // the four lane groups took every fourth block: a fixed order
    total += __shfl_xor(total, 32, VELOX_WAVE);
    if (lane < 16) part[wave][lane] = total;
  }
};

// after the barrier that follows the main loop
template <int WAVES>
__device__ __forceinline__ float row_scale_of(const RowScale& rs, const float (&part)[WAVES][16], int row) {
  if (rs.partial == nullptr) return 1.f;
  float total = part[0][row];
#pragma unroll
  for (int wv = 1; wv < WAVES; ++wv) total += part[wv][row];
  return rsqrtf(total * rs.inv_width + rs.eps);
}

template <int WAVES, typename After>
struct ScaleHooks {
  const RowScale& rs;
  const typename RowScaleLoads<WAVES>::Stage& stage;
  float (&part)[WAVES][16];
  After after;
  __device__ __forceinline__ void after_first() const { after(); }
  __device__ __forceinline__ void before_barrier() const { RowScaleLoads<WAVES>::leave(rs, stage, part); }
};
struct Nothing {
  __device__ __forceinline__ void operator()() const {}
};

// SCALED = true: the instantiation that can scale its rows; rs.partial is set then.
template <int RT, int CT, int WAVES, typename TO, bool GLU = false, bool PACKED = false, bool SCALED = false>
__global__ void __launch_bounds__(WAVES * 64) skinny_gemm_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                 const float* __restrict__ bias, TO* __restrict__ out, int m, int n, int k,
                                                                 RowScale rs, int a_packed, bf16_t* __restrict__ out_packed) {
  __shared__ float4_t partial[WAVES][RT * CT][64];
  __shared__ float scale_part[SCALED ? WAVES : 1][16];
  __shared__ float scale_stage[SCALED ? WAVES : 1][SCALED ? ROW_SCALE_ROUNDS : 1][SCALED ? 64 : 1];
  constexpr int RTO = GLU ? RT / 2 : RT;
  const int n0 = blockIdx.x * 16 * RTO;
  if constexpr (SCALED) {
    RowScaleLoads<WAVES>::issue(rs, m, scale_stage);
    skinny_partial_sums<RT, CT, WAVES, GLU, PACKED>(a, a_packed, w, m, n, k, partial, ScaleHooks<WAVES, Nothing>{rs, scale_stage, scale_part, Nothing()});
  } else {
    skinny_partial_sums<RT, CT, WAVES, GLU, PACKED>(a, a_packed, w, m, n, k, partial);
  }
  // add the waves' partial sums in wave order; each tile's 64 lanes are spread over the workgroup
  for (int item = threadIdx.x; item < RTO * CT * 64; item += WAVES * 64) {
    const int tile = item >> 6, l = item & 63;
    float4_t sum = partial[0][tile][l];
#pragma unroll
    for (int wv = 1; wv < WAVES; ++wv) sum += partial[wv][tile][l];
    float row_scale = 1.f;  // (unless the rows of A wait for their norm)
    if constexpr (SCALED) {
      row_scale = row_scale_of<WAVES>(rs, scale_part, l & 15);
      sum = sum * row_scale;
    }
    if constexpr (GLU) {
      float4_t up = partial[0][tile + RTO * CT][l];
#pragma unroll
      for (int wv = 1; wv < WAVES; ++wv) up += partial[wv][tile + RTO * CT][l];
      if constexpr (SCALED) up = up * row_scale;
#pragma unroll
      for (int j = 0; j < 4; ++j) sum[j] = sum[j] / (1.f + expf(-sum[j])) * up[j];
    }
    const int rt = tile / CT, ct = tile % CT;
    const int col_m = 16 * ct + (l & 15);           // batch row
    const int row_n = n0 + 16 * rt + 4 * (l >> 4);  // first of four output columns
    if (col_m >= m) continue;
    __attribute__((aligned(8))) bf16_t four[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      four[j] = from_f32<bf16_t>(0.f);
      if (row_n + j >= n) break;
      float v = sum[j];
      if (bias) v += bias[row_n + j];
      out[(size_t)col_m * n + row_n + j] = from_f32<TO>(v);
      four[j] = from_f32<bf16_t>(v);
    }
    if constexpr (GLU && CT == 1) {  // the same values in the order the next product's lanes read them (n % 64 == 0 then)
      typedef float float2_t __attribute__((ext_vector_type(2)));
      if (out_packed) *reinterpret_cast<float2_t*>(out_packed + packed_row_offset(col_m, row_n)) = *reinterpret_cast<const float2_t*>(four);
    }
  }
}

template <int RT, int CT, int WAVES>
static int launch_skinny_glu(const void* a, const void* w, void* out, int m, int n, int k, bool packed, RowScale rs, int a_packed, void* out_packed, hipStream_t stream) {
  const int blocks = (n + 8 * RT - 1) / (8 * RT);
  if (packed && rs.partial != nullptr) {
    if constexpr (CT == 1)  // (rows are scaled only for M <= 16)
      skinny_gemm_kernel<RT, CT, WAVES, bf16_t, true, true, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, nullptr, (bf16_t*)out, m, n, k, rs, a_packed, (bf16_t*)out_packed);
    else
      return -1;
  } else if (rs.partial != nullptr) {
    return -1;  // (only the packed weight's kernels scale rows)
  } else if (packed)
    skinny_gemm_kernel<RT, CT, WAVES, bf16_t, true, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, nullptr, (bf16_t*)out, m, n, k, rs, a_packed, (bf16_t*)out_packed);
  else
    skinny_gemm_kernel<RT, CT, WAVES, bf16_t, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, nullptr, (bf16_t*)out, m, n, k, rs, a_packed, (bf16_t*)out_packed);
  return (int)hipGetLastError();
}

template <int RT, int CT, int WAVES>
static int launch_skinny(const void* a, const void* w, const float* bias, void* out, int m, int n, int k, int out_dtype, bool packed, RowScale rs, int a_packed, hipStream_t stream) {
  const int blocks = (n + 16 * RT - 1) / (16 * RT);
  if (rs.partial != nullptr) {
    if constexpr (CT == 1) {  // (rows are scaled only for M <= 16, and only by the packed weight's kernels)
      if (!packed) return -1;
      if (out_dtype == VELOX_BF16)
        skinny_gemm_kernel<RT, CT, WAVES, bf16_t, false, true, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (bf16_t*)out, m, n, k, rs, a_packed, nullptr);
      else
        skinny_gemm_kernel<RT, CT, WAVES, float, false, true, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (float*)out, m, n, k, rs, a_packed, nullptr);
      return (int)hipGetLastError();
    }
    return -1;
  }
  if (packed) {
    if (out_dtype == VELOX_BF16)
      skinny_gemm_kernel<RT, CT, WAVES, bf16_t, false, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (bf16_t*)out, m, n, k, rs, a_packed, nullptr);
    else
      skinny_gemm_kernel<RT, CT, WAVES, float, false, true><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (float*)out, m, n, k, rs, a_packed, nullptr);
    return (int)hipGetLastError();
  }
  if (out_dtype == VELOX_BF16)
    skinny_gemm_kernel<RT, CT, WAVES, bf16_t><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (bf16_t*)out, m, n, k, rs, a_packed, nullptr);
  else
    skinny_gemm_kernel<RT, CT, WAVES, float><<<blocks, WAVES * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, bias, (float*)out, m, n, k, rs, a_packed, nullptr);
  return (int)hipGetLastError();
}

// waves: how many waves of a workgroup split K (4, 8 or 16; rounded down to what the tile shape allows); the
// caller picks it so that the launch fills the GPU.
// row_tiles: 16-row tiles of W per wave for M <= 16 (1 or 4).  With 4 a wave reuses each activation fragment for 64 rows
// of W, which quarters the traffic of the activations; worth it when N is large enough that N / 64 workgroups still fill the GPU.
// scale_partial (or null), scale_blocks, inv_width, eps: see RowScale; only with M <= 16.
// a_packed != 0: a is in the lanes' order (see packed_row_offset); only with M <= 16.
extern "C" int velox_skinny_gemm_bf16(const void* a, const void* w, const float* bias, void* out, int m, int n, int k, int out_dtype,
                                      int waves, int row_tiles, int packed, const float* scale_partial, int scale_blocks,
                                      float inv_width, float eps, int a_packed, hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (k % 64 != 0 || m > 64 || (scale_partial != nullptr && (m > 16 || scale_blocks > ROW_SCALE_BLOCKS)) || (a_packed && m > 16)) return -1;
  if (scale_partial != nullptr && waves < 8) waves = 8;  // (rows are scaled by the eight-wave kernels)
  const RowScale rs{scale_partial, scale_blocks, inv_width, eps};
#define PICK(RT, CT, W) return launch_skinny<RT, CT, W>(a, w, bias, out, m, n, k, out_dtype, packed != 0, rs, a_packed, stream)
  if (m <= 16 && row_tiles >= 4) {
    if (waves >= 8) PICK(4, 1, 8);
    PICK(4, 1, 4);
  }
  if (m <= 16) {
    if (waves >= 16) PICK(1, 1, 16);
    if (waves >= 8) PICK(1, 1, 8);
    PICK(1, 1, 4);
  }
  // more tiles per wave: registers (and the LDS for the final sum) allow 8 waves at most
  if (m <= 32) {
    if (waves >= 8) PICK(2, 2, 8);
    PICK(2, 2, 4);
  }
  if (waves >= 8) PICK(2, 4, 8);
  PICK(2, 4, 4);
#undef PICK
}

// ---------------------------------------------------------------------------------------------------------------
// The query/key/value projection of a decode step with everything that follows it before attention: bias, rotation
// and the write into the paged cache are the epilogue of the product, so the [M, (heads + 2 kv_heads) d] result never
// goes to memory and one launch is saved.  W is packed (see above) with its rows reordered so that a workgroup's two
// row tiles are what one rotation needs: for a query or key head the 16 channels c0 .. c0 + 15 of the low half and
// their partners c0 + d/2 ..; for a value head two consecutive tiles.  Needs d % 32 == 0 and a rotation of the
// whole head (tables of d / 2 angles per position).
// ---------------------------------------------------------------------------------------------------------------
struct RotaryWrite {
  const float* bias;       // [(heads + 2 kv_heads) * d] in the original row order, or null
  const int* positions;    // [M]
  const float* cos_table;  // [positions, d / 2]
  const float* sin_table;
  const int* slots;        // [M]: page * page_size + offset of the token's key
  bf16_t* q_out;           // [M, heads * d]
  bf16_t* k_cache;         // [pages, kv_heads, page_size, d]
  bf16_t* v_cache;         // [pages, kv_heads, d, page_size]
  int heads, kv_heads, d, page_size;
};

template <int WAVES>
__global__ void __launch_bounds__(WAVES * 64) skinny_qkv_rotary_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                       RotaryWrite args, int m, int n, int k, RowScale rs, int a_packed) {
  __shared__ float4_t partial[WAVES][2][64];
  __shared__ float scale_part[WAVES][16];
  __shared__ float scale_stage[WAVES][ROW_SCALE_ROUNDS][64];
  // What the epilogue reads is asked for before and inside the main loop (no branch around a load: every thread asks, a
  // row beyond M for row 0's; the first 64 threads use it): the slot and the position first, the bias and, behind the
  // first round of weights, the angles at that position, so that none of these trips to memory is left for the end.
  const int l = threadIdx.x;
  const int row = l & 15;  // batch row
  const int row_in = row < m ? row : 0;
  const int d = args.d, half = d / 2;
  const int pairs_per_head = d / 32;
  const int head = blockIdx.x / pairs_per_head, j = blockIdx.x % pairs_per_head;
  const int r4 = 4 * ((l & 63) >> 4);
  const bool rotated = head < args.heads + args.kv_heads;
  const int c = (rotated ? 16 : 32) * j + r4;  // first of four channels; their partners are half (16 for values) further on
  const int slot = args.slots[row_in];
  const int position = args.positions[row_in];
  // (without a bias the same loads read the start of the angle table and their values are dropped)
  const float* bias_at = args.bias ? args.bias + (size_t)head * d + c : args.cos_table;
  float4_t bias_first = *reinterpret_cast<const float4_t*>(bias_at);
  float4_t bias_second = *reinterpret_cast<const float4_t*>(bias_at + (args.bias ? (rotated ? half : 16) : 0));
  float4_t cs = float4_t{1.f, 1.f, 1.f, 1.f}, sn = float4_t{0.f, 0.f, 0.f, 0.f};
  auto fetch_angles = [&]() {
    const size_t angle = (size_t)position * half + (rotated ? c : 0);
    cs = *reinterpret_cast<const float4_t*>(args.cos_table + angle);
    sn = *reinterpret_cast<const float4_t*>(args.sin_table + angle);
  };
  RowScaleLoads<WAVES>::issue(rs, m, scale_stage);
  skinny_partial_sums<2, 1, WAVES, false, true>(a, a_packed, w, m, n, k, partial, ScaleHooks<WAVES, decltype(fetch_angles)>{rs, scale_stage, scale_part, fetch_angles});
  if (l >= 64) return;
  const float row_scale = row_scale_of<WAVES>(rs, scale_part, row_in);
  if (row >= m) return;
  float4_t first = partial[0][0][l], second = partial[0][1][l];
#pragma unroll
  for (int wv = 1; wv < WAVES; ++wv) {
    first += partial[wv][0][l];
    second += partial[wv][1][l];
  }
  if (!args.bias) bias_first = bias_second = float4_t{0.f, 0.f, 0.f, 0.f};
  first = first * row_scale + bias_first;
  second = second * row_scale + bias_second;
  const size_t page = (size_t)(slot / args.page_size);
  const int offset = slot % args.page_size;
  if (rotated) {
    __attribute__((aligned(8))) bf16_t lo[4];
    __attribute__((aligned(8))) bf16_t hi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = from_f32<bf16_t>(first[e] * cs[e] - second[e] * sn[e]);
      hi[e] = from_f32<bf16_t>(first[e] * sn[e] + second[e] * cs[e]);
    }
    bf16_t* dst = head < args.heads
                      ? args.q_out + ((size_t)row * args.heads + head) * d + c
                      : args.k_cache + (((page * args.kv_heads + (head - args.heads)) * args.page_size) + offset) * d + c;
    typedef float float2_t __attribute__((ext_vector_type(2)));
    *reinterpret_cast<float2_t*>(dst) = *reinterpret_cast<const float2_t*>(lo);
    *reinterpret_cast<float2_t*>(dst + half) = *reinterpret_cast<const float2_t*>(hi);
  } else {
    const int vh = head - args.heads - args.kv_heads;
    bf16_t* dst = args.v_cache + ((page * args.kv_heads + vh) * d + c) * args.page_size + offset;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      dst[(size_t)e * args.page_size] = from_f32<bf16_t>(first[e]);
      dst[(size_t)(16 + e) * args.page_size] = from_f32<bf16_t>(second[e]);
    }
  }
}

// a [M, K] (M <= 16), w: packed rows of [Wq; Wk; Wv] in the rotary order; q_out [M, heads * d]; keys and values go to
// the cache at slots[M].  waves: kept for the call's shape; 8 are used.
extern "C" int velox_skinny_qkv_rotary_bf16(const void* a, const void* w, const float* bias, const int* positions,
                                            const float* cos_table, const float* sin_table, const int* slots, void* q_out,
                                            void* k_cache, void* v_cache, int m, int k, int heads, int kv_heads, int d,
                                            int page_size, int waves, const float* scale_partial, int scale_blocks, float inv_width,
                                            float eps, int a_packed, hipStream_t stream) {
  if (m <= 0) return 0;
  if (m > 16 || k % 64 != 0 || d % 32 != 0 || heads < 1 || kv_heads < 1 || page_size < 1) return -1;
  if (scale_partial != nullptr && scale_blocks > ROW_SCALE_BLOCKS) return -1;
  RotaryWrite args{bias, positions, cos_table, sin_table, slots, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                   heads, kv_heads, d, page_size};
  const RowScale rs{scale_partial, scale_blocks, inv_width, eps};
  const int n = (heads + 2 * kv_heads) * d;
  const int blocks = n / 32;
  (void)waves;  // (16 waves leave 128 registers per lane, which this kernel does not fit without spilling, and measured no faster)
  skinny_qkv_rotary_kernel<8><<<blocks, 8 * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, args, m, n, k, rs, a_packed);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------------
// The last product of a sub-layer at decode size, with the residual add and the first half of the next norm as its
// epilogue: residual[M, N] += A W^T (float32, in place; every element belongs to one workgroup), next[M, N] =
// bfloat16(residual * norm_weight), and sums[m][block] = the sum of squares of the block's 16 new residual values of
// row m.  Whoever multiplies `next` scales its rows with the sums (RowScale above): the norm costs no kernel.
// ---------------------------------------------------------------------------------------------------------------
// HALF: two workgroups share a 16-row tile of W, each reading eight of its rows (a narrow W then still gives every compute
// unit a workgroup); the sums of squares are then per block of 8 columns.
template <int WAVES, int RT = 1, bool HALF = false>
__global__ void __launch_bounds__(WAVES * 64) skinny_residual_norm_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                          float* __restrict__ residual, const float* __restrict__ norm_weight,
                                                                          bf16_t* __restrict__ next, float* __restrict__ sums, int m, int n, int k,
                                                                          int a_packed, bf16_t* __restrict__ next_packed) {
  static_assert(!HALF || RT == 1, "half tiles come one to a workgroup");
  __shared__ float4_t partial[WAVES][RT][64];
  // what the epilogue reads is fetched before the main loop (by the 64 threads per tile that will need it)
  const int l = threadIdx.x & 63, tile = threadIdx.x >> 6;  // (in the epilogue: wave t finishes tile t)
  const int row = l & 15;
  const int tiles_total = (n + 15) / 16;
  const int tile_n = HALF ? blockIdx.x >> 1 : blockIdx.x * RT + tile;
  const int half = HALF ? blockIdx.x & 1 : -1;
  const bool mine = !HALF || (l >> 5) == half;  // (lane group g holds rows 4g .. 4g + 3 of the tile)
  const int col = tile_n * 16 + 4 * (l >> 4);  // first of this lane's four columns
  float old_residual[4], weight[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const bool inside = tile < RT && mine && row < m && col + j < n;
    old_residual[j] = inside ? residual[(size_t)row * n + col + j] : 0.f;
    weight[j] = inside ? norm_weight[col + j] : 0.f;
  }
  if constexpr (HALF) skinny_partial_sums<1, 1, WAVES, false, true>(a, a_packed, w, m, n, k, partial, NoHooks(), tile_n, half);
  else skinny_partial_sums<RT, 1, WAVES, false, true>(a, a_packed, w, m, n, k, partial);
  if (tile >= RT || tile_n >= tiles_total) return;
  float4_t sum = partial[0][tile][l];
#pragma unroll
  for (int wv = 1; wv < WAVES; ++wv) sum += partial[wv][tile][l];
  float squares = 0.f;
  if (row < m && mine) {
    __attribute__((aligned(8))) bf16_t four[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      four[j] = from_f32<bf16_t>(0.f);
      if (col + j >= n) break;
      const size_t at = (size_t)row * n + col + j;
      const float r = old_residual[j] + sum[j];
      residual[at] = r;
      four[j] = from_f32<bf16_t>(r * weight[j]);
      next[at] = four[j];
      squares += r * r;
    }
    // the same values in the order the next product's lanes read them (n % 64 == 0 then)
    typedef float float2_t __attribute__((ext_vector_type(2)));
    if (next_packed) *reinterpret_cast<float2_t*>(next_packed + packed_row_offset(row, col)) = *reinterpret_cast<const float2_t*>(four);
  }
  // the lane groups hold four columns each of the same rows: added in a fixed order
  squares += __shfl_xor(squares, 16, VELOX_WAVE);
  if constexpr (HALF) {
    if ((l >> 4) == 2 * half) sums[(size_t)row * (2 * tiles_total) + blockIdx.x] = squares;
  } else {
    squares += __shfl_xor(squares, 32, VELOX_WAVE);
    if (l < 16) sums[(size_t)l * tiles_total + tile_n] = squares;
  }
}

// a [M, K] bfloat16 (M <= 16; a_packed != 0: in the lanes' order, see packed_row_offset), w packed [N, K]; sums: float32
// [16][blocks], blocks = ceil(N / 16), or twice that with row_tiles = 0.  next_packed (or null; needs N % 64 == 0): room
// for N / 64 * 1024 elements, `next` once more in the lanes' order.  waves: 4, 8 or 16.  row_tiles: 16-row tiles of W per
// workgroup: 1; 2 (every activation fragment a wave loads feeds two tiles: half the activations' bytes, half as many
// workgroups; eight waves); or 0 for half a tile (twice as many workgroups; eight waves).
extern "C" int velox_skinny_residual_norm_bf16(const void* a, const void* w, float* residual, const float* norm_weight, void* next,
                                               float* sums, int m, int n, int k, int waves, int row_tiles, int a_packed, void* next_packed,
                                               hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (m > 16 || k % 64 != 0 || (next_packed != nullptr && n % 64 != 0)) return -1;
  const int tiles = (n + 15) / 16;
#define RESIDUAL_NORM(W, RT, HALF, GRID) \
  skinny_residual_norm_kernel<W, RT, HALF><<<GRID, W * 64, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, residual, norm_weight, (bf16_t*)next, sums, \
                                                                         m, n, k, a_packed, (bf16_t*)next_packed)
  if (row_tiles == 0) RESIDUAL_NORM(8, 1, true, 2 * tiles);
  else if (row_tiles >= 2) RESIDUAL_NORM(8, 2, false, (tiles + 1) / 2);
  else if (waves >= 16) RESIDUAL_NORM(16, 1, false, tiles);
  else if (waves >= 8) RESIDUAL_NORM(8, 1, false, tiles);
  else RESIDUAL_NORM(4, 1, false, tiles);
#undef RESIDUAL_NORM
  return (int)hipGetLastError();
}

// out[M, n] = silu(A Wgate^T) * (A Wup^T) with W = [Wgate; Wup] of 2n rows, bfloat16 in and out, M <= 32.
// pairs: gate/up tile pairs per wave (1 or 2).
// a_packed != 0: a is in the lanes' order (see packed_row_offset); out_packed (or null; needs n % 64 == 0): room for
// n / 64 * 1024 elements, the result once more in that order.  Both only with M <= 16.
extern "C" int velox_skinny_gemm_glu_bf16(const void* a, const void* w, void* out, int m, int n, int k, int waves, int pairs, int packed,
                                          const float* scale_partial, int scale_blocks, float inv_width, float eps, int a_packed,
                                          void* out_packed, hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (k % 64 != 0 || m > 32 || (scale_partial != nullptr && (m > 16 || scale_blocks > ROW_SCALE_BLOCKS))) return -1;
  if ((a_packed || out_packed != nullptr) && (m > 16 || (out_packed != nullptr && n % 64 != 0))) return -1;
  const RowScale rs{scale_partial, scale_blocks, inv_width, eps};
  if (scale_partial != nullptr && waves < 8) waves = 8;  // (rows are scaled by the eight-wave kernels)
  if (m <= 16) {
    if (pairs >= 2) {
      if (waves >= 8) return launch_skinny_glu<4, 1, 8>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
      return launch_skinny_glu<4, 1, 4>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
    }
    if (waves >= 8) return launch_skinny_glu<2, 1, 8>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
    return launch_skinny_glu<2, 1, 4>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
  }
  if (waves >= 8) return launch_skinny_glu<2, 2, 8>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
  return launch_skinny_glu<2, 2, 4>(a, w, out, m, n, k, packed != 0, rs, a_packed, out_packed, stream);
}

// ---------------------------------------------------------------------------------------------------------------
// Split-K variant for 17 .. 64 rows and matrices with few rows of W but a long K (the output and down projections):
// partial[s, M, N] = A[:, K_s] * W[:, K_s]^T in float32 for each of S slices K_s of K; whoever consumes the result adds the
// S partial sums (the residual-add + norm kernel does, in a fixed order).  A workgroup owns 64 rows of W (one 16-row
// tile per wave) and one slice of K.  W streams through a ring of three register sets, two chunks (of 4 blocks of 64
// indices) ahead of the arithmetic; the activations of a chunk (up to 64 rows x 256 indices) are asked for one chunk
// ahead, staged in LDS once per workgroup and read by all four waves.  It runs best with one workgroup per compute
// unit (the caller picks the number of slices for that).
// ---------------------------------------------------------------------------------------------------------------
template <int CT, bool PACKED>
__global__ void __launch_bounds__(256) skinny_gemm_splitk_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                float* __restrict__ partial, int m, int n, int k, int blocks_per_split) {
  constexpr int CHUNK = 4;                 // blocks of 64 indices per staging step
  constexpr int ROWS = 16 * CT;            // activation rows held in LDS
  constexpr int AS = 64 + 8;               // row stride of one block of activations, in elements
  constexpr int A_VECS = ROWS * CHUNK * 8; // 16-byte vectors per chunk of activations
  constexpr int A_ITERS = A_VECS / 256;
  static_assert(A_VECS % 256 == 0, "every thread stages the same number of vectors");
  __shared__ __attribute__((aligned(16))) bf16_t a_tile[CHUNK * ROWS * AS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i = lane & 15;
  const int row = blockIdx.x * 64 + 16 * wave + i;
  // (rows beyond N: row 0 stands in and nothing is stored; the packed layout pads its last tile with zeros)
  const bf16_t* w_ptr = PACKED ? w + (size_t)(16 * (blockIdx.x * 4 + wave) < n ? blockIdx.x * 4 + wave : 0) * (k / 64) * 1024 + lane * 8
                               : w + (size_t)(row < n ? row : 0) * k + 16 * g;
  constexpr int W_BLOCK = PACKED ? 1024 : 64;  // elements from one block of 64 indices to the next
  const int blocks_total = k / 64;
  const int kb_lo = blockIdx.y * blocks_per_split;
  int kb_hi = kb_lo + blocks_per_split;
  if (kb_hi > blocks_total) kb_hi = blocks_total;

  float4_t acc[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) acc[ct] = float4_t{0.f, 0.f, 0.f, 0.f};

  // W streams through a ring of three register sets: while a chunk is multiplied the loads of the next two are in
  // flight.  No load sits behind a branch (the compiler would make each wait for the ones before): a block beyond the
  // slice is read from the slice's last block and its activations are zeroed on their way to LDS; rows beyond N or M
  // are read from row 0 and their results never stored.
  Run16 w_ring[3][CHUNK];
  float4_t a_next[A_ITERS];
  auto fetch_w = [&](int kb, Run16 (&set)[CHUNK]) {
#pragma unroll
    for (int u = 0; u < CHUNK; ++u) {
      const int block = kb + u < kb_hi ? kb + u : kb_hi - 1;
      set[u] = PACKED ? load_run_packed(w_ptr + (size_t)block * W_BLOCK) : load_run(w_ptr + (size_t)block * W_BLOCK);
    }
  };
  auto fetch_a = [&](int kb) {
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      const int v = tid + it * 256;  // vector index: (block u, row r, 16-byte piece p)
      const int u = v / (ROWS * 8), r = (v / 8) % ROWS, p = v % 8;
      const int block = kb + u < kb_hi ? kb + u : kb_hi - 1;
      a_next[it] = *reinterpret_cast<const float4_t*>(a + (size_t)(r < m ? r : 0) * k + (size_t)block * 64 + p * 8);
    }
  };
  // one chunk: its activations go to LDS, the next chunk's activations and the weights two chunks on are asked for
  // (the activations first: loads come back in order, and they are needed first), then the chunk is multiplied
  auto step = [&](int kb, Run16 (&w_cur)[CHUNK], Run16 (&w_far)[CHUNK]) {
    __syncthreads();  // the previous chunk has been read by every wave
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      const int v = tid + it * 256;
      const int u = v / (ROWS * 8), r = (v / 8) % ROWS, p = v % 8;
      if (kb + u >= kb_hi) a_next[it] = float4_t{0.f, 0.f, 0.f, 0.f};  // (only in a slice's last chunk)
      *reinterpret_cast<float4_t*>(a_tile + (u * ROWS + r) * AS + p * 8) = a_next[it];
    }
    __syncthreads();
    fetch_a(kb + CHUNK);
    fetch_w(kb + 2 * CHUNK, w_far);
#pragma unroll
    for (int u = 0; u < CHUNK; ++u)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const bf16_t* src = a_tile + (u * ROWS + 16 * ct + i) * AS + 16 * g;
        const bf16x8_t lo = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const float4_t*>(src));
        const bf16x8_t hi = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const float4_t*>(src + 8));
        acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[u].lo, lo, acc[ct], 0, 0, 0);
        acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[u].hi, hi, acc[ct], 0, 0, 0);
      }
  };

  if (kb_lo < kb_hi) {
    fetch_a(kb_lo);
    fetch_w(kb_lo, w_ring[0]);
    fetch_w(kb_lo + CHUNK, w_ring[1]);
  }
  for (int kb = kb_lo; kb < kb_hi;) {  // (unrolled by the ring's length: register sets are named at compile time)
    step(kb, w_ring[0], w_ring[2]);
    if ((kb += CHUNK) >= kb_hi) break;
    step(kb, w_ring[1], w_ring[0]);
    if ((kb += CHUNK) >= kb_hi) break;
    step(kb, w_ring[2], w_ring[1]);
    kb += CHUNK;
  }
  // Never true.  It keeps what was asked for ahead alive on the way out of the loop: otherwise the compiler moves those
  // loads behind the loop's exit tests, to the place of their use, where nothing hides their latency any more.
  if (blocks_per_split < 0) {
    float4_t keep = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) keep += a_next[it];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int u = 0; u < CHUNK; ++u)
        keep += __builtin_bit_cast(float4_t, w_ring[r][u].lo) + __builtin_bit_cast(float4_t, w_ring[r][u].hi);
    acc[0] += keep;
  }
  float* dst = partial + (size_t)blockIdx.y * m * n;
  const int col_n = blockIdx.x * 64 + 16 * wave + 4 * g;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col_m = 16 * ct + i;
    if (col_m >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (col_n + j < n) dst[(size_t)col_m * n + col_n + j] = acc[ct][j];
  }
}

// partial: float32 [splits, M, N].  blocks_per_split * splits must cover K / 64.
// packed != 0: w is in the packed layout (see skinny_partial_sums).
extern "C" int velox_skinny_gemm_splitk_bf16(const void* a, const void* w, float* partial, int m, int n, int k, int splits, int packed, hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (k % 64 != 0 || m > 64 || splits < 1) return -1;
  const int blocks_total = k / 64;
  const int per_split = (blocks_total + splits - 1) / splits;
  dim3 grid((n + 63) / 64, splits);
  if (m <= 32 && packed)
    skinny_gemm_splitk_kernel<2, true><<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, partial, m, n, k, per_split);
  else if (m <= 32)
    skinny_gemm_splitk_kernel<2, false><<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, partial, m, n, k, per_split);
  else if (packed)
    skinny_gemm_splitk_kernel<4, true><<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, partial, m, n, k, per_split);
  else
    skinny_gemm_splitk_kernel<4, false><<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, partial, m, n, k, per_split);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------------
// silu(A Wgate^T) * (A Wup^T) for 17 .. 64 rows: the gate/up product of a decode step at those sizes with its
// activation as the epilogue, so that the [M, 2n] product is never written.  W = [Wgate; Wup] packed, each matrix
// padded to whole 16-row tiles.  A workgroup of ten waves owns five gate tiles (waves 0 .. 4) and the five up tiles of
// the same output columns (waves 5 .. 9) and all of K; the up waves hand their sums to the gate waves through LDS at
// the end.  37888 rows of W are 1184 pairs, 237 workgroups: one round on 256 compute units.  As in the split-K kernel
// W streams through a ring of three register sets, two chunks (of 4 blocks of 64 indices) ahead of the arithmetic,
// and the activations of a chunk are asked for one chunk ahead, staged in LDS once per workgroup and read by all waves.
// ---------------------------------------------------------------------------------------------------------------
// GLU_ROWS_PAIRS: pairs of (gate, up) tiles per workgroup, chosen by the caller so that the launch is one round of
// workgroups (up to 6: twelve waves leave a lane the registers the ring needs).
template <int CT, int GLU_ROWS_PAIRS>
__global__ void __launch_bounds__(128 * GLU_ROWS_PAIRS) skinny_glu_rows_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                              bf16_t* __restrict__ out, int m, int n, int k) {
  constexpr int CHUNK = 4;
  constexpr int THREADS = 128 * GLU_ROWS_PAIRS;
  constexpr int ROWS = 16 * CT;
  constexpr int AS = 64 + 8;
  constexpr int A_VECS = ROWS * CHUNK * 8;
  constexpr int A_ITERS = (A_VECS + THREADS - 1) / THREADS;
  constexpr int TILE_BYTES = CHUNK * ROWS * AS * 2, HAND_BYTES = GLU_ROWS_PAIRS * CT * 64 * 16;
  __shared__ __attribute__((aligned(16))) char smem[TILE_BYTES > HAND_BYTES ? TILE_BYTES : HAND_BYTES];
  bf16_t* const a_tile = reinterpret_cast<bf16_t*>(smem);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i = lane & 15;
  const int tiles = (n + 15) / 16;  // per matrix
  const bool is_up = wave >= GLU_ROWS_PAIRS;
  const int pair = blockIdx.x * GLU_ROWS_PAIRS + (is_up ? wave - GLU_ROWS_PAIRS : wave);
  const bool pair_ok = pair < tiles;
  const int blocks_total = k / 64;
  const int kb_hi = blocks_total;
  // (a pair beyond N: tile 0 stands in and nothing is stored)
  const bf16_t* w_ptr = w + (size_t)((pair_ok ? pair : 0) + (is_up ? tiles : 0)) * blocks_total * 1024 + lane * 8;

  float4_t acc[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) acc[ct] = float4_t{0.f, 0.f, 0.f, 0.f};

  Run16 w_ring[3][CHUNK];
  float4_t a_next[A_ITERS];
  auto fetch_w = [&](int kb, Run16 (&set)[CHUNK]) {  // no branch around a load: a block beyond K is read from the last block
#pragma unroll
    for (int u = 0; u < CHUNK; ++u) {
      const int block = kb + u < kb_hi ? kb + u : kb_hi - 1;
      set[u] = load_run_packed(w_ptr + (size_t)block * 1024);
    }
  };
  auto fetch_a = [&](int kb) {
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      int v = tid + it * THREADS;  // vector index: (block u, row r, 16-byte piece p)
      v = v < A_VECS ? v : A_VECS - 1;
      const int u = v / (ROWS * 8), r = (v / 8) % ROWS, p = v % 8;
      const int block = kb + u < kb_hi ? kb + u : kb_hi - 1;
      a_next[it] = *reinterpret_cast<const float4_t*>(a + (size_t)(r < m ? r : 0) * k + (size_t)block * 64 + p * 8);
    }
  };
  auto step = [&](int kb, Run16 (&w_cur)[CHUNK], Run16 (&w_far)[CHUNK]) {
    __syncthreads();  // the previous chunk has been read by every wave
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      const int v = tid + it * THREADS;
      if (v < A_VECS) {
        const int u = v / (ROWS * 8), r = (v / 8) % ROWS, p = v % 8;
        if (kb + u >= kb_hi) a_next[it] = float4_t{0.f, 0.f, 0.f, 0.f};  // (only in the last chunk)
        *reinterpret_cast<float4_t*>(a_tile + (u * ROWS + r) * AS + p * 8) = a_next[it];
      }
    }
    __syncthreads();
    fetch_a(kb + CHUNK);
    fetch_w(kb + 2 * CHUNK, w_far);
#pragma unroll
    for (int u = 0; u < CHUNK; ++u)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const bf16_t* src = a_tile + (u * ROWS + 16 * ct + i) * AS + 16 * g;
        const bf16x8_t lo = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const float4_t*>(src));
        const bf16x8_t hi = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const float4_t*>(src + 8));
        acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[u].lo, lo, acc[ct], 0, 0, 0);
        acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[u].hi, hi, acc[ct], 0, 0, 0);
      }
  };

  fetch_a(0);
  fetch_w(0, w_ring[0]);
  fetch_w(CHUNK, w_ring[1]);
  for (int kb = 0; kb < kb_hi;) {  // (unrolled by the ring's length: register sets are named at compile time)
    step(kb, w_ring[0], w_ring[2]);
    if ((kb += CHUNK) >= kb_hi) break;
    step(kb, w_ring[1], w_ring[0]);
    if ((kb += CHUNK) >= kb_hi) break;
    step(kb, w_ring[2], w_ring[1]);
    kb += CHUNK;
  }
  // Never true; keeps the loads that were asked for ahead alive on the way out of the loop (otherwise the compiler moves
  // them behind the loop's exit tests, where nothing hides their latency).
  if (k < 0) {
    float4_t keep = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) keep += a_next[it];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int u = 0; u < CHUNK; ++u) keep += __builtin_bit_cast(float4_t, w_ring[r][u].lo) + __builtin_bit_cast(float4_t, w_ring[r][u].hi);
    acc[0] += keep;
  }
  // the up waves' sums go to the gate waves through LDS (the last chunk's activations are no longer needed)
  __syncthreads();
  float4_t* const handed = reinterpret_cast<float4_t*>(smem);
  if (is_up) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) handed[((wave - GLU_ROWS_PAIRS) * CT + ct) * 64 + lane] = acc[ct];
  }
  __syncthreads();
  if (is_up || !pair_ok) return;
  const int col_n = pair * 16 + 4 * g;  // first of this lane's four output columns
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col_m = 16 * ct + i;
    if (col_m >= m) continue;
    const float4_t up = handed[(wave * CT + ct) * 64 + lane];
    __attribute__((aligned(8))) bf16_t four[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) four[j] = from_f32<bf16_t>(acc[ct][j] / (1.f + expf(-acc[ct][j])) * up[j]);
    bf16_t* dst = out + (size_t)col_m * n + col_n;
    if (col_n + 3 < n && n % 4 == 0) {
      typedef float float2_t __attribute__((ext_vector_type(2)));
      *reinterpret_cast<float2_t*>(dst) = *reinterpret_cast<const float2_t*>(four);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (col_n + j < n) dst[j] = four[j];
    }
  }
}

template <int P>
static int launch_glu_rows(const void* a, const void* w, void* out, int m, int n, int k, hipStream_t stream) {
  const int tiles = (n + 15) / 16;
  const int blocks = (tiles + P - 1) / P;
  if (m <= 32)
    skinny_glu_rows_kernel<2, P><<<blocks, 128 * P, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, m, n, k);
  else
    skinny_glu_rows_kernel<4, P><<<blocks, 128 * P, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, m, n, k);
  return (int)hipGetLastError();
}

// a [M, K] bfloat16 (17 <= M <= 64 pays; any M <= 64 works), w: [Wgate; Wup] packed (2n rows), out [M, n] bfloat16.
// pairs: pairs of (gate, up) tiles per workgroup, 2 .. 6 (the caller aims at one workgroup per compute unit).
extern "C" int velox_skinny_glu_rows_bf16(const void* a, const void* w, void* out, int m, int n, int k, int pairs, hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  if (k % 64 != 0 || k < 64 || m > 64) return -1;
  switch (pairs) {
    case 2: return launch_glu_rows<2>(a, w, out, m, n, k, stream);
    case 3: return launch_glu_rows<3>(a, w, out, m, n, k, stream);
    case 4: return launch_glu_rows<4>(a, w, out, m, n, k, stream);
    case 5: return launch_glu_rows<5>(a, w, out, m, n, k, stream);
    case 6: return launch_glu_rows<6>(a, w, out, m, n, k, stream);
    default: return -1;
  }
}
