// out[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) with float32 accumulation, for gfx950.
//
// `gemm_fma_kernel` is the exact path: operands are widened to float32 (exactly, for bfloat16) and
// multiplied with plain fused multiply-adds, so a float32 run never touches a reduced-precision
// matrix mode.  It also serves operand mixes no library call covers (bfloat16 activations with
// weights a checkpoint stores in float32).  Each output element is summed over k in one fixed
// order by one thread, so a row's result does not depend on the other rows of the batch.  The sum
// is built from sums of GEMM_FOLD consecutive terms, each started at zero: the rounding error of a
// long sum (the down projection adds 18944 terms) then grows with the square roots of the two
// lengths and not with that of their product, which keeps the float32 path as close to the exact
// result as a blocked library product on a CPU is.
#include "common.h"

#define GEMM_BM 64
#define GEMM_BN 64
#define GEMM_BK 16
#define GEMM_PAD 4
#define GEMM_FOLD 128  // terms per inner sum (a multiple of GEMM_BK)

template <typename T>
__device__ __forceinline__ void load4(const T* __restrict__ base, size_t row_offset, int k, int k_limit, bool row_ok, bool vec_ok, float (&v)[4]) {
  if (!row_ok) { v[0] = v[1] = v[2] = v[3] = 0.f; return; }
  const T* p = base + row_offset + k;
  if (vec_ok && k + 3 < k_limit) {
    if constexpr (sizeof(T) == 4) {
      const float4_t x = *reinterpret_cast<const float4_t*>(p);
      v[0] = x[0]; v[1] = x[1]; v[2] = x[2]; v[3] = x[3];
    } else {
      const short4_t x = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(((uint32_t)(uint16_t)x[i]) << 16);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (k + i < k_limit) ? to_f32(p[i]) : 0.f;
  }
}

template <typename TA, typename TW, typename TO>
__global__ void __launch_bounds__(256) gemm_fma_kernel(const TA* __restrict__ a, const TW* __restrict__ w, const float* __restrict__ bias,
                                                       TO* __restrict__ out, int m, int n, int k, int a_vec, int w_vec) {
  __shared__ float a_tile[GEMM_BK][GEMM_BM + GEMM_PAD];
  __shared__ float w_tile[GEMM_BK][GEMM_BN + GEMM_PAD];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
  const int load_row = tid / 4;          // 0..63
  const int load_k = (tid % 4) * 4;      // 0, 4, 8, 12
  const bool a_row_ok = m0 + load_row < m;
  const bool w_row_ok = n0 + load_row < n;
  const size_t a_off = (size_t)(m0 + load_row) * k;
  const size_t w_off = (size_t)(n0 + load_row) * k;

  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

  for (int k0 = 0; k0 < k; k0 += GEMM_BK) {
    if (k0 % GEMM_FOLD == 0) {  // (also at 0: adds zeros)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    float av[4], wv[4];
    load4<TA>(a, a_off, k0 + load_k, k, a_row_ok, a_vec != 0, av);
    load4<TW>(w, w_off, k0 + load_k, k, w_row_ok, w_vec != 0, wv);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_tile[load_k + i][load_row] = av[i];
      w_tile[load_k + i][load_row] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GEMM_BK; ++kk) {
      const float4_t ar = *reinterpret_cast<const float4_t*>(&a_tile[kk][ty * 4]);
      const float4_t wr = *reinterpret_cast<const float4_t*>(&w_tile[kk][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
    if (row >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= n) continue;
      float v = total[i][j] + acc[i][j];
      if (bias) v += bias[col];
      out[(size_t)row * n + col] = from_f32<TO>(v);
    }
  }
}

// The same product for few rows (M <= 16), where it is bound by reading W once: the decode steps of a float32 run.
// A wave owns SKINNY_ROWS consecutive rows of W and all of K; lane l takes indices 4 l .. 4 l + 3 of every block of
// 256, so a wave's load of a row's block is one contiguous kilobyte (float32) and the activations (from L2) are used
// for SKINNY_ROWS rows of W at once.  A lane adds its terms in the order of k, the 64 lanes' sums are added in a fixed
// tree: an element's sum depends on nothing but its own row of A and row of W.
#define SKINNY_ROWS 4

template <typename TA, typename TW, typename TO, int MT>
__global__ void __launch_bounds__(256) skinny_fma_kernel(const TA* __restrict__ a, const TW* __restrict__ w, const float* __restrict__ bias,
                                                         TO* __restrict__ out, int m, int n, int k) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 4 + wave) * SKINNY_ROWS;
  if (n0 >= n) return;
  float acc[SKINNY_ROWS][MT];
#pragma unroll
  for (int r = 0; r < SKINNY_ROWS; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[r][i] = 0.f;
  size_t w_off[SKINNY_ROWS], a_off[MT];
#pragma unroll
  for (int r = 0; r < SKINNY_ROWS; ++r) w_off[r] = (size_t)(n0 + r < n ? n0 + r : n0) * k;  // (a row beyond N: row n0 again, never stored)
#pragma unroll
  for (int i = 0; i < MT; ++i) a_off[i] = (size_t)(i < m ? i : 0) * k;
  for (int k0 = 4 * lane; k0 < k; k0 += 256) {
    float wv[SKINNY_ROWS][4], av[MT][4];
#pragma unroll
    for (int r = 0; r < SKINNY_ROWS; ++r) load4<TW>(w, w_off[r], k0, k, true, true, wv[r]);
#pragma unroll
    for (int i = 0; i < MT; ++i) load4<TA>(a, a_off[i], k0, k, true, true, av[i]);
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int r = 0; r < SKINNY_ROWS; ++r)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[r][i] = fmaf(av[i][e], wv[r][e], acc[r][i]);
  }
#pragma unroll
  for (int r = 0; r < SKINNY_ROWS; ++r)
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const float total = wave_sum(acc[r][i]);
      if (lane == 0 && i < m && n0 + r < n) out[(size_t)i * n + n0 + r] = from_f32<TO>(total + (bias ? bias[n0 + r] : 0.f));
    }
}

template <typename TA, typename TW, typename TO>
static void launch_skinny_fma(const void* a, const void* w, const float* bias, void* out, int m, int n, int k, hipStream_t stream) {
  const int waves = (n + SKINNY_ROWS - 1) / SKINNY_ROWS;
  dim3 grid((waves + 3) / 4);
#define SKINNY(MT) skinny_fma_kernel<TA, TW, TO, MT><<<grid, 256, 0, stream>>>((const TA*)a, (const TW*)w, bias, (TO*)out, m, n, k)
  if (m <= 1) SKINNY(1);
  else if (m <= 2) SKINNY(2);
  else if (m <= 4) SKINNY(4);
  else if (m <= 8) SKINNY(8);
  else SKINNY(16);
#undef SKINNY
}

extern "C" int velox_gemm_fma(const void* a, const void* w, const float* bias, void* out, int m, int n, int k,
                              int a_dtype, int w_dtype, int out_dtype, hipStream_t stream) {
  if (m <= 0 || n <= 0) return 0;
  dim3 grid((n + GEMM_BN - 1) / GEMM_BN, (m + GEMM_BM - 1) / GEMM_BM);
  const int a_size = a_dtype == VELOX_BF16 ? 2 : 4, w_size = w_dtype == VELOX_BF16 ? 2 : 4;
  const int a_vec = (k % 4 == 0) && (((uintptr_t)a) % (4 * a_size) == 0);
  const int w_vec = (k % 4 == 0) && (((uintptr_t)w) % (4 * w_size) == 0);
#define LAUNCH(TA, TW, TO) \
  gemm_fma_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((const TA*)a, (const TW*)w, bias, (TO*)out, m, n, k, a_vec, w_vec)
  const int key = a_dtype * 4 + w_dtype * 2 + out_dtype;
  if (m <= 16 && a_vec && w_vec) {  // (rows of whole 16-byte pieces: every load is a vector)
    switch (key) {
      case 0: launch_skinny_fma<float, float, float>(a, w, bias, out, m, n, k, stream); break;
      case 1: launch_skinny_fma<float, float, bf16_t>(a, w, bias, out, m, n, k, stream); break;
      case 2: launch_skinny_fma<float, bf16_t, float>(a, w, bias, out, m, n, k, stream); break;
      case 3: launch_skinny_fma<float, bf16_t, bf16_t>(a, w, bias, out, m, n, k, stream); break;
      case 4: launch_skinny_fma<bf16_t, float, float>(a, w, bias, out, m, n, k, stream); break;
      case 5: launch_skinny_fma<bf16_t, float, bf16_t>(a, w, bias, out, m, n, k, stream); break;
      case 6: launch_skinny_fma<bf16_t, bf16_t, float>(a, w, bias, out, m, n, k, stream); break;
      case 7: launch_skinny_fma<bf16_t, bf16_t, bf16_t>(a, w, bias, out, m, n, k, stream); break;
      default: return -1;
    }
    VELOX_RETURN_LAUNCH_STATUS();
  }
  switch (key) {
    case 0: LAUNCH(float, float, float); break;
    case 1: LAUNCH(float, float, bf16_t); break;
    case 2: LAUNCH(float, bf16_t, float); break;
    case 3: LAUNCH(float, bf16_t, bf16_t); break;
    case 4: LAUNCH(bf16_t, float, float); break;
    case 5: LAUNCH(bf16_t, float, bf16_t); break;
    case 6: LAUNCH(bf16_t, bf16_t, float); break;
    case 7: LAUNCH(bf16_t, bf16_t, bf16_t); break;
    default: return -1;
  }
#undef LAUNCH
  VELOX_RETURN_LAUNCH_STATUS();
}
