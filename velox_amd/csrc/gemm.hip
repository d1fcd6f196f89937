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
