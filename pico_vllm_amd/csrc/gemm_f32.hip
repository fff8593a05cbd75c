// True float32 matrix product C = A W^T (+ bias): plain FMA, no matrix-core reduced
// precision.  Every output element is accumulated by one thread in an order that depends
// on K alone, so a row's result does not depend on how many other rows the call has.
// The sum is a tree of radix 16 over k: 16 products are added up one after the other, 16
// such sums likewise, and so on for four levels (the last takes what is left), so the
// rounding error of a sum grows like the square root of the number of levels times 16
// rather than like the square root of K: with one running sum over K = 8,960 terms the
// error of a product was twenty times that of storing its result in float32.
// It is the GEMM of the 32-bit engine (the reference uses the library through nn.Linear,
// pico_vllm/model.py:200,225,316,318,445); speed is secondary.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

// A [M, K] row stride lda; W [N, K] row stride ldw; C [M, N] row stride ldc.  TA is the
// storage type of A (float, or bfloat16 bits that are widened on load).
template <typename TA>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const TA* __restrict__ A, const float* __restrict__ W,
                                                       const float* __restrict__ bias, float* __restrict__ C,
                                                       int M, int N, int K, int lda, int ldw, int ldc) {
  __shared__ float As[BK][BM + 1];
  __shared__ float Ws[BK][BN + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  // lvl[0]: the running sum of the current 16 products; lvl[i]: of up to 16 finished sums of level i - 1
  // (level 3 of all of them)
  float lvl[4][4][4] = {};
  int tile = 0;
  for (int k0 = 0; k0 < K; k0 += BK, tile++) {
    // 64 x 16 elements per tile, 256 threads: 4 each
    for (int i = threadIdx.x; i < BM * BK; i += 256) {
      const int r = i / BK, c = i % BK;
      const int m = m0 + r, n = n0 + r, k = k0 + c;
      As[c][r] = (m < M && k < K) ? load_f32(A + (size_t)m * lda + k) : 0.f;
      Ws[c][r] = (n < N && k < K) ? W[(size_t)n * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; k++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) lvl[0][i][j] = fmaf(a[i], b[j], lvl[0][i][j]);
    }
    // carry: after every tile level 0 goes up; after every 16th tile level 1 does, after every 256th level 2
    // (the same for all threads: no divergence)
#pragma unroll
    for (int L = 0; L < 3; L++) {
      if (((tile + 1) & ((1 << (4 * L)) - 1)) != 0) break;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          lvl[L + 1][i][j] += lvl[L][i][j];
          lvl[L][i][j] = 0.f;
        }
    }
    __syncthreads();
  }
  // what the lower levels still hold goes up in the same fixed order
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = ((lvl[0][i][j] + lvl[1][i][j]) + lvl[2][i][j]) + lvl[3][i][j];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = acc[i][j] + (bias ? bias[n] : 0.f);
    }
  }
}

extern "C" int pico_gemm_f32(const void* A, int a_dtype, const float* W, const float* bias, float* C, int M, int N,
                             int K, int lda, int ldw, int ldc, hipStream_t stream) {
  PICO_REQUIRE(M >= 0 && N > 0 && K > 0, "pico_gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  PICO_REQUIRE(lda >= K && ldw >= K && ldc >= N, "pico_gemm_f32: a row stride is smaller than its row");
  if (M == 0) return 0;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  PICO_REQUIRE(grid.y <= 65535, "pico_gemm_f32: M=%d is too large for one launch", M);
  if (a_dtype == PICO_DTYPE_F32)
    gemm_f32_kernel<float><<<grid, 256, 0, stream>>>((const float*)A, W, bias, C, M, N, K, lda, ldw, ldc);
  else if (a_dtype == PICO_DTYPE_BF16)
    gemm_f32_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, W, bias, C, M, N, K, lda, ldw, ldc);
  else
    PICO_REQUIRE(false, "pico_gemm_f32: unknown dtype %d", a_dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
