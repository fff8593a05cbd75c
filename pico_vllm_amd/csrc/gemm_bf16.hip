// bfloat16 matrix product on the matrix cores: C = A W^T (+ bias), float32 accumulate,
// float32 or bfloat16 result.  A [M, K] and W [N, K] are both K-contiguous, which is what
// v_mfma_f32_32x32x16_bf16 wants for both operands: lane l supplies 8 consecutive k of row
// l % 32, the k offset being 8 * (l / 32).  The 32 x 32 result tile has column l % 32 (an
// index of W's rows) in lane l and rows 8 * (r / 4) + 4 * (l / 32) + r % 4 in register r.
//
// This kernel reads both operands straight from global memory (no LDS staging): it is
// meant for few rows of A (decode, the output matrix on the wanted rows), where W is
// streamed once and A stays in cache.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// 8 consecutive bf16 of a row starting at column k; columns >= K read as zero.
__device__ __forceinline__ bf16x8 load_row8(const bf16_t* row, int k, int K, bool row_ok, bool vec_ok) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (row_ok) {
    if (vec_ok && k + 8 <= K) {
      v = *reinterpret_cast<const uint4*>(row + k);
    } else {
      bf16_t e[8];
#pragma unroll
      for (int i = 0; i < 8; i++) e[i] = (k + i < K) ? row[k + i] : (bf16_t)0;
      v.x = e[0] | ((uint32_t)e[1] << 16);
      v.y = e[2] | ((uint32_t)e[3] << 16);
      v.z = e[4] | ((uint32_t)e[5] << 16);
      v.w = e[6] | ((uint32_t)e[7] << 16);
    }
  }
  return __builtin_bit_cast(bf16x8, v);
}

// Workgroup of 4 waves; wave w owns W rows [n0 + 32 w, +32) and all MT 32-row tiles of A.
template <int MT, typename TC>
__global__ __launch_bounds__(256) void gemm_bf16_small_m_kernel(const bf16_t* __restrict__ A,
                                                                const bf16_t* __restrict__ W,
                                                                const float* __restrict__ bias, TC* __restrict__ C,
                                                                int M, int N, int K, int lda, int ldw, int ldc,
                                                                int vec_ok) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.x * 128 + wave * 32 + (lane & 31);
  const int m_base = blockIdx.y * (32 * MT);
  const int kq = (lane >> 5) * 8;
  const bool n_ok = n < N;
  const bf16_t* wrow = W + (size_t)(n_ok ? n : 0) * ldw;
  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
  const bf16_t* arow[MT];
  bool a_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int m = m_base + 32 * t + (lane & 31);
    a_ok[t] = m < M;
    arow[t] = A + (size_t)(a_ok[t] ? m : 0) * lda;
  }
  for (int k0 = 0; k0 < K; k0 += 16) {
    const bf16x8 b = load_row8(wrow, k0 + kq, K, n_ok, vec_ok);
#pragma unroll
    for (int t = 0; t < MT; t++) {
      const bf16x8 a = load_row8(arow[t], k0 + kq, K, a_ok[t], vec_ok);
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
    }
  }
  if (!n_ok) return;
  const float bv = bias ? bias[n] : 0.f;
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = m_base + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (m < M) store_f32(C + (size_t)m * ldc + n, acc[t][r] + bv);
    }
}

extern "C" int pico_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N,
                              int K, int lda, int ldw, int ldc, hipStream_t stream) {
  PICO_REQUIRE(M >= 0 && N > 0 && K > 0, "pico_gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  PICO_REQUIRE(lda >= K && ldw >= K && ldc >= N, "pico_gemm_bf16: a row stride is smaller than its row");
  PICO_REQUIRE(c_dtype == PICO_DTYPE_F32 || c_dtype == PICO_DTYPE_BF16, "pico_gemm_bf16: unknown dtype %d", c_dtype);
  if (M == 0) return 0;
  // 16-byte loads need rows that start on 16 bytes
  const int vec_ok = (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  const int mt = M <= 32 ? 1 : 2;
  dim3 grid((N + 127) / 128, (M + 32 * mt - 1) / (32 * mt));
  PICO_REQUIRE(grid.y <= 65535, "pico_gemm_bf16: M=%d is too large for one launch", M);
#define LAUNCH(MT, TC)                                                                                          \
  gemm_bf16_small_m_kernel<MT, TC><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, bias, (TC*)C, \
                                                             M, N, K, lda, ldw, ldc, vec_ok)
  if (c_dtype == PICO_DTYPE_F32) {
    if (mt == 1) LAUNCH(1, float); else LAUNCH(2, float);
  } else {
    if (mt == 1) LAUNCH(1, bf16_t); else LAUNCH(2, bf16_t);
  }
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}
