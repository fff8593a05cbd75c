// Weight-streaming matrix product for few rows of activations (decode, small mixed steps):
// out = X W^T with X [M <= 64 per launch block, K] and W [N, K] bfloat16, K contiguous in both.
// The cost is reading W once from HBM, so the kernel is built around that stream:
//
//   * a workgroup owns 32 rows of W (one output tile) and one range of k; its 4 waves take
//     interleaved 64-wide k slices of that range and are summed through LDS in a fixed order,
//     so the split over k needs no atomics and results are reproducible;
//   * inside a 64-wide slice lane (i, h) reads the 64 contiguous bytes W[row i][k0 + 32 h ..],
//     four 16-byte loads that feed four v_mfma_f32_32x32x16_bf16 steps; the activations are read
//     with the same k order (the contraction does not care about the order of k);
//   * when the matrix is too small to fill the chip (N small), the k range is also split over
//     workgroups (grid y); each writes a float32 partial slab that the consumer sums.
//
// Epilogues on the float32 sums: bias; SwiGLU (the tile holds 16 gate rows and the 16 matching up
// rows, so silu(gate) * up is local to a lane; pico_vllm/kernels/swiglu.py:36-41); float32 or
// bfloat16 store.  Layout of the 32x32 result tile: lane l holds output column (token) l % 32 and
// tile rows 8 (r / 4) + 4 (l / 32) + r % 4 in register r.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define EPI_BF16 0     // out bf16 [M, N]
#define EPI_F32 1      // out float32 [M, N] (slab `blockIdx.y` when the k range is split over the grid)
#define EPI_SWIGLU 2   // W = [gate rows; up rows], out bf16 [M, N / 2]

template <int MT, int EPI, bool TAIL>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ X, int ldx,
                                                          const bf16_t* __restrict__ W, int ldw,
                                                          const float* __restrict__ bias, void* __restrict__ out,
                                                          int ldo, long long slab_stride, int M, int N, int K,
                                                          int k_per_wg) {
  __shared__ float red[4][MT][16][64];   // [wave][column block][register][lane]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int tile = blockIdx.x;
  const int m0 = blockIdx.z * 32 * MT;
  // the row of W that tile row `col` stands for
  int wrow;
  bool w_ok;
  if (EPI == EPI_SWIGLU) {
    const int I = N / 2, gi = tile * 16 + (col & 15);
    w_ok = gi < I;
    wrow = (col < 16 ? 0 : I) + gi;
  } else {
    wrow = tile * 32 + col;
    w_ok = wrow < N;
  }
  // Rows beyond the matrix are clamped to its last row: what they contribute is never stored.
  // Only a k tail must read as zero, because it is summed into outputs that are stored.
  const int n_rows = N;
  const bf16_t* wrow0 = W + (size_t)min(wrow, n_rows - 1) * ldw;
  const bf16_t* xrow0[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) xrow0[t] = X + (size_t)min(m0 + 32 * t + col, M - 1) * ldx;
  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;

  const int k_begin = blockIdx.y * k_per_wg, k_end = min(K, k_begin + k_per_wg);
  struct Stage {
    uint4 w[4], x[MT][4];
  };
  auto multiply = [&](const Stage& st) {
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int t = 0; t < MT; t++)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, st.w[s]),
                                                         __builtin_bit_cast(bf16x8, st.x[t][s]), acc[t], 0, 0, 0);
  };
  // this wave's slices start at k_begin + 64 (wave + 4 i)
  const int first = k_begin + 64 * wave;
  if (!TAIL) {
    // K % 64 == 0: every slice is whole.  DEPTH slices are in flight per wave.  The slices are
    // taken in rounds of DEPTH: inside a round there is no branch (a branch between a load and the
    // wait for an older one makes the compiler wait for everything); every step of a round
    // multiplies one stage and refills it with the slice DEPTH ahead (beyond the wave's last
    // slice the last one is read again and not used); the last round, the only one that can be
    // partial, does not refill and multiplies only the slices that exist.
    constexpr int DEPTH = MT == 1 ? 3 : 2;
    if (first < k_end) {
      const int n_slices = (k_end - first + 255) / 256;
      const int rounds = (n_slices + DEPTH - 1) / DEPTH;
      const int last = first + (n_slices - 1) * 256;
      auto load_stage = [&](Stage& st, int slice) {
        const int k0 = min(first + 256 * slice, last);
#pragma unroll
        for (int s = 0; s < 4; s++) {
          st.w[s] = *reinterpret_cast<const uint4*>(wrow0 + k0 + 32 * h + 8 * s);
#pragma unroll
          for (int t = 0; t < MT; t++) st.x[t][s] = *reinterpret_cast<const uint4*>(xrow0[t] + k0 + 32 * h + 8 * s);
        }
      };
      Stage st[DEPTH];
#pragma unroll
      for (int d = 0; d < DEPTH; d++) load_stage(st[d], d);
      __builtin_amdgcn_sched_barrier(0);
      for (int r = 0; r + 1 < rounds; r++) {      // every slice of these rounds exists
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
          multiply(st[d]);
          __builtin_amdgcn_sched_barrier(0);     // keeps the refill from sinking next to its use
          load_stage(st[d], (r + 1) * DEPTH + d);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      const int left = n_slices - (rounds - 1) * DEPTH;           // 1..DEPTH slices in the last round
#pragma unroll
      for (int d = 0; d < DEPTH; d++)
        if (d < left) multiply(st[d]);
    }
  } else {
    for (int k0 = first; k0 < k_end; k0 += 256) {
      Stage st;
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const int k = k0 + 32 * h + 8 * s;          // 8 consecutive k; K % 8 == 0, so all or nothing
        const bool ok = k < k_end;
        const uint4 wv = *reinterpret_cast<const uint4*>(wrow0 + (ok ? k : 0));
        st.w[s] = ok ? wv : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < MT; t++) {
          const uint4 xv = *reinterpret_cast<const uint4*>(xrow0[t] + (ok ? k : 0));
          st.x[t][s] = ok ? xv : make_uint4(0, 0, 0, 0);
        }
      }
      multiply(st);
    }
  }
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) red[wave][t][r][lane] = acc[t][r];
  __syncthreads();

  // thread (a = wave, lane) finishes tile rows 8 a + 4 h + 0..3 of column `col`: sum of the 4 waves
  const int a = wave;
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int m = m0 + 32 * t + col;
    if (m >= M) continue;
    if (EPI == EPI_SWIGLU) {
      if (a >= 2) continue;
      const int I = N / 2, gi = tile * 16 + 8 * a + 4 * h;
      float v[4];
#pragma unroll
      for (int b = 0; b < 4; b++) {
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
          g += red[w][t][4 * a + b][lane];
          u += red[w][t][4 * (a + 2) + b][lane];
        }
        v[b] = g / (1.0f + __expf(-g)) * u;
      }
      bf16_t* o = (bf16_t*)out + (size_t)m * ldo + gi;
#pragma unroll
      for (int b = 0; b < 4; b++)
        if (gi + b < I) store_f32(o + b, v[b]);
    } else {
      const int n = tile * 32 + 8 * a + 4 * h;
      float v[4];
#pragma unroll
      for (int b = 0; b < 4; b++) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) s += red[w][t][4 * a + b][lane];
        v[b] = s + ((bias && blockIdx.y == 0 && n + b < N) ? bias[n + b] : 0.f);
      }
      if (EPI == EPI_F32) {
        float* o = (float*)out + (size_t)blockIdx.y * slab_stride + (size_t)m * ldo + n;
#pragma unroll
        for (int b = 0; b < 4; b++)
          if (n + b < N) o[b] = v[b];
      } else {
        bf16_t* o = (bf16_t*)out + (size_t)m * ldo + n;
#pragma unroll
        for (int b = 0; b < 4; b++)
          if (n + b < N) store_f32(o + b, v[b]);
      }
    }
  }
}

// k_splits > 1 is allowed for EPI_F32 only: slab y (float32 [M, ldo]) lies at out + y * slab_stride and
// holds the partial sum over its k range; the bias goes into slab 0.
extern "C" int pico_gemm_skinny(const void* X, int ldx, const void* W, int ldw, const float* bias, void* out, int ldo,
                                long long slab_stride, int epilogue, int M, int N, int K, int k_splits,
                                hipStream_t stream) {
  PICO_REQUIRE(M > 0 && N > 0 && K > 0, "pico_gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  PICO_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K,
               "pico_gemm_skinny: K and the row strides must be multiples of 8 (K=%d ldx=%d ldw=%d)", K, ldx, ldw);
  PICO_REQUIRE((uintptr_t)X % 16 == 0 && (uintptr_t)W % 16 == 0, "pico_gemm_skinny: operands must be 16-byte aligned");
  PICO_REQUIRE(epilogue >= 0 && epilogue <= 2, "pico_gemm_skinny: unknown epilogue %d", epilogue);
  PICO_REQUIRE(k_splits >= 1 && (k_splits == 1 || epilogue == EPI_F32), "pico_gemm_skinny: only the float32 epilogue can split k over the grid");
  PICO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && bias == nullptr), "pico_gemm_skinny: SwiGLU needs an even N and no bias");
  const int n_out = epilogue == EPI_SWIGLU ? N / 2 : N;
  PICO_REQUIRE(ldo >= n_out, "pico_gemm_skinny: output row stride too small");
  const int mt = M <= 32 ? 1 : 2;
  const int tiles = epilogue == EPI_SWIGLU ? (N / 2 + 15) / 16 : (N + 31) / 32;
  const int k_per_wg = ((K + k_splits - 1) / k_splits + 255) / 256 * 256;
  const int ky = (K + k_per_wg - 1) / k_per_wg;
  PICO_REQUIRE(ky == k_splits, "pico_gemm_skinny: K=%d cannot be cut into %d ranges of whole 256-wide steps (got %d)", K, k_splits, ky);
  dim3 grid(tiles, ky, (M + 32 * mt - 1) / (32 * mt));
  PICO_REQUIRE(grid.z <= 65535 && grid.y <= 65535, "pico_gemm_skinny: too many blocks");
  const float* b0 = bias;
  const bool tail = K % 64 != 0;
#define LAUNCH2(MT, EPI, TAIL) \
  gemm_skinny_kernel<MT, EPI, TAIL><<<grid, 256, 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, ldw, b0, out, ldo, slab_stride, M, N, K, k_per_wg)
#define LAUNCH(MT, EPI) do { if (tail) LAUNCH2(MT, EPI, true); else LAUNCH2(MT, EPI, false); } while (0)
  if (epilogue == EPI_BF16) { if (mt == 1) LAUNCH(1, EPI_BF16); else LAUNCH(2, EPI_BF16); }
  else if (epilogue == EPI_F32) { if (mt == 1) LAUNCH(1, EPI_F32); else LAUNCH(2, EPI_F32); }
  else { if (mt == 1) LAUNCH(1, EPI_SWIGLU); else LAUNCH(2, EPI_SWIGLU); }
#undef LAUNCH2
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}
