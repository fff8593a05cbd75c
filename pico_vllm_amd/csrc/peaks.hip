// What this GPU reaches on the two resources the engine's kernels are bound by, measured rather than
// quoted: a read stream over a buffer far larger than the caches (what a decode step's weight stream could
// reach at best) and back-to-back bfloat16 matrix-core products on registers (what a prefill's products
// could reach at the clock the chip holds under that load).  The benchmark reports both beside the
// published peaks.  The reference measures its bandwidth use against a quoted peak only (README.md:9,46).
#include "common.h"

typedef __bf16 pk_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pk_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t pk_u32x4 __attribute__((ext_vector_type(4)));

// Every workgroup reads its share of the buffer with 16-byte loads, eight in flight per thread, and keeps an
// xor of what it read so that the loads cannot be dropped; one word per workgroup goes to `sink`.
__global__ __launch_bounds__(256) void peak_read_kernel(const pk_u32x4* __restrict__ buf, long long n16,
                                                        uint32_t* __restrict__ sink) {
  // a workgroup reads runs of 32 KB (eight loads of 16 bytes a thread), the runs of the grid side by side
  const long long stride = (long long)gridDim.x * 2048;
  pk_u32x4 acc = {0, 0, 0, 0};
  long long i = (long long)blockIdx.x * 2048 + threadIdx.x;
  for (; i + 2048 <= n16 + threadIdx.x; i += stride) {        // the whole run exists
    pk_u32x4 v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = buf[i + j * 256];
#pragma unroll
    for (int j = 0; j < 8; j++) acc ^= v[j];
  }
  for (int j = 0; j < 8; j++)                                  // the last, partial run of the buffer
    if (i + j * 256 < n16) acc ^= buf[i + j * 256];
  uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x ^= __shfl_xor(x, off, 64);
  __shared__ uint32_t part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) sink[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

// sink: at least `blocks` words.  bytes is rounded down to whole 16-byte units.
extern "C" int pico_peak_read(const void* buf, long long bytes, void* sink, int blocks, hipStream_t stream) {
  PICO_REQUIRE(bytes >= 16 && blocks > 0 && blocks <= 65535 * 16, "pico_peak_read: bad sizes");
  PICO_REQUIRE((uintptr_t)buf % 16 == 0, "pico_peak_read: the buffer must be 16-byte aligned");
  peak_read_kernel<<<blocks, 256, 0, stream>>>((const pk_u32x4*)buf, bytes / 16, (uint32_t*)sink);
  PICO_LAUNCH_CHECK();
  return 0;
}

// `iters` rounds of eight independent v_mfma_f32_32x32x16_bf16 per wave (eight accumulators, so that a product
// never waits for the one before it), four waves a workgroup.  One product is 2 * 32 * 32 * 16 flops.
__global__ __launch_bounds__(256) void peak_mfma_kernel(int iters, float* __restrict__ sink) {
  pk_f32x16 acc[8];
#pragma unroll
  for (int a = 0; a < 8; a++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[a][r] = 0.f;
  const uint32_t seed = 0x3f803f80u + threadIdx.x;          // two bfloat16 near one
  pk_bf16x8 x = __builtin_bit_cast(pk_bf16x8, pk_u32x4{seed, seed, seed, seed});
  pk_bf16x8 y = __builtin_bit_cast(pk_bf16x8, pk_u32x4{seed ^ 1u, seed, seed ^ 1u, seed});
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int a = 0; a < 8; a++) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[a], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int a = 0; a < 8; a++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[a][r];
  if (s == 12345.678f) sink[0] = s;                          // never true; keeps the products alive
}

extern "C" long long pico_peak_mfma_flops(int blocks, int iters) {
  return (long long)blocks * 4 * iters * 8 * (2LL * 32 * 32 * 16);
}

extern "C" int pico_peak_mfma(int blocks, int iters, void* sink, hipStream_t stream) {
  PICO_REQUIRE(blocks > 0 && iters > 0, "pico_peak_mfma: bad sizes");
  peak_mfma_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  PICO_LAUNCH_CHECK();
  return 0;
}
