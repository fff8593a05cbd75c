// Shared helpers of the HIP kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define PICO_DTYPE_F32 0
#define PICO_DTYPE_BF16 1

// Every entry point returns 0 on success, or a negative code after storing a message
// that pico_last_error() hands out.
extern "C" const char* pico_last_error();
void pico_set_error(const char* fmt, ...);

#define PICO_REQUIRE(cond, ...)        \
  do {                                 \
    if (!(cond)) {                     \
      pico_set_error(__VA_ARGS__);     \
      return -1;                       \
    }                                  \
  } while (0)

#define PICO_LAUNCH_CHECK()                                              \
  do {                                                                   \
    hipError_t e__ = hipGetLastError();                                  \
    if (e__ != hipSuccess) {                                             \
      pico_set_error("%s: launch failed: %s", __func__, hipGetErrorString(e__)); \
      return -2;                                                         \
    }                                                                    \
  } while (0)

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even; on gfx950 the cast is one v_cvt_pk_bf16_f32
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

// two floats as two bfloat16 in one 32-bit word (a in the low half)
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t));
}

template <typename T> __device__ __forceinline__ float load_f32(const T* p);
template <> __device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// Reductions over a 64-lane wave; every lane gets the result.  The order of the
// additions is fixed, so results do not depend on anything but the inputs.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sum over a workgroup of up to 1024 threads (blockDim.x a multiple of 64);
// scratch holds 16 floats of LDS.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; i++) t += scratch[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nw; i++) t = fmaxf(t, scratch[i]);
  return t;
}
