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

// A value combined with the one 16 (32) lanes across, in both lanes: one vector instruction of gfx950
// (v_permlane16_swap / v_permlane32_swap give both values in two registers) where an exchange through the LDS crossbar
// (what __shfl_xor compiles to) waits in line behind the tiles' reads.  Maximum and sum are symmetric, so both lanes
// get the same bits.
__device__ __forceinline__ float max_across_16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_across_32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_across_16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_across_32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The value of another lane of the same row of 16, by a pattern that is part of the instruction (DPP): lane ^ 1,
// lane ^ 2, 7 - lane within a half row, 15 - lane within the row.
template <int PATTERN>
__device__ __forceinline__ float lane_pattern(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), PATTERN, 0xf, 0xf, true));
}
constexpr int LANE_XOR_1 = 0xB1, LANE_XOR_2 = 0x4E, HALF_ROW_MIRROR = 0x141, ROW_MIRROR = 0x140;

// Reductions over a 64-lane wave; every lane gets the result, the same bits in every lane (each step combines two
// values that are the same on both sides).  The order of the additions is fixed, so results do not depend on
// anything but the inputs.  Pairs, quads, half rows and rows of 16 by lane patterns, then the rows by the lane
// swaps above: six vector instructions, where six exchanges through the LDS crossbar made a chain of their latencies.
__device__ __forceinline__ float wave_sum(float v) {
  v += lane_pattern<LANE_XOR_1>(v);
  v += lane_pattern<LANE_XOR_2>(v);
  v += lane_pattern<HALF_ROW_MIRROR>(v);
  v += lane_pattern<ROW_MIRROR>(v);
  return sum_across_32(sum_across_16(v));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lane_pattern<LANE_XOR_1>(v));
  v = fmaxf(v, lane_pattern<LANE_XOR_2>(v));
  v = fmaxf(v, lane_pattern<HALF_ROW_MIRROR>(v));
  v = fmaxf(v, lane_pattern<ROW_MIRROR>(v));
  return max_across_32(max_across_16(v));
}

// The first maximum of a wave (the lowest index among equal values); every lane gets it.  The same steps as above.
__device__ __forceinline__ void keep_first_max(float& mx, int& mi, float ov, int oi) {
  if (ov > mx || (ov == mx && oi < mi)) { mx = ov; mi = oi; }
}
template <int PATTERN>
__device__ __forceinline__ void first_max_step(float& mx, int& mi) {
  const float ov = lane_pattern<PATTERN>(mx);
  const int oi = (int)__builtin_amdgcn_update_dpp(0u, (uint32_t)mi, PATTERN, 0xf, 0xf, true);
  keep_first_max(mx, mi, ov, oi);
}
__device__ __forceinline__ void wave_first_max(float& mx, int& mi) {
  first_max_step<LANE_XOR_1>(mx, mi);
  first_max_step<LANE_XOR_2>(mx, mi);
  first_max_step<HALF_ROW_MIRROR>(mx, mi);
  first_max_step<ROW_MIRROR>(mx, mi);
  {
    const auto v = __builtin_amdgcn_permlane16_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    const auto i = __builtin_amdgcn_permlane16_swap((uint32_t)mi, (uint32_t)mi, false, false);
    mx = __uint_as_float(v[0]); mi = (int)i[0];
    keep_first_max(mx, mi, __uint_as_float(v[1]), (int)i[1]);
  }
  {
    const auto v = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    const auto i = __builtin_amdgcn_permlane32_swap((uint32_t)mi, (uint32_t)mi, false, false);
    mx = __uint_as_float(v[0]); mi = (int)i[0];
    keep_first_max(mx, mi, __uint_as_float(v[1]), (int)i[1]);
  }
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
