// Row-wise and element-wise kernels: embedding gather, RMSNorm with optional fused
// residual add, SwiGLU, and rotate-half position encoding fused with the store of
// keys and values into the paged cache.  All arithmetic is float32; T is the storage
// type of activations (float or raw bfloat16 bits).  The residual stream is float32
// in both engine dtypes.
#include "common.h"

// ---------------------------------------------------------------------------
// embedding: out[t, :] = table[ids[t], :] * scale as float32.  An id outside [0, V) gives a
// row of zeros (the host checks ids before a step; this only keeps the kernel in bounds).
// Reference: nn.Embedding lookup, pico_vllm/model.py:427.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                 float* __restrict__ out, int H, int V, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (size_t)(ok ? id : 0) * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = ok ? load_f32(row + i) * scale : 0.f;
}

extern "C" int pico_embedding(const void* table, int table_dtype, const int* ids, float* out, int T, int H,
                              int V, float scale, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && V > 0, "pico_embedding: bad sizes T=%d H=%d V=%d", T, H, V);
  if (T == 0) return 0;
  if (table_dtype == PICO_DTYPE_F32)
    embedding_kernel<float><<<T, 256, 0, stream>>>((const float*)table, ids, out, H, V, scale);
  else if (table_dtype == PICO_DTYPE_BF16)
    embedding_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)table, ids, out, H, V, scale);
  else
    PICO_REQUIRE(false, "pico_embedding: unknown dtype %d", table_dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// RMSNorm: y = x / sqrt(mean(x^2) + eps) * w   (pico_vllm/RMSNorm.py:22-31)
// with the residual sum fused in front (the reference has such a kernel,
// kernels/fused_add_norm.py:21-36, but does not call it):
//   rows == nullptr:  resid[t] += delta[t] (if delta);  out[t] = norm(resid[t])
//   rows != nullptr:  out[i] = norm(resid[rows[i]] + delta[rows[i]]);  resid unchanged
// delta may come as `slabs` partial sums (slab s at delta + s * slab_stride), which a GEMM that
// splits its k range over workgroups leaves behind; they are added in slab order.
// One workgroup per row.  The sum of squares is taken over the float32 sum.
// ---------------------------------------------------------------------------
#define MAX_SLABS 8

template <typename TD> __device__ __forceinline__ float4 load4_f32(const TD* p);
template <> __device__ __forceinline__ float4 load4_f32<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4_f32<bf16_t>(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
template <typename TO> __device__ __forceinline__ void store4_f32(TO* p, float4 v);
template <> __device__ __forceinline__ void store4_f32<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void store4_f32<bf16_t>(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v.x, v.y), pack2_bf16(v.z, v.w));
}

// VEC: rows are handled four elements at a time (H % 4 == 0, so every row starts on 16 bytes).
template <typename TD, typename TO, bool VEC, int VPT = 4>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   const float* __restrict__ w, TO* __restrict__ out,
                                   const int* __restrict__ rows, int H, float eps, int slabs, size_t slab_stride) {
  __shared__ float scratch[16];
  const int src = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)src * H;
  const TD* dl = delta ? delta + (size_t)src * H : nullptr;
  TO* o = out + (size_t)blockIdx.x * H;
  float ss = 0.f;
  if (VEC) {
    // The launch gives a row H / 4 threads (up to 1024), so that a thread holds one group of four
    // elements (up to VPT for a longer row) from the sum of squares to the scaling, and everything
    // it needs (stream, slabs, weight) is requested before it waits for anything.
    const int stride = blockDim.x * 4;
    if (H <= VPT * stride) {
      float4 v[VPT], g[VPT];
#pragma unroll
      for (int j = 0; j < VPT; j++) {
        const int i = threadIdx.x * 4 + j * stride;
        v[j] = g[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (j * stride < H && i < H) {
          v[j] = *reinterpret_cast<const float4*>(x + i);
          g[j] = *reinterpret_cast<const float4*>(w + i);
          if (dl) {
            float4 d[MAX_SLABS];
#pragma unroll
            for (int s = 0; s < MAX_SLABS; s++)
              d[s] = s < slabs ? load4_f32(dl + s * slab_stride + i) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int s = 0; s < MAX_SLABS; s++) { v[j].x += d[s].x; v[j].y += d[s].y; v[j].z += d[s].z; v[j].w += d[s].w; }
            if (!rows) *reinterpret_cast<float4*>(x + i) = v[j];
          }
          ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
        }
      }
      ss = block_sum(ss, scratch);
      const float r = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
      for (int j = 0; j < VPT; j++) {
        const int i = threadIdx.x * 4 + j * stride;
        if (j * stride < H && i < H)
          store4_f32(o + i, make_float4(v[j].x * r * g[j].x, v[j].y * r * g[j].y, v[j].z * r * g[j].z, v[j].w * r * g[j].w));
      }
      return;
    }
    // a row longer than 16384 elements is read twice
    for (int i = threadIdx.x * 4; i < H; i += stride) {
      float4 v = *reinterpret_cast<const float4*>(x + i);
      if (dl) {
        for (int s = 0; s < slabs; s++) {
          const float4 d = load4_f32(dl + s * slab_stride + i);
          v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        if (!rows) *reinterpret_cast<float4*>(x + i) = v;
      }
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = block_sum(ss, scratch);
    const float r = 1.0f / sqrtf(ss / (float)H + eps);
    for (int i = threadIdx.x * 4; i < H; i += stride) {
      float4 v = *reinterpret_cast<const float4*>(x + i);
      if (dl && rows) {
        for (int s = 0; s < slabs; s++) {
          const float4 d = load4_f32(dl + s * slab_stride + i);
          v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
      }
      const float4 g = *reinterpret_cast<const float4*>(w + i);
      store4_f32(o + i, make_float4(v.x * r * g.x, v.y * r * g.y, v.z * r * g.z, v.w * r * g.w));
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (dl) {
      for (int s = 0; s < slabs; s++) v += load_f32(dl + s * slab_stride + i);
      if (!rows) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (dl && rows)
      for (int s = 0; s < slabs; s++) v += load_f32(dl + s * slab_stride + i);
    store_f32(o + i, v * r * w[i]);
  }
}

extern "C" int pico_add_rmsnorm(float* resid, const void* delta, int delta_dtype, int slabs, long long slab_stride,
                                const float* w, void* out, int out_dtype, const int* rows, int T, int H, float eps,
                                hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0, "pico_add_rmsnorm: bad sizes T=%d H=%d", T, H);
  PICO_REQUIRE(slabs >= 1 && slabs <= MAX_SLABS && slab_stride >= 0, "pico_add_rmsnorm: 1 to %d slabs, got %d", MAX_SLABS, slabs);
  const bool vec = H % 4 == 0 && (uintptr_t)resid % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0 &&
                   (uintptr_t)delta % 16 == 0 && slab_stride % 4 == 0;
  PICO_REQUIRE(eps > 0.f, "pico_add_rmsnorm: eps must be positive");
  if (T == 0) return 0;
  // vector path: one thread per four elements, in whole waves, up to 1024
  const int threads = vec ? min(1024, max(64, (H / 4 + 63) / 64 * 64)) : (H >= 4096 ? 512 : (H >= 1024 ? 256 : 128));
  // groups of four elements per thread: one where the row fits (fewer registers, more rows in flight)
  const bool one = vec && H <= threads * 4;
#define LAUNCH(TD, TO)                                                                                                \
  do {                                                                                                                \
    if (one)                                                                                                          \
      add_rmsnorm_kernel<TD, TO, true, 1><<<T, threads, 0, stream>>>(resid, (const TD*)delta, w, (TO*)out, rows, H,   \
                                                                     eps, slabs, (size_t)slab_stride);               \
    else if (vec)                                                                                                     \
      add_rmsnorm_kernel<TD, TO, true><<<T, threads, 0, stream>>>(resid, (const TD*)delta, w, (TO*)out, rows, H, eps, \
                                                                  slabs, (size_t)slab_stride);                       \
    else                                                                                                              \
      add_rmsnorm_kernel<TD, TO, false><<<T, threads, 0, stream>>>(resid, (const TD*)delta, w, (TO*)out, rows, H,    \
                                                                   eps, slabs, (size_t)slab_stride);                 \
  } while (0)
  if (delta_dtype == PICO_DTYPE_F32 && out_dtype == PICO_DTYPE_F32) LAUNCH(float, float);
  else if (delta_dtype == PICO_DTYPE_BF16 && out_dtype == PICO_DTYPE_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == PICO_DTYPE_F32 && out_dtype == PICO_DTYPE_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == PICO_DTYPE_BF16 && out_dtype == PICO_DTYPE_F32) LAUNCH(bf16_t, float);
  else PICO_REQUIRE(false, "pico_add_rmsnorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

// resid[t] += delta[t] without a norm (for an arrangement that ends on an add)
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ resid, const TD* __restrict__ delta, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) resid[i] += load_f32(delta + i);
}

extern "C" int pico_residual_add(float* resid, const void* delta, int delta_dtype, long long n, hipStream_t stream) {
  PICO_REQUIRE(n >= 0, "pico_residual_add: bad size");
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (delta_dtype == PICO_DTYPE_F32)
    residual_add_kernel<float><<<blocks, 256, 0, stream>>>(resid, (const float*)delta, (size_t)n);
  else if (delta_dtype == PICO_DTYPE_BF16)
    residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(resid, (const bf16_t*)delta, (size_t)n);
  else
    PICO_REQUIRE(false, "pico_residual_add: unknown dtype %d", delta_dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// SwiGLU: out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(g) = g * sigmoid(g)
// (pico_vllm/kernels/swiglu.py:22-41: gate is the first half of the last dim).
// ---------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / I, col = idx % I;
  const float g = load_f32(gu + row * 2 * (size_t)I + col);
  const float u = load_f32(gu + row * 2 * (size_t)I + I + col);
  const float s = g / (1.0f + expf(-g));
  store_f32(out + idx, s * u);
}

// bfloat16 rows whose halves start on 16 bytes (I % 8 == 0): eight elements per thread, 16-byte loads and stores
__global__ void swiglu_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int I8, size_t total8) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const size_t row = idx / I8, col = idx % I8;
  const u32x4 g = *reinterpret_cast<const u32x4*>(gu + (row * 2 * I8 + col) * 8);
  const u32x4 u = *reinterpret_cast<const u32x4*>(gu + (row * 2 * I8 + I8 + col) * 8);
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float g0 = __uint_as_float(g[i] << 16), g1 = __uint_as_float(g[i] & 0xffff0000u);
    const float u0 = __uint_as_float(u[i] << 16), u1 = __uint_as_float(u[i] & 0xffff0000u);
    o[i] = pack2_bf16(g0 / (1.0f + expf(-g0)) * u0, g1 / (1.0f + expf(-g1)) * u1);
  }
  *reinterpret_cast<u32x4*>(out + idx * 8) = o;
}

extern "C" int pico_swiglu(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && I > 0, "pico_swiglu: bad sizes T=%d I=%d", T, I);
  if (T == 0) return 0;
  const size_t total = (size_t)T * I;
  if (dtype == PICO_DTYPE_BF16 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t total8 = total / 8;
    swiglu_bf16x8_kernel<<<(unsigned)((total8 + 255) / 256), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I / 8, total8);
    PICO_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == PICO_DTYPE_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
  else if (dtype == PICO_DTYPE_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
  else
    PICO_REQUIRE(false, "pico_swiglu: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Rotate-half position encoding of q and k, fused with the store of k and v into the
// paged cache (pico_vllm/kernels/fused_rope_kvcache_store.py:51-101 does this for decode
// only; prefill there uses eager RoPE, model.py:99-124, plus kernels/store_kvcache.py).
//   pair (j, j + rot/2), angle = position * inv_freq[j] in float32:
//     out[j]         = x[j] * cos - x[j + rot/2] * sin
//     out[j + rot/2] = x[j + rot/2] * cos + x[j] * sin
//   entries at index >= rot pass through unrotated.
// Cosine and sine come from a table cos_sin [T][rot/2][2] that pico_rope_table fills once per
// step: every layer of a step rotates by the same angles.
// qkv: [T, (nq + 2 nkv) * d], rows [q heads | k heads | v heads]; q is rotated in place.
// Cache of one layer: K pages [page][kv head][slot in page][d],
//                     V pages [page][kv head][d][slot in page]  (slot contiguous).
// slots[t] = page * P + position % P says where token t's key and value go (the host computes it
// from the block table, as the reference does, pico_vllm/cache.py:143-156); a negative slot means
// "store nothing" (padding rows of a captured batch).
// Grid T; block 256 (one workgroup per token).
// ---------------------------------------------------------------------------
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float2* __restrict__ cos_sin, int half) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float c, s;
    sincosf(pos * inv_freq[j], &s, &c);
    cos_sin[(size_t)t * half + j] = make_float2(c, s);
  }
}

extern "C" int pico_rope_table(const int* positions, const float* inv_freq, float* cos_sin, int T, int half,
                               hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && half >= 0, "pico_rope_table: bad sizes");
  PICO_REQUIRE((uintptr_t)cos_sin % 8 == 0, "pico_rope_table: the table must be 8-byte aligned");
  if (T == 0 || half == 0) return 0;
  rope_table_kernel<<<T, 64, 0, stream>>>(positions, inv_freq, (float2*)cos_sin, half);
  PICO_LAUNCH_CHECK();
  return 0;
}

// a cos - b sin and b cos + a sin with the roundings spelled out (one product rounded, then one fused multiply-add), so
// that the kernel for few tokens and the one with 16-byte accesses give the same bits: left to the compiler, which of
// the two products is fused differs from kernel to kernel
__device__ __forceinline__ float rotate_lo(float a, float b, float c, float s) { return __fmaf_rn(a, c, -__fmul_rn(b, s)); }
__device__ __forceinline__ float rotate_hi(float a, float b, float c, float s) { return __fmaf_rn(b, c, __fmul_rn(a, s)); }

template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, const float2* __restrict__ cos_sin,
                                  const int* __restrict__ slots,
                                  T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int nkv, int d, int rot,
                                  int P, int num_pages) {
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * (nq + 2 * nkv) * d;
  const int half = rot >> 1;
  const float2* cs = cos_sin + (size_t)t * half;
  const int slot = slots[t];
  const int page = slot / P, off = slot % P;
  const bool store = slot >= 0 && page < num_pages;       // not a padding row; the host has checked the rest
  // one pair (j, j + rot/2) of one q or k head per thread and turn; q is rotated in place, k goes to its page
  for (int u = threadIdx.x; u < (nq + nkv) * half; u += blockDim.x) {
    const int head = u / half, j = u - head * half;
    const T* x = row + (size_t)head * d;
    T* o;
    if (head < nq) {
      o = row + (size_t)head * d;
    } else {
      if (!store) continue;
      o = k_cache + (((size_t)page * nkv + (head - nq)) * P + off) * d;
    }
    const float c = cs[j].x, s = cs[j].y;
    const float a = load_f32(x + j), b = load_f32(x + j + half);
    store_f32(o + j, rotate_lo(a, b, c, s));
    store_f32(o + j + half, rotate_hi(a, b, c, s));
  }
  if (!store) return;
  for (int u = threadIdx.x; u < nkv * (d - rot); u += blockDim.x) {      // what is not rotated of k
    const int g = u / (d - rot), j = rot + u % (d - rot);
    k_cache[(((size_t)page * nkv + g) * P + off) * d + j] = row[(size_t)(nq + g) * d + j];
  }
  for (int u = threadIdx.x; u < nkv * d; u += blockDim.x) {
    const int g = u / d, j = u - g * d;
    v_cache[(((size_t)page * nkv + g) * d + j) * P + off] = row[(size_t)(nq + nkv + g) * d + j];
  }
}

// The same for bfloat16 with 16-byte accesses (d and rot / 2 multiples of 8).  A unit of work is 8 consecutive
// head dimensions of one token: a rotated pair of such runs of a q or k head, a run of k that is not rotated,
// or a run of v; every thread takes one unit, so that all loads of the launch are on their way at once (a
// thread that loops over units waits for each one's loads in turn, because its stores may alias the next loads).
// Grid x: blocks of RS_TOK consecutive tokens, grid y: the units of such a block in workgroups of 256.  The
// units of v are numbered with the token fastest, so that the eight 2-byte stores of neighbouring lanes, which
// go to neighbouring slots of a page when the tokens follow one another in a sequence, fall into one 16-byte
// piece of V^T instead of eight 32-byte sectors.
constexpr int RS_TOK = 8;
typedef uint32_t rs_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void rope_store_bf16x8_kernel(bf16_t* __restrict__ qkv, const float2* __restrict__ cos_sin,
                                                                const int* __restrict__ slots, bf16_t* __restrict__ k_cache,
                                                                bf16_t* __restrict__ v_cache, int T, int nq, int nkv, int d,
                                                                int rot, int P, int num_pages) {
  const int t0 = blockIdx.x * RS_TOK;
  const int half = rot >> 1, hc = half >> 3;                 // 8-wide runs in half the rotated part
  const int row_len = (nq + 2 * nkv) * d;
  const int u_rot = (nq + nkv) * hc, u_copy = nkv * ((d - rot) >> 3), u_v = nkv * (d >> 3);
  const int u_qk = RS_TOK * (u_rot + u_copy);
  int u = blockIdx.y * blockDim.x + threadIdx.x;
  if (u < u_qk) {                                            // rotated pairs and the rest of k: token-major
    const int i = u / (u_rot + u_copy), w = u - i * (u_rot + u_copy);
    const int t = t0 + i;
    if (t >= T) return;
    bf16_t* row = qkv + (size_t)t * row_len;
    const int slot = slots[t];
    const int page = slot / P, off = slot % P;
    const bool store = slot >= 0 && page < num_pages;         // not a padding row; the host has checked the rest
    if (w < u_rot) {
      const int head = w / hc, j = (w - head * hc) << 3;
      const bf16_t* x = row + (size_t)head * d;
      bf16_t* o;
      if (head < nq) {
        o = row + (size_t)head * d;
      } else {
        if (!store) return;
        o = k_cache + (((size_t)page * nkv + (head - nq)) * P + off) * d;
      }
      const rs_u32x4 lo = *reinterpret_cast<const rs_u32x4*>(x + j), hi = *reinterpret_cast<const rs_u32x4*>(x + j + half);
      const float4* cs = reinterpret_cast<const float4*>(cos_sin + (size_t)t * half + j);   // (cos, sin) of two dimensions each
      rs_u32x4 olo, ohi;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float4 c2 = cs[e];
        const float a0 = __uint_as_float(lo[e] << 16), a1 = __uint_as_float(lo[e] & 0xffff0000u);
        const float b0 = __uint_as_float(hi[e] << 16), b1 = __uint_as_float(hi[e] & 0xffff0000u);
        olo[e] = pack2_bf16(rotate_lo(a0, b0, c2.x, c2.y), rotate_lo(a1, b1, c2.z, c2.w));
        ohi[e] = pack2_bf16(rotate_hi(a0, b0, c2.x, c2.y), rotate_hi(a1, b1, c2.z, c2.w));
      }
      *reinterpret_cast<rs_u32x4*>(o + j) = olo;
      *reinterpret_cast<rs_u32x4*>(o + j + half) = ohi;
    } else if (store) {
      const int w2 = w - u_rot, per = (d - rot) >> 3;
      const int g = w2 / per, j = rot + ((w2 - g * per) << 3);
      *reinterpret_cast<rs_u32x4*>(k_cache + (((size_t)page * nkv + g) * P + off) * d + j) =
          *reinterpret_cast<const rs_u32x4*>(row + (size_t)(nq + g) * d + j);
    }
    return;
  }
  u -= u_qk;                                                 // v: token fastest
  if (u >= RS_TOK * u_v) return;
  const int i = u % RS_TOK, w = u / RS_TOK;
  const int t = t0 + i;
  if (t >= T) return;
  const int slot = slots[t];
  const int page = slot / P, off = slot % P;
  if (slot < 0 || page >= num_pages) return;
  const int g = w / (d >> 3), j = (w - g * (d >> 3)) << 3;
  const rs_u32x4 v = *reinterpret_cast<const rs_u32x4*>(qkv + (size_t)t * row_len + (size_t)(nq + nkv + g) * d + j);
  bf16_t* o = v_cache + (((size_t)page * nkv + g) * d + j) * P + off;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    o[(size_t)(2 * e) * P] = (bf16_t)(v[e] & 0xffffu);
    o[(size_t)(2 * e + 1) * P] = (bf16_t)(v[e] >> 16);
  }
}

extern "C" int pico_rope_kv_store(void* qkv, int dtype, const float* cos_sin, const int* slots,
                                  void* k_cache, void* v_cache, int T, int nq, int nkv, int d,
                                  int rot, int P, int num_pages, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && d > 0 && P > 0 && num_pages > 0, "pico_rope_kv_store: bad sizes");
  PICO_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "pico_rope_kv_store: rotary size %d does not fit head size %d", rot, d);
  PICO_REQUIRE(rot == 0 || (cos_sin != nullptr && (uintptr_t)cos_sin % 8 == 0), "pico_rope_kv_store: no table of cosines and sines");
  if (T == 0) return 0;
  const dim3 grid(T);
  const int threads = (nq + nkv) * (rot / 2) >= 256 || nkv * d >= 256 ? 256 : 64;
  if (dtype == PICO_DTYPE_F32)
    rope_store_kernel<float><<<grid, threads, 0, stream>>>((float*)qkv, (const float2*)cos_sin, slots, (float*)k_cache,
                                                      (float*)v_cache, nq, nkv, d, rot, P, num_pages);
  else if (dtype == PICO_DTYPE_BF16 && T >= RS_TOK && d % 8 == 0 && rot % 16 == 0 && (uintptr_t)qkv % 16 == 0 &&
           (uintptr_t)k_cache % 16 == 0 && (rot == 0 || (uintptr_t)cos_sin % 16 == 0))
    rope_store_bf16x8_kernel<<<dim3((T + RS_TOK - 1) / RS_TOK, (RS_TOK * ((nq + nkv) * (rot / 16) + nkv * ((d - rot) / 8) + nkv * (d / 8)) + 255) / 256),
                               256, 0, stream>>>(
        (bf16_t*)qkv, (const float2*)cos_sin, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, T, nq, nkv, d, rot, P, num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    rope_store_kernel<bf16_t><<<grid, threads, 0, stream>>>((bf16_t*)qkv, (const float2*)cos_sin, slots, (bf16_t*)k_cache,
                                                       (bf16_t*)v_cache, nq, nkv, d, rot, P, num_pages);
  else
    PICO_REQUIRE(false, "pico_rope_kv_store: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}


// ---------------------------------------------------------------------------
// soft cap of logits in place: x = cap * tanh(x / cap), float32 (not used by the reference's model; a model
// description may ask for it)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long long n, float cap, float inv_cap) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    x[i] = cap * tanhf(x[i] * inv_cap);
}

extern "C" int pico_softcap(float* x, long long n, float cap, hipStream_t stream) {
  PICO_REQUIRE(n >= 0 && cap > 0.f, "pico_softcap: bad arguments n=%lld cap=%g", n, (double)cap);
  if (n == 0) return 0;
  const long long blocks = (n + 255) / 256;
  softcap_kernel<<<(int)(blocks < 4096 ? blocks : 4096), 256, 0, stream>>>(x, n, cap, 1.0f / cap);
  PICO_LAUNCH_CHECK();
  return 0;
}
