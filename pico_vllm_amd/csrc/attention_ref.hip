// Plain paged attention: one wave per (query token, query head), float32 arithmetic.
// It serves every batch shape (prompt portions beside decode tokens), any head size up to
// 256, any page size, an optional window.  It is the attention of the 32-bit engine and the
// fallback of the bfloat16 engine for sizes the matrix-core kernels refuse.
//
//   query head h reads kv head h / (nq / nkv)              (pico_vllm/kernels/attention.py:31,139)
//   s_k = (q . K_k) * scale, keys k <= position visible     (attention.py:190-197)
//   window > 0: only keys k > position - window
//   online softmax over blocks of keys, o = sum p_k V_k / sum p_k   (attention.py:199-211)
//
// Keys are visited in blocks of 64 aligned to absolute positions, so the result at a
// position does not depend on how the sequence was cut into steps.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_ref_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ positions,
    const int* __restrict__ token_seq, T* __restrict__ out, int nq, int nkv, int d, int P, int window, float scale,
    int num_pages) {
  extern __shared__ float lds[];
  float* qs = lds;       // [d]
  float* ps = lds + d;   // [64]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (nq / nkv);
  const int pos = positions[t];
  const int* bt = block_table + (size_t)token_seq[t] * max_pages;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const T* qrow = q + (size_t)t * q_stride + (size_t)h * d;
  for (int j = lane; j < d; j += 64) qs[j] = load_f32(qrow + j);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = (lo / 64) * 64; c0 <= pos; c0 += 64) {
    const int key = c0 + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      int page = bt[key / P];
      page = min(max(page, 0), num_pages - 1);
      const T* kp = k_cache + (((size_t)page * nkv + g) * P + key % P) * d;
      float dot = 0.f;
      for (int j = 0; j < d; j++) dot = fmaf(qs[j], load_f32(kp + j), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    // the block's part of P V is summed on its own and then joins the running sum: two short sums instead of one
    // over the whole context
    float blk[4] = {0.f, 0.f, 0.f, 0.f};
    const int kend = min(64, pos - c0 + 1);
    for (int kk = max(0, lo - c0); kk < kend; kk++) {
      const int kpos = c0 + kk;
      int page = bt[kpos / P];
      page = min(max(page, 0), num_pages - 1);
      const T* vp = v_cache + ((size_t)page * nkv + g) * d * P + kpos % P;
      const float pk = ps[kk];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int dim = lane + 64 * i;
        if (dim < d) blk[i] = fmaf(pk, load_f32(vp + (size_t)dim * P), blk[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = fmaf(acc[i], alpha, blk[i]);
    m = m_new;
  }
  T* o = out + ((size_t)t * nq + h) * d;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int dim = lane + 64 * i;
    if (dim < d) store_f32(o + dim, acc[i] / l);
  }
}

extern "C" int pico_paged_attention_ref(const void* q, int q_stride, int dtype, const void* k_cache,
                                        const void* v_cache, const int* block_table, int max_pages,
                                        const int* positions, const int* token_seq, void* out, int T, int nq,
                                        int nkv, int d, int P, int window, float scale, int num_pages,
                                        hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && d > 0 && P > 0 && max_pages > 0 && num_pages > 0,
               "pico_paged_attention_ref: bad sizes");
  PICO_REQUIRE(nq % nkv == 0, "pico_paged_attention_ref: %d query heads are not a multiple of %d kv heads", nq, nkv);
  PICO_REQUIRE(d <= 256, "pico_paged_attention_ref: head size %d is larger than 256", d);
  PICO_REQUIRE(nq <= 65535, "pico_paged_attention_ref: too many heads");
  PICO_REQUIRE(q_stride >= nq * d, "pico_paged_attention_ref: query row stride too small");
  if (T == 0) return 0;
  dim3 grid(T, nq);
  const size_t lds = (size_t)(d + 64) * sizeof(float);
  if (dtype == PICO_DTYPE_F32)
    paged_attention_ref_kernel<float><<<grid, 64, lds, stream>>>(
        (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, block_table, max_pages, positions,
        token_seq, (float*)out, nq, nkv, d, P, window, scale, num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    paged_attention_ref_kernel<bf16_t><<<grid, 64, lds, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages,
        positions, token_seq, (bf16_t*)out, nq, nkv, d, P, window, scale, num_pages);
  else
    PICO_REQUIRE(false, "pico_paged_attention_ref: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
