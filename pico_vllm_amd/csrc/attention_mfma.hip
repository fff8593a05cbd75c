// Paged attention on the matrix cores for bfloat16, specialised at compile time for one head
// size D = PICO_HEAD_DIM (a multiple of 16 up to 256).  Two kernels share the tile code:
//
//   prefill / mixed  one workgroup (4 waves) per 128 query tokens of one sequence and one query
//                    head; each wave owns 32 queries; keys and values of the sequence stream
//                    through LDS in tiles of BN keys, from position 0 to the causal frontier.
//                    A decode token is a sequence that brings one query.
//   decode           one workgroup per (sequence, kv head, split of the context); the
//                    "queries" are the G query heads that share the kv head, so keys and values
//                    are read once for the whole group (the reference's kernel re-reads them per
//                    query head, pico_vllm/kernels/attention.py:96-105); two waves split the keys of a tile
//                    (the other two only help to move tiles);
//                    partial (max, sum, output) per split are merged by a second kernel.
//
// Formulas as in pico_vllm/kernels/attention.py:136-213: scores (q.k) * scale, key visible iff its
// position <= the query's, online softmax in float32, probabilities rounded to bfloat16 for the
// P.V product, float32 accumulators.
//
// Matrix-core layout (v_mfma_f32_32x32x16_bf16, D = A B, A 32x16, B 16x32): lane l supplies
// A[l % 32][8 (l / 32) + 0..7] and B[8 (l / 32) + 0..7][l % 32]; it receives, in register r,
// D[8 (r / 4) + 4 (l / 32) + r % 4][l % 32].  Scores are computed TRANSPOSED, S^T = K Q^T, so a
// query is a column: its 32 scores of a key tile sit in the 16 registers of two lanes (l, l ^ 32)
// and the softmax needs one exchange across lanes.  The same registers, rounded to bfloat16, ARE
// the B operand of O^T += V^T P^T if the contraction index runs over the keys in the order in
// which the registers hold them; V^T is read from LDS in that order.  That is why the cache
// keeps V transposed inside a page ([head size][slot]).
#include "common.h"

#ifndef PICO_HEAD_DIM
#error "compile with -DPICO_HEAD_DIM=<head size>"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int D = PICO_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 up to 256");
constexpr int DP = (D + 31) / 32 * 32;   // head size padded to whole 32-wide output tiles
constexpr int KSTEPS = D / 16;           // contraction steps of K Q^T
constexpr int DT = DP / 32;              // 32-wide tiles of the output's head dimension
constexpr int BN = D <= 128 ? 64 : 32;   // keys per LDS tile
constexpr int KROW = D + 8;              // LDS row strides in elements; the pad spreads rows over banks
constexpr int VROW = BN + 8;
constexpr int BM = 128;                  // queries per workgroup in the prefill kernel
#if PICO_HEAD_DIM > 128
#define PICO_ATTN_WAVES_PER_SIMD 1       // accumulators of a large head need the whole register file
#else
#define PICO_ATTN_WAVES_PER_SIMD 2
#endif

struct alignas(16) Tiles {
  alignas(16) bf16_t k[BN * KROW];    // [key][dim]
  alignas(16) bf16_t vt[DP * VROW];   // [dim][key]
};

// A tile of BN keys travels global -> registers (fetch: every thread issues all its 16-byte loads
// before it waits for any) -> LDS (commit).  The fetch of the next tile is issued before the
// current tile is computed, so its latency hides behind the matrix products.
// Positions at or beyond kv_end read as zero (their pages may not exist).  P % 8 == 0 and
// tile_start % 8 == 0, so a 16-byte chunk of V^T (8 keys of one head dimension) lies in one page.
template <int NT>
struct TileRegs {
  static constexpr int KCH = D / 8;                        // 16-byte chunks per key
  static constexpr int VCH = BN / 8;                       // 16-byte chunks (8 keys) per head dimension
  static constexpr int NK = (BN * KCH + NT - 1) / NT;      // chunks per thread
  static constexpr int NV = (D * VCH + NT - 1) / NT;
  uint4 k[NK], v[NV];

  // No branch stands between the loads: chunks that do not exist (beyond the tile's chunk count or
  // beyond kv_end) read a clamped, valid address instead.  Keys beyond kv_end need no zeroing, their
  // scores are masked; values do, which commit() takes care of.
  __device__ __forceinline__ void fetch(const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                        const int* __restrict__ bt, int g, int nkv, int pshift, int num_pages,
                                        int tile_start, int kv_end) {
    const int P = 1 << pshift, last_key = kv_end - 1, last_chunk = last_key & ~7;
#pragma unroll
    for (int i = 0; i < NK; i++) {
      const int c = min((int)threadIdx.x + i * NT, BN * KCH - 1);
      const int pos = min(tile_start + c / KCH, last_key);
      const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
      k[i] = *reinterpret_cast<const uint4*>(k_cache + ((((size_t)page * nkv + g) << pshift) + (pos & (P - 1))) * D +
                                             (c % KCH) * 8);
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int c = min((int)threadIdx.x + i * NT, D * VCH - 1);
      const int pos = min(tile_start + (c % VCH) * 8, last_chunk);
      const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
      v[i] = *reinterpret_cast<const uint4*>(v_cache + ((((size_t)page * nkv + g) * D + c / VCH) << pshift) + (pos & (P - 1)));
    }
  }

  // LDS layout of V^T: per head dimension a row of BN values in OPERAND order: the 8 values that lane
  // half h feeds into product m of sub-tile sub (keys 16 m + 4 h + 0..3 and 16 m + 8 + 4 h + 0..3 of the
  // sub-tile) are contiguous, so the P.V loop reads one 16-byte unit per product.  A chunk from
  // memory (8 consecutive keys) splits into two 8-byte halves that go to the units of h = 0 and 1.
  __device__ __forceinline__ void commit(Tiles& t, int tile_start, int kv_end) const {
#pragma unroll
    for (int i = 0; i < NK; i++) {
      const int c = threadIdx.x + i * NT;
      if (c < BN * KCH) *reinterpret_cast<uint4*>(&t.k[(c / KCH) * KROW + (c % KCH) * 8]) = k[i];
    }
    const bool tail = tile_start + BN > kv_end;              // the same for the whole workgroup
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int c = threadIdx.x + i * NT;
      if (c >= D * VCH) continue;
      const int dim = c / VCH, kc = c % VCH;
      uint4 x = v[i];
      if (tail) {   // values of keys at or beyond kv_end hold whatever the page held before
        const int pos = tile_start + kc * 8;
        uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (pos + e >= kv_end) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
        x = make_uint4(w[0], w[1], w[2], w[3]);
      }
      // chunk kc covers keys 8 kc .. 8 kc + 7 of the tile: sub-tile kc / 4, product (kc % 4) / 2,
      // first or second group of four slots by kc % 2
      bf16_t* unit = &t.vt[dim * VROW + (kc >> 1) * 16 + (kc & 1) * 4];
      *reinterpret_cast<uint2*>(unit) = make_uint2(x.x, x.y);          // keys +0..3: half h = 0
      *reinterpret_cast<uint2*>(unit + 8) = make_uint2(x.z, x.w);      // keys +4..7: half h = 1
    }
  }
};

__device__ __forceinline__ void zero_pad_rows(Tiles& t, int nthreads) {
  if (DP > D)
    for (int i = threadIdx.x; i < (DP - D) * VROW; i += nthreads) t.vt[D * VROW + i] = 0;
}

// State of one wave: 32 query columns; lane l and lane l ^ 32 share column l % 32.
struct WaveState {
  float m, l;        // running maximum and sum of the column
  f32x16 o[DT];      // O^T tiles: rows = head dimension, column = query
};

__device__ __forceinline__ void init_state(WaveState& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int t = 0; t < DT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) st.o[t][r] = 0.f;
}

// One 32-key sub-tile (keys sub * 32 .. + 31 of the LDS tile) against the wave's 32 query columns.
// q[step] is the B operand of step `step`; key_pos0 the absolute position of the sub-tile's first
// key; q_pos the absolute position of this lane's query column (keys beyond it are masked).
__device__ __forceinline__ void attend_subtile(const Tiles& t, int sub, const bf16x8* q, WaveState& st, float scale,
                                               int key_pos0, int q_pos, bool need_mask) {
  const int lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  f32x16 s;
#pragma unroll
  for (int r = 0; r < 16; r++) s[r] = 0.f;
  const bf16_t* krow = &t.k[(sub * 32 + col) * KROW + 8 * h];
#pragma unroll
  for (int step = 0; step < KSTEPS; step++) {
    const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow + 16 * step));
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, q[step], s, 0, 0, 0);
  }
  float mx = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    float v = s[r] * scale;
    if (need_mask) {
      const int kpos = key_pos0 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (kpos > q_pos) v = -INFINITY;
    }
    s[r] = v;
    mx = fmaxf(mx, v);
  }
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  const float m_new = fmaxf(st.m, mx);
  const float m_use = (m_new == -INFINITY) ? 0.f : m_new;   // a column with nothing visible yet
  const float alpha = __expf(st.m - m_use);
  float sum = 0.f;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const float p = __expf(s[r] - m_use);
    s[r] = p;
    sum += p;
  }
  sum += __shfl_xor(sum, 32, 64);
  st.l = st.l * alpha + sum;
  st.m = m_new;
#pragma unroll
  for (int tt = 0; tt < DT; tt++)
#pragma unroll
    for (int r = 0; r < 16; r++) st.o[tt][r] *= alpha;
  // P^T as B operand: contraction slot kk of half h in product m is key 16 m + 8 (kk / 4) + 4 h + kk % 4,
  // which is register 8 m + kk of this lane.
#pragma unroll
  for (int m = 0; m < 2; m++) {
    uint32_t pk[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
      pk[i] = pack2_bf16(s[8 * m + 2 * i], s[8 * m + 2 * i + 1]);
    const bf16x8 b = __builtin_bit_cast(bf16x8, make_uint4(pk[0], pk[1], pk[2], pk[3]));
#pragma unroll
    for (int tt = 0; tt < DT; tt++) {
      const bf16x8 a = __builtin_bit_cast(
          bf16x8, *reinterpret_cast<const uint4*>(&t.vt[(tt * 32 + col) * VROW + sub * 32 + 16 * m + 8 * h]));
      st.o[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, st.o[tt], 0, 0, 0);
    }
  }
}

// A whole LDS tile (its first nsub 32-key sub-tiles) against the wave's 32 query columns with ONE
// softmax update, for the prefill kernel, whose cost is vector instructions rather than matrix ones:
//   * scores stay raw; p = 2^(s c - m c) with c = scale * log2(e) is one fused multiply-add and
//     one v_exp_f32 per score;
//   * the reference maximum m may lag behind the true running maximum by up to 8 in the exponent
//     (p <= 256, harmless in float32 sums and in bfloat16 P); the accumulators are rescaled only
//     when some column of the wave outgrows that, which after the first tiles of a row is rare.
//     Output and sum share the reference, so o / l is unchanged by the lag.
template <int NS>
__device__ __forceinline__ void attend_tile(const Tiles& t, int nsub, const bf16x8* q, WaveState& st, float c,
                                            int key_pos0, int q_pos, bool need_mask) {
  const int lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  f32x16 s[NS];
#pragma unroll
  for (int sub = 0; sub < NS; sub++) {
#pragma unroll
    for (int r = 0; r < 16; r++) s[sub][r] = 0.f;
    if (sub < nsub) {
      const bf16_t* krow = &t.k[(sub * 32 + col) * KROW + 8 * h];
#pragma unroll
      for (int step = 0; step < KSTEPS; step++) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow + 16 * step));
        s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, q[step], s[sub], 0, 0, 0);
      }
    }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int sub = 0; sub < NS; sub++) {
    if (sub < nsub) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        if (need_mask && key_pos0 + 32 * sub + 8 * (r >> 2) + 4 * h + (r & 3) > q_pos) s[sub][r] = -INFINITY;
        mx = fmaxf(mx, s[sub][r]);
      }
    }
  }
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  const float m_new = fmaxf(st.m, mx);
  const bool outgrown = (m_new - st.m) * c > 8.0f;          // also true while the reference is -inf
  if (__builtin_amdgcn_ballot_w64(outgrown) != 0) {          // the same decision for the whole wave
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((st.m - m_use) * c);
    st.l *= alpha;
    st.m = m_new;
#pragma unroll
    for (int tt = 0; tt < DT; tt++)
#pragma unroll
      for (int r = 0; r < 16; r++) st.o[tt][r] *= alpha;
  }
  const float mc = ((st.m == -INFINITY) ? 0.f : st.m) * c;
  float sum = 0.f;
#pragma unroll
  for (int sub = 0; sub < NS; sub++) {
    if (sub < nsub) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[sub][r], c, -mc));
        s[sub][r] = p;
        sum += p;
      }
    }
  }
  sum += __shfl_xor(sum, 32, 64);
  st.l += sum;
#pragma unroll
  for (int sub = 0; sub < NS; sub++) {
    if (sub < nsub) {
#pragma unroll
      for (int m = 0; m < 2; m++) {
        const bf16x8 b = __builtin_bit_cast(
            bf16x8, make_uint4(pack2_bf16(s[sub][8 * m], s[sub][8 * m + 1]), pack2_bf16(s[sub][8 * m + 2], s[sub][8 * m + 3]),
                               pack2_bf16(s[sub][8 * m + 4], s[sub][8 * m + 5]), pack2_bf16(s[sub][8 * m + 6], s[sub][8 * m + 7])));
#pragma unroll
        for (int tt = 0; tt < DT; tt++) {
          const bf16x8 a = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4*>(&t.vt[(tt * 32 + col) * VROW + sub * 32 + 16 * m + 8 * h]));
          st.o[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, st.o[tt], 0, 0, 0);
        }
      }
    }
  }
}

// Q^T operand of one query row: 8 consecutive head dimensions per step, 16-byte loads.
__device__ __forceinline__ void load_q(bf16x8* q, const bf16_t* qrow, bool ok) {
  const int h = (threadIdx.x & 63) >> 5;
#pragma unroll
  for (int step = 0; step < KSTEPS; step++) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (ok) v = *reinterpret_cast<const uint4*>(qrow + 16 * step + 8 * h);
    q[step] = __builtin_bit_cast(bf16x8, v);
  }
}

// ---------------------------------------------------------------------------
// prefill / mixed batches
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256, PICO_ATTN_WAVES_PER_SIMD) void prefill_kernel(const bf16_t* __restrict__ q, int q_stride,
                                                      const bf16_t* __restrict__ k_cache,
                                                      const bf16_t* __restrict__ v_cache,
                                                      const int* __restrict__ block_table, int max_pages,
                                                      const int* __restrict__ cu_seqlens,
                                                      const int* __restrict__ context_lens, int num_seqs,
                                                      bf16_t* __restrict__ out, int nq, int nkv, int P,
                                                      int num_pages, float scale) {
  __shared__ Tiles tiles;
  // which (sequence, query tile) is this workgroup?  heavy (late) tiles of a sequence come first
  int b = 0, tile = (int)blockIdx.x, ntiles = 0;
  for (; b < num_seqs; b++) {
    ntiles = (cu_seqlens[b + 1] - cu_seqlens[b] + BM - 1) / BM;
    if (tile < ntiles) break;
    tile -= ntiles;
  }
  if (b >= num_seqs) return;
  tile = ntiles - 1 - tile;
  const int head = blockIdx.y, g = head / (nq / nkv);
  const int tok0 = cu_seqlens[b], new_len = cu_seqlens[b + 1] - tok0;
  const int ctx = context_lens[b], prefix = ctx - new_len;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int* bt = block_table + (size_t)b * max_pages;

  const int q_idx = tile * BM + wave * 32 + col;          // index among the sequence's new tokens
  const bool q_ok = q_idx < new_len;
  const int q_pos = prefix + q_idx;
  bf16x8 qf[KSTEPS];
  load_q(qf, q + (size_t)(tok0 + (q_ok ? q_idx : 0)) * q_stride + (size_t)head * D, q_ok);
  const int wave_first_pos = prefix + tile * BM + wave * 32;            // lowest query position of the wave
  const int wave_last_pos = min(wave_first_pos + 31, ctx - 1);          // highest real one
  const bool wave_active = tile * BM + wave * 32 < new_len;
  const int kv_end = min(ctx, prefix + min(new_len, (tile + 1) * BM));  // keys beyond the tile's last query are never needed

  const float c = scale * 1.4426950408889634f;               // scores go through 2^x
  const int pshift = 31 - __clz(P);                          // page sizes are powers of two
  WaveState st;
  init_state(st);
  zero_pad_rows(tiles, 256);
  TileRegs<256> regs;
  regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, 0, kv_end);
  for (int tile_start = 0; tile_start < kv_end; tile_start += BN) {
    __syncthreads();                                          // everyone is done with the previous tile
    regs.commit(tiles, tile_start, kv_end);
    __syncthreads();
    if (tile_start + BN < kv_end) regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, tile_start + BN, kv_end);
    if (!wave_active || tile_start > wave_last_pos) continue;
    // sub-tiles wholly beyond the causal frontier of this wave are left out
    const int nsub = min(BN / 32, (wave_last_pos - tile_start) / 32 + 1);
    attend_tile<BN / 32>(tiles, nsub, qf, st, c, tile_start, q_pos, tile_start + 32 * nsub - 1 > wave_first_pos);
  }
  if (!q_ok) return;
  const float inv_l = 1.0f / st.l;
  bf16_t* orow = out + ((size_t)(tok0 + q_idx) * nq + head) * D;
#pragma unroll
  for (int tt = 0; tt < DT; tt++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      const int dim = tt * 32 + 8 * a + 4 * h;
      if (dim < D) {
        uint2 v;
        v.x = pack2_bf16(st.o[tt][4 * a] * inv_l, st.o[tt][4 * a + 1] * inv_l);
        v.y = pack2_bf16(st.o[tt][4 * a + 2] * inv_l, st.o[tt][4 * a + 3] * inv_l);
        *reinterpret_cast<uint2*>(orow + dim) = v;
      }
    }
}

// ---------------------------------------------------------------------------
// decode: one query token per sequence, the G heads of a kv group as the 32 columns
// ---------------------------------------------------------------------------
// partial results per (sequence, query head, split): o [D] unnormalised, then m and l
__global__ __launch_bounds__(256, PICO_ATTN_WAVES_PER_SIMD) void decode_kernel(const bf16_t* __restrict__ q, int q_stride,
                                                     const bf16_t* __restrict__ k_cache,
                                                     const bf16_t* __restrict__ v_cache,
                                                     const int* __restrict__ block_table, int max_pages,
                                                     const int* __restrict__ context_lens,
                                                     float* __restrict__ part, int nsplit, int nq, int nkv, int P,
                                                     int num_pages, float scale) {
  __shared__ Tiles tiles;
  const int b = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int G = nq / nkv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int ctx = context_lens[b];
  // this split's keys: a whole number of LDS tiles
  const int per = ((ctx + nsplit - 1) / nsplit + BN - 1) / BN * BN;
  const int k_begin = split * per, k_end = min(ctx, k_begin + per);
  const int* bt = block_table + (size_t)b * max_pages;
  const bool col_ok = col < G;
  const int head = g * G + (col_ok ? col : 0);
  const int pshift = 31 - __clz(P);
  bf16x8 qf[KSTEPS];
  load_q(qf, q + (size_t)b * q_stride + (size_t)head * D, col_ok && ctx > 0);

  WaveState st;
  init_state(st);
  zero_pad_rows(tiles, 256);
  TileRegs<256> regs;
  if (k_begin < k_end) regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, k_begin, k_end);
  for (int tile_start = k_begin; tile_start < k_end; tile_start += BN) {
    __syncthreads();
    regs.commit(tiles, tile_start, k_end);
    __syncthreads();
    if (tile_start + BN < k_end) regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, tile_start + BN, k_end);
    for (int sub = wave; sub < BN / 32 && wave < 2; sub += 2) {   // waves 2 and 3 only help to move the tiles
      const int key0 = tile_start + sub * 32;
      if (key0 >= k_end) break;
      // every query sits at position ctx - 1: only keys at or beyond k_end need the mask
      attend_subtile(tiles, sub, qf, st, scale, key0, k_end - 1, key0 + 32 > k_end);
    }
  }
  // merge the two waves through LDS (reusing the tile memory), then write the split's partial result
  __syncthreads();
  float* xo = reinterpret_cast<float*>(&tiles);            // [DP][32] output of wave 1
  float* xm = xo + DP * 32;                                // [32] m, [32] l
  static_assert(sizeof(Tiles) >= (DP * 32 + 64) * sizeof(float), "LDS tile memory too small for the merge");
  if (wave == 1) {
#pragma unroll
    for (int tt = 0; tt < DT; tt++)
#pragma unroll
      for (int r = 0; r < 16; r++) xo[(tt * 32 + 8 * (r >> 2) + 4 * h + (r & 3)) * 32 + col] = st.o[tt][r];
    if (h == 0) { xm[col] = st.m; xm[32 + col] = st.l; }
  }
  __syncthreads();
  if (wave != 0 || !col_ok) return;
  const float m1 = xm[col], l1 = xm[32 + col];
  const float m = fmaxf(st.m, m1);
  const float m_use = (m == -INFINITY) ? 0.f : m;
  const float a0 = __expf(st.m - m_use), a1 = __expf(m1 - m_use);
  const float l = st.l * a0 + l1 * a1;
  float* po = part + (((size_t)b * nq + head) * nsplit + split) * (D + 2);
#pragma unroll
  for (int tt = 0; tt < DT; tt++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int dim = tt * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (dim < D) po[dim] = st.o[tt][r] * a0 + xo[dim * 32 + col] * a1;
    }
  if (h == 0) { po[D] = m; po[D + 1] = l; }
}

// ---------------------------------------------------------------------------
// decode without LDS staging, for up to 16 query heads per kv head and D % 32 == 0
// ---------------------------------------------------------------------------
// v_mfma_f32_16x16x32_bf16 (A 16x32, B 32x16): lane l supplies A[l % 16][8 (l / 16) + 0..7] and
// B[8 (l / 16) + 0..7][l % 16] and receives D[4 (l / 16) + r][l % 16] in register r.  A wave owns
// blocks of 32 keys: two 16-key tiles of S^T = K Q^T (the 16 columns are the query heads of the
// group), then O^T += V^T P^T with the 32 keys as the contraction; as in the other kernels the
// contraction order is the order in which the registers hold the keys, so P never moves.
// Operands come straight from the pages: lane (key, kq) reads the 64 contiguous bytes
// K[key][32 kq ..] (the contraction over the head dimension runs in that permuted order for K
// and Q alike), and lane (dim, kq) reads the 8 bytes V^T[dim][4 kq .. 4 kq + 3] of each tile.
// The loads of a wave's next block are issued while the current block is computed.
#if PICO_HEAD_DIM % 32 == 0 && PICO_HEAD_DIM <= 128
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int KS16 = D / 32;   // contraction steps of a 16-key tile
constexpr int DT16 = D / 16;   // 16-wide tiles of the output's head dimension

__global__ __launch_bounds__(256, 2) void decode16_kernel(const bf16_t* __restrict__ q, int q_stride,
                                                          const bf16_t* __restrict__ k_cache,
                                                          const bf16_t* __restrict__ v_cache,
                                                          const int* __restrict__ block_table, int max_pages,
                                                          const int* __restrict__ context_lens,
                                                          float* __restrict__ part, int nsplit, int nq, int nkv, int P,
                                                          int num_pages, float scale) {
  __shared__ float xo[3][D][16];     // outputs of waves 1..3 for the final merge
  __shared__ float xml[3][2][16];
  const int b = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int G = nq / nkv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 15, kq = lane >> 4;
  const int ctx = context_lens[b];
  const int per = ((ctx + nsplit - 1) / nsplit + 31) / 32 * 32;
  const int k_begin = split * per, k_end = min(ctx, k_begin + per);
  const int* bt = block_table + (size_t)b * max_pages;
  const bool col_ok = col < G;
  const int head = g * G + (col_ok ? col : 0);

  bf16x8 qf[KS16];
  {
    const bf16_t* qrow = q + (size_t)b * q_stride + (size_t)head * D + (D / 4) * kq;
#pragma unroll
    for (int st = 0; st < KS16; st++) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col_ok) v = *reinterpret_cast<const uint4*>(qrow + 8 * st);
      qf[st] = __builtin_bit_cast(bf16x8, v);
    }
  }
  float m = -INFINITY, l = 0.f;
  f32x4 o[DT16];
#pragma unroll
  for (int tt = 0; tt < DT16; tt++) o[tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int first = k_begin + 32 * wave;
  const int pshift = 31 - __clz(P);                             // page sizes are powers of two
  if (first < k_end) {
    const int last = first + (k_end - 1 - first) / 128 * 128;   // this wave's last block
    const int last_key = k_end - 1, last_group = last_key / 4 * 4;
    uint4 kr[2][KS16];
    uint2 vr[DT16][2];
    // positions beyond the split are clamped to its last key (group): the pages exist, the scores are masked
    auto load_k = [&](int key0) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int pos = min(key0 + 16 * t + col, last_key);
        const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
        const bf16_t* kp = k_cache + ((((size_t)page * nkv + g) << pshift) + (pos & (P - 1))) * D + (D / 4) * kq;
#pragma unroll
        for (int st = 0; st < KS16; st++) kr[t][st] = *reinterpret_cast<const uint4*>(kp + 8 * st);
      }
    };
    auto load_v = [&](int key0) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int pos = min(key0 + 16 * t + 4 * kq, last_group);
        const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
        const bf16_t* vp = v_cache + ((((size_t)page * nkv + g) * D + col) << pshift) + (pos & (P - 1));
#pragma unroll
        for (int tt = 0; tt < DT16; tt++) vr[tt][t] = *reinterpret_cast<const uint2*>(vp + ((size_t)tt * 16 << pshift));
      }
    };
    load_k(first);
    __builtin_amdgcn_sched_barrier(0);       // keys before values, as in the loop, so the waits there stay partial
    load_v(first);
    __builtin_amdgcn_sched_barrier(0);
    for (int key0 = first;; key0 += 128) {
      const int next = min(key0 + 128, last);
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
      for (int st = 0; st < KS16; st++) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[0][st]), qf[st], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[1][st]), qf[st], s1, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      load_k(next);
      __builtin_amdgcn_sched_barrier(0);
      const bool tail = key0 + 32 > k_end;                     // the same for the whole wave
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        float v = (r < 4 ? s0[r & 3] : s1[r & 3]) * scale;
        if (tail && key0 + 16 * (r >> 2) + 4 * kq + (r & 3) >= k_end) v = -INFINITY;
        sv[r] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m, mx);                        // finite: the block holds at least one key < k_end
      const float alpha = __expf(m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        sv[r] = __expf(sv[r] - m_new);
        sum += sv[r];
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l = l * alpha + sum;
      m = m_new;
      const bf16x8 pb = __builtin_bit_cast(bf16x8, make_uint4(pack2_bf16(sv[0], sv[1]), pack2_bf16(sv[2], sv[3]),
                                                               pack2_bf16(sv[4], sv[5]), pack2_bf16(sv[6], sv[7])));
      if (tail) {   // values of keys beyond the split hold whatever the page held before: make them zero
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int pos = key0 + 16 * t + 4 * kq;
#pragma unroll
          for (int tt = 0; tt < DT16; tt++) {
            if (pos >= k_end) vr[tt][t] = make_uint2(0, 0);
            else {
              if (pos + 1 >= k_end) vr[tt][t].x &= 0x0000ffffu;
              if (pos + 2 >= k_end) vr[tt][t].y = 0;
              else if (pos + 3 >= k_end) vr[tt][t].y &= 0x0000ffffu;
            }
          }
        }
      }
#pragma unroll
      for (int tt = 0; tt < DT16; tt++) {
        o[tt] *= alpha;
        const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(vr[tt][0].x, vr[tt][0].y, vr[tt][1].x, vr[tt][1].y));
        o[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, o[tt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (key0 >= last) break;
      load_v(next);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // merge the four waves; lane (col, kq) of wave 0 holds head dimensions 16 tt + 4 kq + r of head `col`
  if (wave > 0) {
#pragma unroll
    for (int tt = 0; tt < DT16; tt++)
#pragma unroll
      for (int r = 0; r < 4; r++) xo[wave - 1][16 * tt + 4 * kq + r][col] = o[tt][r];
    if (kq == 0) { xml[wave - 1][0][col] = m; xml[wave - 1][1][col] = l; }
  }
  __syncthreads();
  if (wave != 0 || !col_ok) return;
  float M = m;
#pragma unroll
  for (int w = 0; w < 3; w++) M = fmaxf(M, xml[w][0][col]);
  const float m_use = (M == -INFINITY) ? 0.f : M;
  const float a0 = __expf(m - m_use);
  float aw[3], L = l * a0;
#pragma unroll
  for (int w = 0; w < 3; w++) {
    aw[w] = __expf(xml[w][0][col] - m_use);
    L += xml[w][1][col] * aw[w];
  }
  float* po = part + (((size_t)b * nq + head) * nsplit + split) * (D + 2);
#pragma unroll
  for (int tt = 0; tt < DT16; tt++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int dim = 16 * tt + 4 * kq + r;
      float acc = o[tt][r] * a0;
#pragma unroll
      for (int w = 0; w < 3; w++) acc += xo[w][dim][col] * aw[w];
      po[dim] = acc;
    }
  if (kq == 0) { po[D] = M; po[D + 1] = L; }
}
#endif

// out[b, head, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s; one workgroup per (sequence,
// head).  Every wave weighs all splits (lane s holds split s) and sums a quarter of them for all
// head dimensions, all loads issued together; wave 0 adds the four quarters.
__global__ __launch_bounds__(256) void decode_merge_kernel(const float* __restrict__ part, int nsplit,
                                                           bf16_t* __restrict__ out, int nq) {
  constexpr int DPL = (D + 63) / 64;                        // head dimensions per lane
  __shared__ float quarter[3][DPL * 64];
  const int b = blockIdx.x, head = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* p = part + ((size_t)b * nq + head) * nsplit * (D + 2);
  const bool mine = lane < nsplit;                         // nsplit <= 64
  const float m = mine ? p[lane * (D + 2) + D] : -INFINITY;
  const float l = mine ? p[lane * (D + 2) + D + 1] : 0.f;
  const float M = wave_max(m);
  bf16_t* o = out + ((size_t)b * nq + head) * D;
  if (M == -INFINITY) {   // an empty row (padding of a captured batch)
    if (wave == 0)
      for (int dim = lane; dim < D; dim += 64) o[dim] = 0;
    return;
  }
  const float wt = mine ? __expf(m - M) : 0.f;
  const float L = wave_sum(wt * l);
  float acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; i++) acc[i] = 0.f;
  const int s0 = wave * 16;
  float v[16][DPL];
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int s = min(s0 + j, nsplit - 1);
#pragma unroll
    for (int i = 0; i < DPL; i++) {
      const int dim = lane + 64 * i;
      v[j][i] = dim < D ? p[s * (D + 2) + dim] : 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const float ws = (s0 + j < nsplit) ? __shfl(wt, s0 + j, 64) : 0.f;
#pragma unroll
    for (int i = 0; i < DPL; i++) acc[i] += ws * v[j][i];
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < DPL; i++) quarter[wave - 1][lane + 64 * i] = acc[i];
  }
  __syncthreads();
  if (wave != 0) return;
  const float inv = 1.0f / L;
#pragma unroll
  for (int i = 0; i < DPL; i++) {
    const int dim = lane + 64 * i;
    if (dim < D)
      o[dim] = f32_to_bf16((acc[i] + quarter[0][dim] + quarter[1][dim] + quarter[2][dim]) * inv);
  }
}

static int check_common(const char* who, int nq, int nkv, int d, int P, int max_pages, int num_pages, int q_stride) {
  PICO_REQUIRE(d == D, "%s: this library is built for head size %d, got %d", who, D, d);
  PICO_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "%s: %d query heads are not a multiple of %d kv heads", who, nq, nkv);
  PICO_REQUIRE(P >= 8 && (P & (P - 1)) == 0, "%s: page size %d is not a power of two of at least 8", who, P);
  PICO_REQUIRE(max_pages > 0 && num_pages > 0, "%s: empty block table or cache", who);
  PICO_REQUIRE(q_stride >= nq * D && q_stride % 8 == 0, "%s: query row stride %d must be a multiple of 8 and hold all heads", who, q_stride);
  return 0;
}

extern "C" int pico_attn_head_dim() { return D; }

extern "C" int pico_attn_prefill(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                 const int* block_table, int max_pages, const int* cu_seqlens,
                                 const int* context_lens, int num_seqs, int num_tokens, void* out, int nq, int nkv,
                                 int d, int P, int num_pages, float scale, hipStream_t stream) {
  if (check_common("pico_attn_prefill", nq, nkv, d, P, max_pages, num_pages, q_stride)) return -1;
  PICO_REQUIRE(num_seqs > 0 && num_tokens >= num_seqs, "pico_attn_prefill: bad batch (%d sequences, %d tokens)", num_seqs, num_tokens);
  PICO_REQUIRE(nq <= 65535, "pico_attn_prefill: too many heads");
  PICO_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "pico_attn_prefill: misaligned tensors");
  const int max_tiles = num_tokens / BM + num_seqs;       // >= sum over sequences of ceil(len / BM)
  dim3 grid(max_tiles, nq);
  prefill_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                          block_table, max_pages, cu_seqlens, context_lens, num_seqs, (bf16_t*)out,
                                          nq, nkv, P, num_pages, scale);
  PICO_LAUNCH_CHECK();
  return 0;
}

// part: float32 workspace of num_seqs * nq * nsplit * (D + 2) entries
extern "C" int pico_attn_decode(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                const int* block_table, int max_pages, const int* context_lens, int num_seqs,
                                void* out, float* part, int nsplit, int nq, int nkv, int d, int P, int num_pages,
                                float scale, hipStream_t stream) {
  if (check_common("pico_attn_decode", nq, nkv, d, P, max_pages, num_pages, q_stride)) return -1;
  PICO_REQUIRE(nq / nkv <= 32, "pico_attn_decode: %d query heads per kv head are more than 32", nq / nkv);
  PICO_REQUIRE(num_seqs > 0 && nsplit >= 1 && nsplit <= 64 && nkv <= 65535, "pico_attn_decode: bad sizes (1 to 64 splits)");
  PICO_REQUIRE(((uintptr_t)q % 16 == 0), "pico_attn_decode: misaligned queries");
  dim3 grid(num_seqs, nkv, nsplit);
  bool direct = false;
#if PICO_HEAD_DIM % 32 == 0 && PICO_HEAD_DIM <= 128
  direct = nq / nkv <= 16;
  if (direct)
    decode16_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
                                             (const bf16_t*)v_cache, block_table, max_pages, context_lens, part,
                                             nsplit, nq, nkv, P, num_pages, scale);
#endif
  if (!direct)
    decode_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                           block_table, max_pages, context_lens, part, nsplit, nq, nkv, P, num_pages,
                                           scale);
  PICO_LAUNCH_CHECK();
  dim3 mgrid(num_seqs, nq);
  decode_merge_kernel<<<mgrid, 256, 0, stream>>>(part, nsplit, (bf16_t*)out, nq);
  PICO_LAUNCH_CHECK();
  return 0;
}
