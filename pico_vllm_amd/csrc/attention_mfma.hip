// Paged attention on the matrix cores for bfloat16, specialised at compile time for one head
// size D = PICO_HEAD_DIM (a multiple of 16 up to 256).
//
//   prefill / mixed  a workgroup owns a tile of query tokens of one sequence and one query head; keys
//                    and values of the sequence stream through LDS in tiles, from position 0 to the
//                    causal frontier.  A decode token is a sequence that brings one query.
//                    D % 32 == 0: prefill16_kernel, 64 (or 128) queries per workgroup, 16 (or 2 x 16) per wave
//                    (v_mfma_f32_16x16x32_bf16), one to three teams of four waves that share the key loop;
//                    other D: prefill_kernel, 128 queries per workgroup, 32 per wave (32x32x16).
//   decode           one workgroup per (sequence, kv head, split of the context); the
//                    "queries" are the G query heads that share the kv head, so keys and values
//                    are read once for the whole group (the reference's kernel re-reads them per
//                    query head, pico_vllm/kernels/attention.py:96-105).  decode16_kernel (G <= 16,
//                    D % 32 == 0, D <= 128) loads its operands straight from the pages, decode_kernel
//                    stages tiles in LDS; partial (max, sum, output) per split are merged by a second kernel.
//
// Formulas as in pico_vllm/kernels/attention.py:136-213: scores (q.k) * scale, key visible iff its
// position <= the query's, online softmax in float32, probabilities rounded to bfloat16 for the
// P.V product, float32 accumulators.
// A window (not in the reference: its model has none) hides keys at positions <= the query's minus the window; every
// kernel takes it as `reach` = the window, or NO_WINDOW where there is none, so that one comparison serves both,
// starts its key loop at the first tile that a query of the workgroup still sees and masks the lower edge in the
// tiles that hold one.
//
// Matrix-core layout of the 32-query kernels (v_mfma_f32_32x32x16_bf16, D = A B, A 32x16, B 16x32): lane l supplies
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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int NO_WINDOW = 1 << 30;       // a reach no position gets to
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
  u32x4 k[NK];                              // plain vectors: a struct copy would go through memory
  uint4 v[NV];

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
      k[i] = *reinterpret_cast<const u32x4*>(k_cache + ((((size_t)page * nkv + g) << pshift) + (pos & (P - 1))) * D +
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
  // kv_lo: keys before it are seen by no query of the workgroup (a window has passed them; their pages may
  // belong to someone else by now): their values become zero like those beyond kv_end
  __device__ __forceinline__ void commit(Tiles& t, int tile_start, int kv_end, int kv_lo = 0) const {
#pragma unroll
    for (int i = 0; i < NK; i++) {
      const int c = threadIdx.x + i * NT;
      if (c < BN * KCH) *reinterpret_cast<u32x4*>(&t.k[(c / KCH) * KROW + (c % KCH) * 8]) = k[i];
    }
    const bool tail = tile_start + BN > kv_end || tile_start < kv_lo;      // the same for the whole workgroup
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
          if (pos + e >= kv_end || pos + e < kv_lo) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
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
// key; q_pos the absolute position of this lane's query column (keys beyond it are masked, and keys before `lo`).
__device__ __forceinline__ void attend_subtile(const Tiles& t, int sub, const bf16x8* q, WaveState& st, float scale,
                                               int key_pos0, int q_pos, bool need_mask, int lo = 0) {
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
      if (kpos > q_pos || kpos < lo) v = -INFINITY;
    }
    s[r] = v;
    mx = fmaxf(mx, v);
  }
  mx = max_across_32(mx);
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
  sum = sum_across_32(sum);
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
                                            int key_pos0, int q_pos, bool need_mask, int reach = NO_WINDOW) {
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
        if (need_mask) {
          const int kpos = key_pos0 + 32 * sub + 8 * (r >> 2) + 4 * h + (r & 3);
          if (kpos > q_pos || kpos <= q_pos - reach) s[sub][r] = -INFINITY;
        }
        mx = fmaxf(mx, s[sub][r]);
      }
    }
  }
  mx = max_across_32(mx);
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
  sum = sum_across_32(sum);
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
                                                      int num_pages, float scale, int reach) {
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
  // the first key tile that the workgroup's first query still sees (a multiple of 8, as the fetch wants)
  const int kv_lo = max(0, prefix + tile * BM - reach + 1), kv_begin = kv_lo / BN * BN;
  regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, kv_begin, kv_end);
  for (int tile_start = kv_begin; tile_start < kv_end; tile_start += BN) {
    __syncthreads();                                          // everyone is done with the previous tile
    regs.commit(tiles, tile_start, kv_end, kv_lo);
    __syncthreads();
    if (tile_start + BN < kv_end) regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, tile_start + BN, kv_end);
    if (!wave_active || tile_start > wave_last_pos) continue;
    if (tile_start + BN - 1 <= wave_first_pos - reach) continue;         // every key lies before every query's window
    // sub-tiles wholly beyond the causal frontier of this wave are left out
    const int nsub = min(BN / 32, (wave_last_pos - tile_start) / 32 + 1);
    attend_tile<BN / 32>(tiles, nsub, qf, st, c, tile_start, q_pos,
                         tile_start + 32 * nsub - 1 > wave_first_pos || tile_start <= wave_last_pos - reach, reach);
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
// prefill / mixed batches for head sizes that are multiples of 32: 16 queries per wave
// ---------------------------------------------------------------------------
// v_mfma_f32_16x16x32_bf16 (A 16x32, B 32x16): lane l = (c, kq) = (l % 16, l / 16) supplies
// A[c][8 kq + 0..7] and B[8 kq + 0..7][c] and receives D[4 kq + r][c] in register r.
// A workgroup owns 64 queries of one sequence and one head.  Its waves form KT (1 to 3) teams of four;
// the four waves of a team own 16 queries each, and team t works on keys 64 t .. 64 t + 63 of every
// LDS tile of 64 KT keys, so the long key loop of a late query tile is shared by KT waves per
// SIMD whose softmax and matrix products overlap; the teams' results are merged through LDS at the
// end.  A wave's accumulators (O^T: D x 16) take D / 4 registers.  Per 64 keys the scores are four
// 16 x 16 blocks of S^T = K Q^T.  Which key is row a of block j is free; it is key
// 32 (j / 2) + 8 (a / 4) + 4 (j % 2) + a % 4, so that the registers of lane quarter kq in the pair
// of blocks (2 m, 2 m + 1) hold the eight consecutive keys 32 m + 8 kq + 0..7.  Rounded to bfloat16
// they are the B operand of O^T += V^T P^T with contraction slot 8 kq + i = key 32 m + 8 kq + i,
// and the A operand is 16 contiguous bytes of V^T as the pages hold it.
// Offsets into the cache are 32-bit byte offsets: the host checks that K and V are below 4 GiB.
#if PICO_HEAD_DIM % 32 == 0
typedef float f32x4p __attribute__((ext_vector_type(4)));
constexpr int PF_BM = 64;                         // queries per workgroup
constexpr int PF_KT_MAX = D <= 128 ? 2 : 1;       // 2: one, two or three teams of four waves; 1: one team
constexpr int PF_KS = D / 32;                     // contraction steps of a 16-key block
constexpr int PF_DT = D / 16;                     // 16-wide tiles of the output's head dimension
constexpr int PF_PART_ROW = D + 4;                // floats of a chunk's partial result: D sums, the maximum, the sum of p, padding

template <int KT>
struct alignas(16) PfTiles {
  static constexpr int TK = 64 * KT;        // keys per LDS tile
  static constexpr int VROW = TK + 8;
  alignas(16) bf16_t k[TK * KROW];          // [key][dim]
  alignas(16) bf16_t vt[D * VROW];          // [dim][key]
};

// mask of a 32-bit word that holds two bfloat16 of which the first `left` exist
__device__ __forceinline__ uint32_t pair_mask(int left) { return left >= 2 ? 0xffffffffu : (left == 1 ? 0x0000ffffu : 0u); }

// Global -> registers -> LDS, as TileRegs, with the page numbers of a tile read one tile before
// its keys and values so that no load waits for another.  D % 32 == 0 makes the chunk counts whole.
template <int KT>
struct PfFetch {
  static constexpr int PF_NT = 256 * KT, PF_TK = 64 * KT, PF_VROW = PF_TK + 8;
  static constexpr int KCH = D / 8;         // 16-byte chunks per key
  static constexpr int VCH = PF_TK / 8;     // 16-byte chunks (8 keys) per head dimension
  static constexpr int N = D / 32;          // chunks of K and of V^T per thread
  u32x4 k[N], v[N];                         // plain vectors: a struct copy would go through memory
  int page_k[N], page_v;
  // What does not change from tile to tile, for whole tiles (every key exists) of pages of 8 or 16 keys:
  // the thread's chunks of K are 16 KT keys apart, whole pages, so they sit at the same place k_in
  // (in bytes) inside their pages and their page numbers stand 16 KT / P entries apart in the block table,
  // the first at byte k_bt of the tile's entries; v_in and v_bt likewise for its chunks of V^T.
  uint32_t k_in, v_in, k_bt, v_bt;

  __device__ __forceinline__ void init(int g, int nkv, int pshift) {
    const int P = 1 << pshift;
    const int key = (int)threadIdx.x / KCH;
    k_in = (((uint32_t)g << pshift) + (key & (P - 1))) * (2 * D) + ((int)threadIdx.x % KCH) * 16;
    k_bt = (uint32_t)(key >> pshift) * 4;
    const int vkey = 8 * ((int)threadIdx.x % VCH);
    v_in = ((((uint32_t)g * D + threadIdx.x / VCH) << pshift) + (vkey & (P - 1))) * 2;
    v_bt = (uint32_t)(vkey >> pshift) * 4;
  }
  // bt_tile: the block table at the tile's first page
  __device__ __forceinline__ void load_pages_full(const int* __restrict__ bt_tile, int pshift, int num_pages) {
    const char* b = reinterpret_cast<const char*>(bt_tile);
#pragma unroll
    for (int i = 0; i < N; i++)
      page_k[i] = min(max(*reinterpret_cast<const int*>(b + (size_t)((((PF_NT / KCH) * i) >> pshift) * 4) + k_bt), 0), num_pages - 1);
    page_v = min(max(*reinterpret_cast<const int*>(b + v_bt), 0), num_pages - 1);
  }
  // page_bytes: bytes of one page of K (and of V): nkv * P * D * 2, below 2^24 (the caller has checked)
  __device__ __forceinline__ void fetch_full(const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                             uint32_t page_bytes, int pshift) {
    const char* kb = reinterpret_cast<const char*>(k_cache);
    const char* vb = reinterpret_cast<const char*>(v_cache);
#pragma unroll
    for (int i = 0; i < N; i++) k[i] = *reinterpret_cast<const u32x4*>(kb + (__umul24(page_k[i], page_bytes) + k_in));
    const uint32_t off0 = __umul24(page_v, page_bytes) + v_in;
#pragma unroll
    for (int i = 0; i < N; i++)
      v[i] = *reinterpret_cast<const u32x4*>(vb + (size_t)((uint32_t)((PF_NT / VCH) * i) << (pshift + 1)) + off0);
  }
  __device__ __forceinline__ void commit_full(PfTiles<KT>& t) const {
#pragma unroll
    for (int i = 0; i < N; i++) {
      const int c = threadIdx.x + PF_NT * i;
      *reinterpret_cast<u32x4*>(&t.k[(c / KCH) * KROW + (c % KCH) * 8]) = k[i];
    }
    const int kc = threadIdx.x % VCH;
#pragma unroll
    for (int i = 0; i < N; i++)
      *reinterpret_cast<u32x4*>(&t.vt[(threadIdx.x / VCH + (PF_NT / VCH) * i) * PF_VROW + kc * 8]) = v[i];
  }

  // chunk i of this thread: K chunk c = tid + PF_NT i is key c / KCH, part c % KCH; V^T chunk c is
  // head dimension c / VCH, keys 8 (c % VCH) .. + 7, and c % VCH = tid % VCH for every i.
  __device__ __forceinline__ void load_pages(const int* __restrict__ bt, int pshift, int num_pages, int tile_start,
                                             int kv_end) {
    const int last_key = kv_end - 1;
#pragma unroll
    for (int i = 0; i < N; i++) {
      const int pos = min(tile_start + ((int)threadIdx.x + PF_NT * i) / KCH, last_key);
      page_k[i] = min(max(bt[pos >> pshift], 0), num_pages - 1);
    }
    const int pos = min(tile_start + 8 * ((int)threadIdx.x % VCH), last_key & ~7);
    page_v = min(max(bt[pos >> pshift], 0), num_pages - 1);
  }

  // positions at or beyond kv_end read a clamped, valid address: their scores are masked and
  // commit() makes their values zero
  __device__ __forceinline__ void fetch(const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, int g,
                                        int nkv, int pshift, int tile_start, int kv_end) {
    const int P = 1 << pshift, last_key = kv_end - 1;
    const char* kb = reinterpret_cast<const char*>(k_cache);
    const char* vb = reinterpret_cast<const char*>(v_cache);
#pragma unroll
    for (int i = 0; i < N; i++) {
      const int c = (int)threadIdx.x + PF_NT * i;
      const int pos = min(tile_start + c / KCH, last_key);
      const uint32_t off = ((((uint32_t)page_k[i] * nkv + g) << pshift) + (pos & (P - 1))) * (2 * D) + (c % KCH) * 16;
      k[i] = *reinterpret_cast<const u32x4*>(kb + off);
    }
    const int pos = min(tile_start + 8 * ((int)threadIdx.x % VCH), last_key & ~7);
    const uint32_t off0 = (((((uint32_t)page_v * nkv + g) * D + threadIdx.x / VCH) << pshift) + (pos & (P - 1))) * 2;
#pragma unroll
    for (int i = 0; i < N; i++)
      v[i] = *reinterpret_cast<const u32x4*>(vb + (off0 + ((uint32_t)((PF_NT / VCH) * i) << (pshift + 1))));
  }

  // kv_lo: keys before it are seen by no query of the workgroup (a window has passed them)
  __device__ __forceinline__ void commit(PfTiles<KT>& t, int tile_start, int kv_end, int kv_lo = 0) const {
#pragma unroll
    for (int i = 0; i < N; i++) {
      const int c = threadIdx.x + PF_NT * i;
      *reinterpret_cast<u32x4*>(&t.k[(c / KCH) * KROW + (c % KCH) * 8]) = k[i];
    }
    const bool tail = tile_start + PF_TK > kv_end || tile_start < kv_lo;    // the same for the whole workgroup
    const int kc = threadIdx.x % VCH;
#pragma unroll
    for (int i = 0; i < N; i++) {
      u32x4 x = v[i];
      if (tail) {   // values of keys at or beyond kv_end, or before kv_lo, hold whatever the page held before
        const int left = kv_end - (tile_start + kc * 8);       // keys of this chunk that exist
        const int skip = kv_lo - (tile_start + kc * 8);        // keys of this chunk before the first that is seen
        x[0] &= pair_mask(left) & ~pair_mask(skip);
        x[1] &= pair_mask(left - 2) & ~pair_mask(skip - 2);
        x[2] &= pair_mask(left - 4) & ~pair_mask(skip - 4);
        x[3] &= pair_mask(left - 6) & ~pair_mask(skip - 6);
      }
      *reinterpret_cast<u32x4*>(&t.vt[(threadIdx.x / VCH + (PF_NT / VCH) * i) * PF_VROW + kc * 8]) = x;
    }
  }
};

struct PfState {
  float m, l;          // reference maximum of the column; this lane's part of the column's sum
  f32x4p o[PF_DT];     // O^T tiles: rows = head dimension, column = query
};

// The 64 keys of one team (its first NPAIR pairs of 16-key blocks) against the wave's NQB blocks of 16 query
// columns (every operand read from LDS serves the NQB blocks), one softmax update per block: raw scores,
// p = 2^(s c - m c) with c = scale * log2(e); the reference
// maximum may lag behind the running maximum by up to 8 in the exponent and the accumulators are
// rescaled only when a column of the wave outgrows that (see attend_tile).
// krow: row 8 (col / 4) + col % 4 of the team's keys in LDS, vrow: row col of V^T at the team's keys,
// both at this lane quarter's 16 bytes; key_pos0: position of the team's first key.
template <int NPAIR, bool MASK, int PF_VROW, int NQB>
__device__ __forceinline__ void pf_attend(const bf16_t* krow, const bf16_t* vrow, const bf16x8 (&q)[NQB][PF_KS],
                                          PfState (&st)[NQB], float c, int key_pos0, const int (&q_pos)[NQB],
                                          int reach = NO_WINDOW) {
  const int kq = (threadIdx.x & 63) >> 4;
  f32x4p s[NQB][2 * NPAIR];
  // Two query blocks a wave: the operands of a 16-key block (PF_KS reads from LDS) are requested one block ahead of
  // their products, so that a read's latency passes under the products of the block before; left to itself the
  // compiler, short of registers, requests each operand just in front of its use (one query block a wave: it has
  // the registers, and three waves a SIMD to hide the latency with).
  constexpr bool AHEAD = NQB == 2;
  if constexpr (AHEAD) {
    u32x4 ka[2][PF_KS];
#pragma unroll
    for (int step = 0; step < PF_KS; step++) ka[0][step] = *reinterpret_cast<const u32x4*>(krow + 32 * step);
#pragma unroll
    for (int j = 0; j < 2 * NPAIR; j++) {
      if (j + 1 < 2 * NPAIR) {
#pragma unroll
        for (int step = 0; step < PF_KS; step++)
          ka[(j + 1) & 1][step] =
              *reinterpret_cast<const u32x4*>(krow + (32 * ((j + 1) / 2) + 4 * ((j + 1) % 2)) * KROW + 32 * step);
      }
      __builtin_amdgcn_sched_barrier(0);            // the next block's reads stay in front of this block's products
#pragma unroll
      for (int b = 0; b < NQB; b++) s[b][j] = f32x4p{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int step = 0; step < PF_KS; step++) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, ka[j & 1][step]);
#pragma unroll
        for (int b = 0; b < NQB; b++) s[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q[b][step], s[b][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 2 * NPAIR; j++) {
#pragma unroll
      for (int b = 0; b < NQB; b++) s[b][j] = f32x4p{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int step = 0; step < PF_KS; step++) {
        const bf16x8 a = __builtin_bit_cast(
            bf16x8, *reinterpret_cast<const u32x4*>(krow + (32 * (j / 2) + 4 * (j % 2)) * KROW + 32 * step));
#pragma unroll
        for (int b = 0; b < NQB; b++) s[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q[b][step], s[b][j], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int b = 0; b < NQB; b++) {
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 2 * NPAIR; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        if (MASK) {
          const int kpos = key_pos0 + 32 * (j / 2) + 8 * kq + 4 * (j % 2) + r;
          if (kpos > q_pos[b] || kpos <= q_pos[b] - reach) s[b][j][r] = -INFINITY;
        }
        mx = fmaxf(mx, s[b][j][r]);
      }
    mx = max_across_16(mx);
    mx = max_across_32(mx);
    const float m_new = fmaxf(st[b].m, mx);
    const bool outgrown = (m_new - st[b].m) * c > 8.0f;        // also true while the reference is -inf
    if (__builtin_amdgcn_ballot_w64(outgrown) != 0) {          // the same decision for the whole wave
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((st[b].m - m_use) * c);
      st[b].l *= alpha;
      st[b].m = m_new;
#pragma unroll
      for (int tt = 0; tt < PF_DT; tt++) st[b].o[tt] *= alpha;
    }
    const float mc = ((st[b].m == -INFINITY) ? 0.f : st[b].m) * c;
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 2 * NPAIR; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[b][j][r], c, -mc));
        s[b][j][r] = p;
        sum += p;
      }
    st[b].l += sum;
  }
  bf16x8 pb[NPAIR][NQB];
#pragma unroll
  for (int m = 0; m < NPAIR; m++)
#pragma unroll
    for (int b = 0; b < NQB; b++)
      pb[m][b] = __builtin_bit_cast(
          bf16x8, u32x4{pack2_bf16(s[b][2 * m][0], s[b][2 * m][1]), pack2_bf16(s[b][2 * m][2], s[b][2 * m][3]),
                        pack2_bf16(s[b][2 * m + 1][0], s[b][2 * m + 1][1]), pack2_bf16(s[b][2 * m + 1][2], s[b][2 * m + 1][3])});
  if constexpr (AHEAD) {
    // likewise the operands of V^T, in groups of four head-dimension tiles (of two where four do not divide them)
    constexpr int GR = PF_DT % 4 == 0 ? 4 : 2, NG = NPAIR * PF_DT / GR;
    static_assert(PF_DT % GR == 0, "whole groups of tiles");
    u32x4 va[2][GR];
    auto vsrc = [&](int g, int i) { return vrow + 16 * ((g * GR + i) % PF_DT) * PF_VROW + 32 * ((g * GR + i) / PF_DT); };
#pragma unroll
    for (int i = 0; i < GR; i++) va[0][i] = *reinterpret_cast<const u32x4*>(vsrc(0, i));
#pragma unroll
    for (int g = 0; g < NG; g++) {
      if (g + 1 < NG) {
#pragma unroll
        for (int i = 0; i < GR; i++) va[(g + 1) & 1][i] = *reinterpret_cast<const u32x4*>(vsrc(g + 1, i));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < GR; i++) {
        const int tt = (g * GR + i) % PF_DT, m = (g * GR + i) / PF_DT;
        const bf16x8 a = __builtin_bit_cast(bf16x8, va[g & 1][i]);
#pragma unroll
        for (int b = 0; b < NQB; b++) st[b].o[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[m][b], st[b].o[tt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
#pragma unroll
    for (int m = 0; m < NPAIR; m++)
#pragma unroll
      for (int tt = 0; tt < PF_DT; tt++) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(vrow + 16 * tt * PF_VROW + 32 * m));
#pragma unroll
        for (int b = 0; b < NQB; b++) st[b].o[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[m][b], st[b].o[tt], 0, 0, 0);
      }
  }
}

// grid: x = query head, y = (sequence, 64-query tile), late (long) tiles first.  One team keeps three
// workgroups on a compute unit, which serves many long, equal tiles best; two or three teams cut the key
// loop of the longest tile, which decides when the tiles are few or unequal (a causal triangle).
// NQB = 2 (one or two teams): a wave owns two blocks of 16 queries and a workgroup 128, so every K and V^T
// operand read from LDS feeds two products; LDS traffic, which bounds the kernel when there is work for
// every compute unit, halves per product, at the price of registers for two waves per SIMD.
template <int KT, int NQB = 1>
__global__ __launch_bounds__(256 * KT, (KT == 2 || NQB == 2) ? 2 : 3) void prefill16_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, int num_seqs, bf16_t* __restrict__ out, int nq, int nkv, int P, int num_pages,
    float scale, int reach, int chunk_len, int max_chunks, float* __restrict__ part, const int* __restrict__ order) {
  static_assert(NQB == 1 || KT <= 2, "two query blocks a wave: one or two teams (three would leave a wave 170 registers)");
  constexpr int PF_TK = 64 * KT, PF_VROW = PF_TK + 8;
  constexpr int BMQ = PF_BM * NQB;            // queries per workgroup
  // the tiles of keys and values, and after the key loop the sums that the teams beyond the first hand to it
  constexpr size_t MERGE_BYTES = (size_t)(KT - 1) * 4 * NQB * (PF_DT * 4 + 2) * 64 * sizeof(float);
  constexpr size_t LDS_BYTES = sizeof(PfTiles<KT>) > MERGE_BYTES ? sizeof(PfTiles<KT>) : MERGE_BYTES;
  __shared__ alignas(16) char lds[LDS_BYTES];
  PfTiles<KT>& tiles = *reinterpret_cast<PfTiles<KT>*>(lds);
  int b = 0, tile = (int)blockIdx.y, ntiles = 0;
  if (order != nullptr) {       // the tiles of all sequences, longest first (pf_order_kernel): (sequence << 16) | tile, -1 behind the last
    const int e = order[blockIdx.y];
    if (e < 0) return;
    b = e >> 16;
    tile = e & 0xffff;
    // not a tile of a sequence of this step (a list that was never written): nothing is read through it
    if (b >= num_seqs || tile * BMQ >= cu_seqlens[b + 1] - cu_seqlens[b]) return;
  } else {                      // sequence by sequence, each from its last (longest) tile down
    for (; b < num_seqs; b++) {
      ntiles = (cu_seqlens[b + 1] - cu_seqlens[b] + BMQ - 1) / BMQ;
      if (tile < ntiles) break;
      tile -= ntiles;
    }
    if (b >= num_seqs) return;
    tile = ntiles - 1 - tile;
  }
  const int head = blockIdx.x, g = head / (nq / nkv);
  const int tok0 = cu_seqlens[b], new_len = cu_seqlens[b + 1] - tok0;
  const int ctx = context_lens[b], prefix = ctx - new_len;
  const int tile_kv_end = min(ctx, prefix + min(new_len, (tile + 1) * BMQ));   // keys beyond the tile's last query are never needed
  // chunk_len > 0: the keys of a tile are cut into chunks of that many (a multiple of the LDS tile; no window then),
  // each a workgroup of its own (grid z); a tile of several chunks leaves partial results that pf_merge_kernel joins
  const int n_chunks = chunk_len > 0 ? (tile_kv_end + chunk_len - 1) / chunk_len : 1;
  const int chunk = chunk_len > 0 ? (int)blockIdx.z : 0;
  if (chunk >= n_chunks) return;
  const int wave = (threadIdx.x >> 6) & 3, team = threadIdx.x >> 8;
  const int lane = threadIdx.x & 63, col = lane & 15, kq = lane >> 4;
  const int* bt = block_table + (size_t)b * max_pages;

  const int wave_q0 = tile * BMQ + wave * 16 * NQB;            // the wave's first query among the sequence's new tokens
  int q_idx[NQB], q_pos[NQB];
  bool q_ok[NQB];
  bf16x8 qf[NQB][PF_KS];
#pragma unroll
  for (int qb = 0; qb < NQB; qb++) {
    q_idx[qb] = wave_q0 + 16 * qb + col;
    q_ok[qb] = q_idx[qb] < new_len;
    q_pos[qb] = prefix + q_idx[qb];
    const bf16_t* qrow = q + (size_t)(tok0 + (q_ok[qb] ? q_idx[qb] : 0)) * q_stride + (size_t)head * D + 8 * kq;
#pragma unroll
    for (int step = 0; step < PF_KS; step++) {
      u32x4 v = u32x4{0, 0, 0, 0};
      if (q_ok[qb]) v = *reinterpret_cast<const u32x4*>(qrow + 32 * step);
      qf[qb][step] = __builtin_bit_cast(bf16x8, v);
    }
  }
  const int wave_first_pos = prefix + wave_q0;                              // lowest query position of the wave
  const int wave_last_pos = min(wave_first_pos + 16 * NQB - 1, ctx - 1);    // highest real one
  const bool wave_active = wave_q0 < new_len;
  const int kv_end = chunk_len > 0 ? min(tile_kv_end, (chunk + 1) * chunk_len) : tile_kv_end;

  const float c = scale * 1.4426950408889634f;                 // scores go through 2^x
  const int pshift = 31 - __clz(P);                            // page sizes are powers of two
  PfState st[NQB];
#pragma unroll
  for (int qb = 0; qb < NQB; qb++) {
    st[qb].m = -INFINITY;
    st[qb].l = 0.f;
#pragma unroll
    for (int tt = 0; tt < PF_DT; tt++) st[qb].o[tt] = f32x4p{0.f, 0.f, 0.f, 0.f};
  }
  const bf16_t* krow = &tiles.k[(64 * team + 8 * (col >> 2) + (col & 3)) * KROW + 8 * kq];
  const bf16_t* vrow = &tiles.vt[col * PF_VROW + 64 * team + 8 * kq];
  PfFetch<KT> regs;
  // Whole tiles of pages of 8 or 16 keys take the short way: no clamping of positions, nothing to mask,
  // addresses from what init() has prepared.  The last tiles and other pages go the long way.  Two loops
  // and no branch inside them: a branch between the loads would force a wait for the ones before it.
  const uint32_t page_bytes = ((uint32_t)nkv << pshift) * (2 * D);
  // ... and only where a thread's chunks of K are a whole number of pages apart (PfFetch::init): head sizes
  // whose chunks per key do not divide the workgroup's threads, or pages larger than that distance, go the long way
  constexpr int K_APART = PfFetch<KT>::PF_NT / PfFetch<KT>::KCH;            // keys between a thread's chunks
  const bool apart_ok = PfFetch<KT>::PF_NT % PfFetch<KT>::KCH == 0 && ((K_APART >> pshift) << pshift) == K_APART;
  // (and no window: the first tile of a window holds keys whose values must read as zero)
  const int n_full = (apart_ok && reach == NO_WINDOW && pshift <= 4 && page_bytes < (1u << 24) && num_pages < (1 << 24)) ? kv_end / PF_TK : 0;
  // the first key that the workgroup's first query still sees, and its tile
  const int kv_lo = max(0, prefix + tile * BMQ - reach + 1);
  const int first_tile = chunk_len > 0 ? chunk * (chunk_len / PF_TK) : kv_lo / PF_TK;
  const int kv_begin = first_tile * PF_TK;
  regs.init(g, nkv, pshift);
  regs.load_pages(bt, pshift, num_pages, kv_begin, kv_end);
  regs.fetch(k_cache, v_cache, g, nkv, pshift, kv_begin, kv_end);
  regs.load_pages(bt, pshift, num_pages, kv_begin + PF_TK, kv_end);
  auto attend = [&](int tile_start) {
    const int key0 = tile_start + 64 * team;                    // this team's keys
    if (!wave_active || key0 > wave_last_pos) return;
    if (key0 + 63 <= wave_first_pos - reach) return;            // every key lies before every query's window
    if (key0 <= wave_last_pos - reach) {                        // a window's lower edge runs through these keys
      pf_attend<2, true, PF_VROW, NQB>(krow, vrow, qf, st, c, key0, q_pos, reach);
    } else if (key0 + 63 <= wave_first_pos) {
      pf_attend<2, false, PF_VROW, NQB>(krow, vrow, qf, st, c, key0, q_pos);
    } else if (key0 + 32 <= wave_last_pos) {
      pf_attend<2, true, PF_VROW, NQB>(krow, vrow, qf, st, c, key0, q_pos);
    } else {   // the second pair of 16-key blocks lies wholly beyond the causal frontier of this wave
      pf_attend<1, true, PF_VROW, NQB>(krow, vrow, qf, st, c, key0, q_pos);
    }
  };
  int ti = first_tile;
  for (; ti + 2 < n_full; ti++) {            // this tile, the next and the one after it are whole
    __syncthreads();                                            // everyone is done with the previous tile
    regs.commit_full(tiles);
    __syncthreads();
    regs.fetch_full(k_cache, v_cache, page_bytes, pshift);
    regs.load_pages_full(bt + (((ti + 2) * PF_TK) >> pshift), pshift, num_pages);
    attend(ti * PF_TK);
  }
  for (int tile_start = ti * PF_TK; tile_start < kv_end; tile_start += PF_TK) {
    __syncthreads();
    regs.commit(tiles, tile_start, kv_end, kv_lo);
    __syncthreads();
    // the next tile's keys and values (clamped to the last key if there is no next tile) and the
    // page numbers of the tile after it
    regs.fetch(k_cache, v_cache, g, nkv, pshift, tile_start + PF_TK, kv_end);
    regs.load_pages(bt, pshift, num_pages, tile_start + 2 * PF_TK, kv_end);
    attend(tile_start);
  }
  if constexpr (KT > 1) {
    // merge the teams through LDS (reusing the tile memory): lane-wise, the layouts agree
    __syncthreads();
    float* xo = reinterpret_cast<float*>(lds);                 // [team - 1][wave][query block][PF_DT * 4 + 2][64 lanes]
    constexpr int PER_BLOCK = (PF_DT * 4 + 2) * 64, PER_WAVE = NQB * PER_BLOCK;
    static_assert(LDS_BYTES >= (size_t)(KT - 1) * 4 * PER_WAVE * sizeof(float), "LDS too small for the merge");
    if (team > 0) {
#pragma unroll
      for (int qb = 0; qb < NQB; qb++) {
        float* mine = xo + ((team - 1) * 4 + wave) * PER_WAVE + qb * PER_BLOCK + lane;
#pragma unroll
        for (int tt = 0; tt < PF_DT; tt++)
#pragma unroll
          for (int r = 0; r < 4; r++) mine[(4 * tt + r) * 64] = st[qb].o[tt][r];
        mine[(PF_DT * 4) * 64] = st[qb].m;
        mine[(PF_DT * 4 + 1) * 64] = st[qb].l;
      }
    }
    __syncthreads();
    if (team > 0) return;
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
      PfState& s0 = st[qb];
      const float* base = xo + wave * PER_WAVE + qb * PER_BLOCK + lane;       // team t: base + (t - 1) * 4 * PER_WAVE
      float M = s0.m;
#pragma unroll
      for (int t = 1; t < KT; t++) M = fmaxf(M, base[(t - 1) * 4 * PER_WAVE + (PF_DT * 4) * 64]);
      const float m_use = (M == -INFINITY) ? 0.f : M;
      const float a0 = __builtin_amdgcn_exp2f((s0.m - m_use) * c);
      s0.l *= a0;
      s0.m = M;                                                // what the merged sums are relative to (a chunk's part says so)
#pragma unroll
      for (int tt = 0; tt < PF_DT; tt++) s0.o[tt] *= a0;
#pragma unroll
      for (int t = 1; t < KT; t++) {
        const float* theirs = base + (t - 1) * 4 * PER_WAVE;
        const float at = __builtin_amdgcn_exp2f((theirs[(PF_DT * 4) * 64] - m_use) * c);
        s0.l += at * theirs[(PF_DT * 4 + 1) * 64];
#pragma unroll
        for (int tt = 0; tt < PF_DT; tt++)
#pragma unroll
          for (int r = 0; r < 4; r++) s0.o[tt][r] += at * theirs[(4 * tt + r) * 64];
      }
    }
  }
  if (n_chunks > 1) {
    // this chunk's part of the tile: unnormalised sums, the reference maximum they are relative to, and the sum of
    // the probabilities, per (token, head, chunk)
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
      if (!q_ok[qb]) continue;
      float l = st[qb].l;
      l = sum_across_16(l);
      l = sum_across_32(l);
      float* prow = part + (((size_t)(tok0 + q_idx[qb]) * nq + head) * max_chunks + chunk) * PF_PART_ROW + 4 * kq;
#pragma unroll
      for (int tt = 0; tt < PF_DT; tt++) *reinterpret_cast<f32x4p*>(prow + 16 * tt) = st[qb].o[tt];
      if (kq == 0) {
        prow[D] = st[qb].m;
        prow[D + 1] = l;
      }
    }
    return;
  }
#pragma unroll
  for (int qb = 0; qb < NQB; qb++) {
    if (!q_ok[qb]) continue;
    float l = st[qb].l;
    l = sum_across_16(l);
    l = sum_across_32(l);
    const float inv_l = 1.0f / l;
    bf16_t* orow = out + ((size_t)(tok0 + q_idx[qb]) * nq + head) * D + 4 * kq;
#pragma unroll
    for (int tt = 0; tt < PF_DT; tt++) {
      uint2 v;
      v.x = pack2_bf16(st[qb].o[tt][0] * inv_l, st[qb].o[tt][1] * inv_l);
      v.y = pack2_bf16(st[qb].o[tt][2] * inv_l, st[qb].o[tt][3] * inv_l);
      *reinterpret_cast<uint2*>(orow + 16 * tt) = v;
    }
  }
}

// The order in which the workgroups of prefill16_kernel take the query tiles of a step with several sequences: all
// tiles of all sequences by the number of keys they read, most first.  Workgroups start in the order of the grid, and a
// compute unit takes the next one when it has finished one; sequence by sequence, the long tiles of the last sequence
// would start when the others are nearly through and the launch would end on them (eight prompts of 2,048 tokens: the
// compute units finished between 117 and 176 us).  One workgroup; every thread ranks its entries against all others in
// LDS, which is quadratic and therefore offered only up to PF_ORDER_MAX entries.
// order[r] = (sequence << 16) | tile for rank r, -1 from the number of tiles on (capacity entries in all).
constexpr int PF_ORDER_MAX = 512;
__global__ __launch_bounds__(256) void pf_order_kernel(const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
                                                       int num_seqs, int bmq, int* __restrict__ order, int capacity) {
  __shared__ int keys[PF_ORDER_MAX], ids[PF_ORDER_MAX], first[PF_ORDER_MAX + 1];
  if (threadIdx.x == 0) {
    int n = 0;
    for (int b = 0; b < num_seqs; b++) {
      first[b] = n;
      n += (cu_seqlens[b + 1] - cu_seqlens[b] + bmq - 1) / bmq;
    }
    first[num_seqs] = n;
  }
  __syncthreads();
  const int n = min(first[num_seqs], PF_ORDER_MAX);          // the host has checked that it holds all of them
  for (int b = threadIdx.x; b < num_seqs; b += blockDim.x) {
    const int new_len = cu_seqlens[b + 1] - cu_seqlens[b], ctx = context_lens[b], prefix = ctx - new_len;
    for (int e = first[b]; e < min(first[b + 1], PF_ORDER_MAX); e++) {
      const int tile = e - first[b];
      keys[e] = min(ctx, prefix + min(new_len, (tile + 1) * bmq));
      ids[e] = (b << 16) | tile;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    const int key = keys[e];
    int rank = 0;
    for (int o = 0; o < n; o++) rank += (keys[o] > key || (keys[o] == key && o < e)) ? 1 : 0;
    order[rank] = ids[e];
  }
  for (int e = n + threadIdx.x; e < capacity; e += blockDim.x) order[e] = -1;
}

// Joins the chunks of the tiles that prefill16_kernel cut (chunk_len > 0): out[token, head, :] =
// sum_i 2^((m_i - M) c) o_i / sum_i 2^((m_i - M) c) l_i over the tile's chunks; tokens of a tile with one chunk have
// their result already.  One wave per (token, head), four head dimensions a lane, four waves a workgroup (a workgroup
// per row with one dimension a thread took 15.8 us where this takes 11.6 for 2,048 tokens of 12 heads in 2 chunks: too
// many tiny workgroups).  bmq: queries per tile.
__global__ __launch_bounds__(256) void pf_merge_kernel(const float* __restrict__ part, int max_chunks, int chunk_len,
                                                       const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
                                                       int num_seqs, int num_tokens, bf16_t* __restrict__ out, int nq, float scale,
                                                       int bmq) {
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);         // (token, head)
  if (row >= (long long)num_tokens * nq) return;
  const int t = (int)(row / nq), lane = threadIdx.x & 63;
  int b = 0;
  while (b + 1 < num_seqs && cu_seqlens[b + 1] <= t) b++;
  const int tok0 = cu_seqlens[b], new_len = cu_seqlens[b + 1] - tok0;
  if (t < tok0 || t - tok0 >= new_len) return;      // a token in front of the portions (a decode row of a mixed step), or none
  const int ctx = context_lens[b], prefix = ctx - new_len, tile = (t - tok0) / bmq;
  const int tile_kv_end = min(ctx, prefix + min(new_len, (tile + 1) * bmq));
  const int n_chunks = (tile_kv_end + chunk_len - 1) / chunk_len;
  if (n_chunks <= 1 || 4 * lane >= D) return;
  const float c = scale * 1.4426950408889634f;
  const float* rows = part + (size_t)row * max_chunks * PF_PART_ROW;
  float M = -INFINITY;
  for (int i = 0; i < n_chunks; i++) M = fmaxf(M, rows[i * PF_PART_ROW + D]);
  f32x4p o = f32x4p{0.f, 0.f, 0.f, 0.f};
  float l = 0.f;
  for (int i = 0; i < n_chunks; i++) {
    const float m = rows[i * PF_PART_ROW + D];
    const float a = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m - M) * c);     // a chunk that this query sees no key of
    o += a * *reinterpret_cast<const f32x4p*>(rows + i * PF_PART_ROW + 4 * lane);
    l += a * rows[i * PF_PART_ROW + D + 1];
  }
  const float inv = 1.0f / l;
  uint2 v;
  v.x = pack2_bf16(o[0] * inv, o[1] * inv);
  v.y = pack2_bf16(o[2] * inv, o[3] * inv);
  *reinterpret_cast<uint2*>(out + (size_t)row * D + 4 * lane) = v;
}
#endif


// ---------------------------------------------------------------------------
// decode: one query token per sequence, the G heads of a kv group as the 32 columns
// ---------------------------------------------------------------------------
// partial results per (sequence, query head, split): o [D] unnormalised, then m and l
// CUT: the workgroup's keys come from the step's cut into pieces of one length (plan), not from a split of its own sequence
template <bool CUT>
__global__ __launch_bounds__(256, PICO_ATTN_WAVES_PER_SIMD) void decode_kernel(const bf16_t* __restrict__ q, int q_stride,
                                                     const bf16_t* __restrict__ k_cache,
                                                     const bf16_t* __restrict__ v_cache,
                                                     const int* __restrict__ block_table, int max_pages,
                                                     const int* __restrict__ context_lens,
                                                     float* __restrict__ part, int nsplit, int nq, int nkv, int P,
                                                     int num_pages, float scale, int reach, const int4* __restrict__ plan,
                                                     int num_seqs) {
  __shared__ Tiles tiles;
  const int g = blockIdx.y;
  const int G = nq / nkv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  int b, ctx, k_begin, k_end;
  size_t part_slot;                 // this workgroup's place among the partial results, counted in (query heads) rows
  if (CUT) {                        // pieces of one length over all sequences (decode_plan_kernel): grid x is the piece
    const int4 mine = plan[blockIdx.x];
    // an empty slot; or not a piece of a sequence of this step (a cut that was never written): nothing is read through it
    if (mine.x < 0 || mine.x >= num_seqs || mine.y < 0 || mine.y >= mine.z || mine.z > mine.w ||
        mine.w > (long long)max_pages * P) return;
    b = mine.x, k_begin = mine.y, k_end = mine.z, ctx = mine.w;
    part_slot = (size_t)blockIdx.x * nq;
  } else {                          // every sequence in nsplit splits of its own
    b = blockIdx.x;
    ctx = context_lens[b];
    const int lo_tile = max(0, ctx - reach) / BN * BN;
    // this split's keys: a whole number of LDS tiles
    const int per = ((ctx - lo_tile + nsplit - 1) / nsplit + BN - 1) / BN * BN;
    k_begin = lo_tile + (int)blockIdx.z * per, k_end = min(ctx, k_begin + per);
    part_slot = (size_t)b * nq * nsplit + blockIdx.z;
  }
  const size_t part_stride = CUT ? 1 : nsplit;                  // rows of the partial results between two heads
  // the query sits at position ctx - 1 and sees keys lo .. ctx - 1; the splits share them from the tile that holds lo on
  const int lo = max(0, ctx - reach);
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
    regs.commit(tiles, tile_start, k_end, lo);
    __syncthreads();
    if (tile_start + BN < k_end) regs.fetch(k_cache, v_cache, bt, g, nkv, pshift, num_pages, tile_start + BN, k_end);
    for (int sub = wave; sub < BN / 32 && wave < 2; sub += 2) {   // waves 2 and 3 only help to move the tiles
      const int key0 = tile_start + sub * 32;
      if (key0 >= k_end) break;
      if (key0 + 32 <= lo) continue;                 // wholly before the window
      // every query sits at position ctx - 1: only keys at or beyond k_end, or before lo, need the mask
      attend_subtile(tiles, sub, qf, st, scale, key0, k_end - 1, key0 + 32 > k_end || key0 < lo, lo);
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
  float* po = part + (part_slot + (size_t)head * part_stride) * (D + 2);
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
// Operands come straight from the pages, in the order of memory: in step st the four lanes (a, 0..3) of
// row a read the 64 contiguous bytes K[key of row a][32 st ..] (a load instruction touches 16 cache
// lines; with a lane reading its own 64 bytes it touched 32), and lane (dim, kq) reads the 16 bytes
// V^T[dim][8 kq .. 8 kq + 7] of the block.  Which key is row a of tile t is free; it is key
// 8 (a / 4) + 4 t + a % 4 of the block, so that the registers of lane quarter kq hold the scores of the
// eight consecutive keys 8 kq + 0..7, which is the contraction order of the V^T operand.
// The loads of a wave's next block are issued while the current block is computed.
#if PICO_HEAD_DIM % 32 == 0 && PICO_HEAD_DIM <= 128
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int KS16 = D / 32;   // contraction steps of a 16-key tile
constexpr int DT16 = D / 16;   // 16-wide tiles of the output's head dimension

template <bool CUT>
__global__ __launch_bounds__(256, 2) void decode16_kernel(const bf16_t* __restrict__ q, int q_stride,
                                                          const bf16_t* __restrict__ k_cache,
                                                          const bf16_t* __restrict__ v_cache,
                                                          const int* __restrict__ block_table, int max_pages,
                                                          const int* __restrict__ context_lens,
                                                          float* __restrict__ part, int nsplit, int nq, int nkv, int P,
                                                          int num_pages, float scale, int reach, const int4* __restrict__ plan,
                                                          int num_seqs) {
  __shared__ float xo[3][D][16];     // outputs of waves 1..3 for the final merge
  __shared__ float xml[3][2][16];
  const int g = blockIdx.y;
  const int G = nq / nkv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 15, kq = lane >> 4;
  int b, ctx, k_begin, k_end;
  size_t part_slot;                 // this workgroup's place among the partial results, counted in (query heads) rows
  if (CUT) {                        // pieces of one length over all sequences (decode_plan_kernel): grid x is the piece
    const int4 mine = plan[blockIdx.x];
    // an empty slot; or not a piece of a sequence of this step (a cut that was never written): nothing is read through it
    if (mine.x < 0 || mine.x >= num_seqs || mine.y < 0 || mine.y >= mine.z || mine.z > mine.w ||
        mine.w > (long long)max_pages * P) return;
    b = mine.x, k_begin = mine.y, k_end = mine.z, ctx = mine.w;
    part_slot = (size_t)blockIdx.x * nq;
  } else {                          // every sequence in nsplit splits of its own
    b = blockIdx.x;
    ctx = context_lens[b];
    const int lo_block = max(0, ctx - reach) & ~31;
    const int per = ((ctx - lo_block + nsplit - 1) / nsplit + 31) / 32 * 32;
    k_begin = lo_block + (int)blockIdx.z * per, k_end = min(ctx, k_begin + per);
    part_slot = (size_t)b * nq * nsplit + blockIdx.z;
  }
  const size_t part_stride = CUT ? 1 : nsplit;                  // rows of the partial results between two heads
  // the query sits at position ctx - 1 and sees keys lo .. ctx - 1; the splits share them from the block that holds lo on
  const int lo = max(0, ctx - reach);
  const int* bt = block_table + (size_t)b * max_pages;
  const bool col_ok = col < G;
  const int head = g * G + (col_ok ? col : 0);

  bf16x8 qf[KS16];
  {
    const bf16_t* qrow = q + (size_t)b * q_stride + (size_t)head * D + 8 * kq;
#pragma unroll
    for (int st = 0; st < KS16; st++) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col_ok) v = *reinterpret_cast<const uint4*>(qrow + 32 * st);
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
    const int last_key = k_end - 1, last_group = last_key / 8 * 8;
    const int row_key = 8 * (col >> 2) + (col & 3);             // key of this lane's row in tile 0; tile 1: 4 more
    uint4 kr[2][KS16];
    uint4 vr[DT16];
    // positions beyond the split are clamped to its last key (group of 8, which lies in one page as pages hold
    // at least 8 keys): the pages exist, the scores are masked
    auto load_k = [&](int key0) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int pos = min(key0 + row_key + 4 * t, last_key);
        const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
        const bf16_t* kp = k_cache + ((((size_t)page * nkv + g) << pshift) + (pos & (P - 1))) * D + 8 * kq;
#pragma unroll
        for (int st = 0; st < KS16; st++) kr[t][st] = *reinterpret_cast<const uint4*>(kp + 32 * st);
      }
    };
    auto load_v = [&](int key0) {
      const int pos = min(key0 + 8 * kq, last_group);
      const int page = min(max(bt[pos >> pshift], 0), num_pages - 1);
      const bf16_t* vp = v_cache + ((((size_t)page * nkv + g) * D + col) << pshift) + (pos & (P - 1));
#pragma unroll
      for (int tt = 0; tt < DT16; tt++) vr[tt] = *reinterpret_cast<const uint4*>(vp + ((size_t)tt * 16 << pshift));
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
      const bool tail = key0 + 32 > k_end || key0 < lo;        // the same for the whole wave
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        float v = (r < 4 ? s0[r & 3] : s1[r & 3]) * scale;
        if (tail && (key0 + 8 * kq + r >= k_end || key0 + 8 * kq + r < lo)) v = -INFINITY;
        sv[r] = v;
        mx = fmaxf(mx, v);
      }
      mx = max_across_16(mx);
      mx = max_across_32(mx);
      const float m_new = fmaxf(m, mx);                        // finite: the block holds at least one key in lo .. k_end - 1
      const float alpha = __expf(m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        sv[r] = __expf(sv[r] - m_new);
        sum += sv[r];
      }
      sum = sum_across_16(sum);
      sum = sum_across_32(sum);
      l = l * alpha + sum;
      m = m_new;
      const bf16x8 pb = __builtin_bit_cast(bf16x8, make_uint4(pack2_bf16(sv[0], sv[1]), pack2_bf16(sv[2], sv[3]),
                                                               pack2_bf16(sv[4], sv[5]), pack2_bf16(sv[6], sv[7])));
      if (tail) {   // values of keys beyond the split or before the window hold whatever the page held before: make them zero
        const int left = k_end - (key0 + 8 * kq);               // this lane's eight keys exist below `left` ...
        const int skip = lo - (key0 + 8 * kq);                  // ... and from `skip` on
        uint32_t keep[4];
#pragma unroll
        for (int w = 0; w < 4; w++)
          keep[w] = ((left >= 2 * w + 2 ? 0xffffffffu : left == 2 * w + 1 ? 0x0000ffffu : 0u) &
                     (skip <= 2 * w ? 0xffffffffu : skip == 2 * w + 1 ? 0xffff0000u : 0u));
#pragma unroll
        for (int tt = 0; tt < DT16; tt++) {
          vr[tt].x &= keep[0];
          vr[tt].y &= keep[1];
          vr[tt].z &= keep[2];
          vr[tt].w &= keep[3];
        }
      }
#pragma unroll
      for (int tt = 0; tt < DT16; tt++) {
        o[tt] *= alpha;
        o[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vr[tt]), pb, o[tt], 0, 0, 0);
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
  float* po = part + (part_slot + (size_t)head * part_stride) * (D + 2);
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
// head).  Every wave weighs all splits (lane s % 64 holds split s, up to four of them) and sums a
// quarter of each 64 splits for all head dimensions, the loads of a quarter issued together; wave 0
// adds the four quarters.
constexpr int MERGE_MAX_SPLITS = 256;
// rows (with splits of equal length over all sequences): (first split, number of splits) of every sequence; the partial
// results of a split's heads then lie together, nq rows apart from split to split.
template <bool CUT>
__global__ __launch_bounds__(256) void decode_merge_kernel(const float* __restrict__ part, int nsplit,
                                                           bf16_t* __restrict__ out, int nq, const int2* __restrict__ rows,
                                                           int slots) {
  constexpr int DPL = (D + 63) / 64;                        // head dimensions per lane
  constexpr int CH = MERGE_MAX_SPLITS / 64;
  __shared__ float quarter[3][DPL * 64];
  const int b = blockIdx.x, head = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* p = part + ((size_t)b * nq + head) * nsplit * (D + 2);
  const size_t step = CUT ? (size_t)nq * (D + 2) : D + 2;   // floats from one split of this head to the next
  if (CUT) {
    int2 mine = rows[b];
    if (mine.x < 0 || mine.y < 0 || mine.y > MERGE_MAX_SPLITS || mine.x + mine.y > slots) mine = make_int2(0, 0);   // never written
    nsplit = mine.y;
    p = part + ((size_t)mine.x * nq + head) * (D + 2);
  }
  float m[CH], l[CH], wt[CH];
  float mx = -INFINITY;
#pragma unroll
  for (int c = 0; c < CH; c++) {
    const bool mine = 64 * c + lane < nsplit;
    m[c] = mine ? p[(64 * c + lane) * step + D] : -INFINITY;
    l[c] = mine ? p[(64 * c + lane) * step + D + 1] : 0.f;
    mx = fmaxf(mx, m[c]);
  }
  const float M = wave_max(mx);
  bf16_t* o = out + ((size_t)b * nq + head) * D;
  if (M == -INFINITY) {   // an empty row (padding of a captured batch)
    if (wave == 0)
      for (int dim = lane; dim < D; dim += 64) o[dim] = 0;
    return;
  }
  float lsum = 0.f;
#pragma unroll
  for (int c = 0; c < CH; c++) {
    wt[c] = 64 * c + lane < nsplit ? __expf(m[c] - M) : 0.f;
    lsum += wt[c] * l[c];
  }
  const float L = wave_sum(lsum);
  float acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; i++) acc[i] = 0.f;
#pragma unroll
  for (int c = 0; c < CH; c++) {
    if (64 * c >= nsplit) break;
    const int s0 = 64 * c + wave * 16;
    float v[16][DPL];
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const int s = min(s0 + j, nsplit - 1);
#pragma unroll
      for (int i = 0; i < DPL; i++) {
        const int dim = lane + 64 * i;
        v[j][i] = dim < D ? p[s * step + dim] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const float ws = (s0 + j < nsplit) ? __shfl(wt[c], wave * 16 + j, 64) : 0.f;
#pragma unroll
      for (int i = 0; i < DPL; i++) acc[i] += ws * v[j][i];
    }
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

// Splits of equal length over all sequences of a decode step.  With the same number of splits for every sequence a
// step of unequal contexts ends on the workgroups of its longest sequences (64 sequences of 128 to 4,224 tokens: 35 us a
// layer where equal contexts of the same total take 27).  Here all sequences are cut into pieces of one length T, the
// smallest whole number of `unit` keys for which the pieces of all sequences fit the `slots` workgroups of the launch
// (and no sequence has more than the merging kernel takes); with equal contexts that is the cut they had before.  T
// depends on the contexts of the step alone (rows without a context, the padding of a recorded step, count for
// nothing), so a sequence is cut alike whether the step is recorded and padded or not.
// plan[slot] = (sequence, first key, end, context) or (-1, ..) for a slot that stays empty; rows[b] = (first slot, slots).
// At most PLAN_MAX_ROWS sequences.
constexpr int PLAN_MAX_ROWS = 1024;
__device__ __forceinline__ int plan_wave_sum(int v) {
#pragma unroll
  for (int w = 32; w >= 1; w >>= 1) v += __shfl_xor(v, w, 64);
  return v;
}
__device__ __forceinline__ int plan_wave_max(int v) {
#pragma unroll
  for (int w = 32; w >= 1; w >>= 1) v = max(v, __shfl_xor(v, w, 64));
  return v;
}
// One wave: its sums and maxima need no barrier, and the search below is a dozen of them.
__global__ __launch_bounds__(64) void decode_plan_kernel(const int* __restrict__ context_lens, int num_seqs, int slots,
                                                         int reach, int unit, int4* __restrict__ plan, int2* __restrict__ rows) {
  __shared__ int len[PLAN_MAX_ROWS], low[PLAN_MAX_ROWS], first[PLAN_MAX_ROWS + 1];
  const int lane = threadIdx.x;
  int my_sum = 0, my_max = 0;
  for (int b = lane; b < num_seqs; b += 64) {
    const int ctx = context_lens[b];
    const int lo = max(0, ctx - reach) / unit * unit;        // the splits share the keys from the unit that holds the first visible one on
    low[b] = lo;
    len[b] = ctx > 0 ? ctx - lo : 0;
    my_sum += (len[b] + unit - 1) / unit;                    // counted in units, so the sums stay small
    my_max = max(my_max, len[b]);
  }
  const int total_units = plan_wave_sum(my_sum), longest = plan_wave_max(my_max);
  // the smallest T = t units with sum over b of ceil(len_b / T) <= slots: t lies between what fills every slot exactly and
  // one piece a sequence (which fits: the launch has a slot for every sequence)
  int t_lo = max(1, max((total_units + slots - 1) / slots, ((longest + MERGE_MAX_SPLITS - 1) / MERGE_MAX_SPLITS + unit - 1) / unit));
  int t_hi = max(t_lo, (longest + unit - 1) / unit);
  while (t_lo < t_hi) {                                       // the same for all lanes
    const int mid = (t_lo + t_hi) / 2, T = mid * unit;
    int mine = 0;
    for (int b = lane; b < num_seqs; b += 64) mine += (len[b] + T - 1) / T;
    if (plan_wave_sum(mine) <= slots) t_hi = mid;
    else t_lo = mid + 1;
  }
  const int T = t_lo * unit;
  // first[b]: the pieces of the sequences before b; 64 sequences a turn, a prefix sum over the lanes
  int base = 0;
  for (int b0 = 0; b0 < num_seqs; b0 += 64) {
    const int b = b0 + lane;
    const int count = b < num_seqs ? (len[b] + T - 1) / T : 0;
    int incl = count;
#pragma unroll
    for (int w = 1; w < 64; w <<= 1) {
      const int up = __shfl_up(incl, w, 64);
      if (lane >= w) incl += up;
    }
    if (b < num_seqs) first[b] = base + incl - count;
    base += __shfl(incl, 63, 64);
  }
  if (lane == 0) first[num_seqs] = base;
  __syncthreads();
  for (int b = lane; b < num_seqs; b += 64) {
    const int count = first[b + 1] - first[b], ctx = low[b] + len[b];
    rows[b] = make_int2(first[b], count);
    for (int i = 0; i < count; i++) plan[first[b] + i] = make_int4(b, low[b] + i * T, min(ctx, low[b] + (i + 1) * T), ctx);
  }
  for (int e = first[num_seqs] + lane; e < slots; e += 64) plan[e] = make_int4(-1, 0, 0, 0);
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

// teams: the shape of the workgroups (1 to 3 teams of four waves that share the key loop of a 64-query tile; 4: one
// team of 128 queries; 6: two teams of 128 queries; 0: two teams of 64 where the head size allows it); a hint, any
// value gives the same result up to rounding.  chunk_len > 0 (a multiple of 128, no window, not three teams, head sizes in steps of 32): the keys of every tile are cut
// into chunks of that many, each a workgroup of its own, and a second launch joins the chunks of a tile; part is
// their workspace, float32 [num_tokens, nq, max_chunks, D + 4], and max_chunks at least ceil(longest context / chunk_len).
// order (may be null): room for order_capacity >= num_tokens / 64 + num_seqs integers; with several sequences their query
// tiles are taken longest first from the list that pf_order_kernel writes there, when order_build is set (the first
// layer of a step) or has written there (the others: same sequences, same `teams`).
extern "C" int pico_attn_prefill(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                 const int* block_table, int max_pages, const int* cu_seqlens,
                                 const int* context_lens, int num_seqs, int num_tokens, void* out, int nq, int nkv,
                                 int d, int P, int num_pages, float scale, int teams, int window, int chunk_len,
                                 int max_chunks, float* part, int* order, int order_capacity, int order_build, hipStream_t stream) {
  if (check_common("pico_attn_prefill", nq, nkv, d, P, max_pages, num_pages, q_stride)) return -1;
  PICO_REQUIRE(window >= 0 && window < NO_WINDOW, "pico_attn_prefill: bad window %d", window);
  const int reach = window > 0 ? window : NO_WINDOW;
  PICO_REQUIRE(num_seqs > 0 && num_tokens >= num_seqs, "pico_attn_prefill: bad batch (%d sequences, %d tokens)", num_seqs, num_tokens);
  PICO_REQUIRE(nq <= 65535, "pico_attn_prefill: too many heads");
  PICO_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "pico_attn_prefill: misaligned tensors");
  PICO_REQUIRE(chunk_len >= 0, "pico_attn_prefill: bad chunk length %d", chunk_len);
#if PICO_HEAD_DIM % 32 == 0
  // the 16-query kernel addresses the cache with 32-bit byte offsets
  if ((uint64_t)num_pages * nkv * P * D * sizeof(bf16_t) < (1ull << 32)) {
    const int max_tiles = num_tokens / PF_BM + num_seqs;  // >= sum over sequences of ceil(len / PF_BM)
    PICO_REQUIRE(max_tiles <= 65535, "pico_attn_prefill: %d tokens are too many for one launch", num_tokens);
    dim3 grid(nq, max_tiles);
    if (chunk_len > 0) {
      // (a chunk holds whole LDS tiles of every team shape but the one with three teams, whose tiles are 192 keys)
      PICO_REQUIRE(window == 0 && teams != 3 && chunk_len % 128 == 0 && max_chunks >= 1 && max_chunks <= 64 &&
                       part != nullptr && (uintptr_t)part % 16 == 0,
                   "pico_attn_prefill: chunks of keys need no window, one or two teams, a length that is a multiple of 128 "
                   "(got %d), 1 to 64 chunks (got %d) and an aligned workspace", chunk_len, max_chunks);
      grid.z = max_chunks;
    }
    // 4 and 6: 128 queries a workgroup (two blocks of 16 a wave), in one team or two
    const bool wide = (teams == 4 || teams == 6) && PF_KT_MAX == 2;
    const int bmq = wide ? 2 * PF_BM : PF_BM;
    if (wide) grid.y = num_tokens / (2 * PF_BM) + num_seqs;
    // several sequences: their tiles longest first, from the caller's list (built here when the caller says so: once a
    // step, the layers of a step share it); a step of more tiles than the ordering kernel takes goes sequence by sequence
    const int* ord = nullptr;
    if (order != nullptr && num_seqs >= 2 && num_seqs <= PF_ORDER_MAX && (int)grid.y <= PF_ORDER_MAX) {
      PICO_REQUIRE(order_capacity >= (int)grid.y, "pico_attn_prefill: the list of tiles holds %d entries, the step may have %d",
                   order_capacity, (int)grid.y);
      if (order_build) {
        pf_order_kernel<<<1, 256, 0, stream>>>(cu_seqlens, context_lens, num_seqs, bmq, order, (int)grid.y);
        PICO_LAUNCH_CHECK();
      }
      ord = order;
    }
#define PF_ARGS (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, \
                cu_seqlens, context_lens, num_seqs, (bf16_t*)out, nq, nkv, P, num_pages, scale, reach, chunk_len, max_chunks, part, ord
    if (teams == 6 && PF_KT_MAX == 2)             // 128 queries a workgroup and two key teams
      prefill16_kernel<PF_KT_MAX == 2 ? 2 : 1, PF_KT_MAX == 2 ? 2 : 1><<<grid, 512, 0, stream>>>(PF_ARGS);
    else if (teams == 4 && PF_KT_MAX == 2)        // 128 queries a workgroup, two blocks of 16 a wave
      prefill16_kernel<1, PF_KT_MAX == 2 ? 2 : 1><<<grid, 256, 0, stream>>>(PF_ARGS);
    else if (teams == 1 || PF_KT_MAX == 1)
      prefill16_kernel<1><<<grid, 256, 0, stream>>>(PF_ARGS);
    else if (teams == 3 && PF_KT_MAX == 2)
      prefill16_kernel<PF_KT_MAX == 2 ? 3 : 1><<<grid, 768, 0, stream>>>(PF_ARGS);
    else
      prefill16_kernel<PF_KT_MAX><<<grid, 256 * PF_KT_MAX, 0, stream>>>(PF_ARGS);
#undef PF_ARGS
    PICO_LAUNCH_CHECK();
    if (chunk_len > 0 && max_chunks > 1) {
      const long long rows = (long long)num_tokens * nq;
      PICO_REQUIRE((rows + 3) / 4 <= 0x7fffffffLL, "pico_attn_prefill: too many rows to join");
      pf_merge_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, stream>>>(part, max_chunks, chunk_len, cu_seqlens, context_lens,
                                                                      num_seqs, num_tokens, (bf16_t*)out, nq, scale, bmq);
      PICO_LAUNCH_CHECK();
    }
    return 0;
  }
#endif
  PICO_REQUIRE(chunk_len == 0, "pico_attn_prefill: chunks of keys are for head sizes in steps of 32 and caches below 4 GiB");
  const int max_tiles = num_tokens / BM + num_seqs;       // >= sum over sequences of ceil(len / BM)
  dim3 grid(max_tiles, nq);
  prefill_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                          block_table, max_pages, cu_seqlens, context_lens, num_seqs, (bf16_t*)out,
                                          nq, nkv, P, num_pages, scale, reach);
  PICO_LAUNCH_CHECK();
  return 0;
}

// part: float32 workspace of num_seqs * nq * nsplit * (D + 2) entries
// plan (may be null): 4 * plan_slots + 2 * num_seqs integers; the contexts of all sequences are then cut into pieces of
// one length, at most plan_slots >= num_seqs of them in all (pico_attn_decode_plan writes the cut when plan_build is
// set, the first layer of a step; the other layers find it there), and part holds plan_slots * nq * (D + 2) floats.
extern "C" int pico_attn_decode(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                const int* block_table, int max_pages, const int* context_lens, int num_seqs,
                                void* out, float* part, int nsplit, int nq, int nkv, int d, int P, int num_pages,
                                float scale, int window, int* plan, int plan_slots, int plan_build, hipStream_t stream) {
  if (check_common("pico_attn_decode", nq, nkv, d, P, max_pages, num_pages, q_stride)) return -1;
  PICO_REQUIRE(window >= 0 && window < NO_WINDOW, "pico_attn_decode: bad window %d", window);
  const int reach = window > 0 ? window : NO_WINDOW;
  PICO_REQUIRE(nq / nkv <= 32, "pico_attn_decode: %d query heads per kv head are more than 32", nq / nkv);
  PICO_REQUIRE(num_seqs > 0 && nsplit >= 1 && nsplit <= MERGE_MAX_SPLITS && nkv <= 65535, "pico_attn_decode: bad sizes (1 to %d splits)", MERGE_MAX_SPLITS);
  PICO_REQUIRE(((uintptr_t)q % 16 == 0), "pico_attn_decode: misaligned queries");
  dim3 grid(num_seqs, nkv, nsplit);
  bool direct = false;
#if PICO_HEAD_DIM % 32 == 0 && PICO_HEAD_DIM <= 128
  direct = nq / nkv <= 16;
#endif
  const int4* cut = nullptr;
  const int2* rows = nullptr;
  if (plan != nullptr) {
    PICO_REQUIRE(plan_slots >= num_seqs && num_seqs <= PLAN_MAX_ROWS && (uintptr_t)plan % 16 == 0,
                 "pico_attn_decode: a cut of %d sequences into %d pieces (at most %d sequences, a piece each at least, 16-byte aligned)",
                 num_seqs, plan_slots, PLAN_MAX_ROWS);
    cut = reinterpret_cast<const int4*>(plan);
    rows = reinterpret_cast<const int2*>(plan + 4 * (size_t)plan_slots);
    if (plan_build) {
      decode_plan_kernel<<<1, 64, 0, stream>>>(context_lens, num_seqs, plan_slots, reach, direct ? 32 : BN,
                                                reinterpret_cast<int4*>(plan), reinterpret_cast<int2*>(plan + 4 * (size_t)plan_slots));
      PICO_LAUNCH_CHECK();
    }
    grid = dim3(plan_slots, nkv, 1);
  }
#define DECODE_ARGS (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, context_lens, \
                    part, nsplit, nq, nkv, P, num_pages, scale, reach, cut, num_seqs
#if PICO_HEAD_DIM % 32 == 0 && PICO_HEAD_DIM <= 128
  if (direct) {
    if (cut != nullptr) decode16_kernel<true><<<grid, 256, 0, stream>>>(DECODE_ARGS);
    else decode16_kernel<false><<<grid, 256, 0, stream>>>(DECODE_ARGS);
  }
#endif
  if (!direct) {
    if (cut != nullptr) decode_kernel<true><<<grid, 256, 0, stream>>>(DECODE_ARGS);
    else decode_kernel<false><<<grid, 256, 0, stream>>>(DECODE_ARGS);
  }
#undef DECODE_ARGS
  PICO_LAUNCH_CHECK();
  dim3 mgrid(num_seqs, nq);
  if (rows != nullptr) decode_merge_kernel<true><<<mgrid, 256, 0, stream>>>(part, nsplit, (bf16_t*)out, nq, rows, plan_slots);
  else decode_merge_kernel<false><<<mgrid, 256, 0, stream>>>(part, nsplit, (bf16_t*)out, nq, rows, plan_slots);
  PICO_LAUNCH_CHECK();
  return 0;
}
