// Weight-streaming matrix product for few rows of activations (decode, small mixed steps):
// out = X W^T with X [M <= 64 per launch block, K] and W [N, K] bfloat16, K contiguous in both.
// The cost is reading W once from HBM, so the kernel is built around that stream:
//
//   * a workgroup owns up to 32 rows of W (one output tile; how many of the 32 the host decides, see
//     TileRows) and one range of k; its waves take interleaved 64-wide k slices of that range and are
//     summed through LDS in a fixed order, so the split over k needs no atomics and results are reproducible;
//   * a slice of a wave (32 rows x 128 bytes of W, and of the activations as many 8-token groups
//     as hold tokens) does not go through registers.  A lane that reads its own row of W makes
//     every load instruction touch 32 cache lines, and the address unit of the compute unit, not
//     HBM, then bounds the stream (measured: 16 us against 13 us for the 55 MB gate/up matrix with
//     8 tokens, 34 us against 22 us with 64).  Instead `global_load_lds_dwordx4` copies the slice
//     global -> LDS in the order of memory (8 lanes share one 128-byte line, 8 lines per
//     instruction) and the v_mfma_f32_32x32x16_bf16 operands are read back from LDS (lane (i, h)
//     takes chunks 4 h + 0..3 of row i, W and activations alike: the contraction does not care
//     about the order of k).  The copy is asynchronous: DEPTH slices per wave are in flight
//     without holding registers;
//   * up to 32 tokens: 4 waves per workgroup; 33 to 64 tokens: 2 waves, each with both blocks of
//     32 tokens, so that three workgroups still share the LDS of a compute unit, or on large grids
//     4 waves with two tiles of W that share the activations (gemm_skinny_pair_kernel);
//   * when the matrix is too small to fill the chip (N small), the k range is also split over
//     workgroups (grid y); each writes a float32 partial slab that the consumer sums;
//   * K % 64 != 0 (any multiple of 8): a plain loop with operands in registers.
//
// Epilogues on the float32 sums: bias; SwiGLU (the tile holds 16 gate rows and the 16 matching up
// rows, so silu(gate) * up is local to a lane; pico_vllm/kernels/swiglu.py:36-41); float32 or
// bfloat16 store.  Layout of the 32x32 result tile: lane l holds output column (token) l % 32 and
// tile rows 8 (r / 4) + 4 (l / 32) + r % 4 in register r.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The rows of W behind a 32-row tile: tile rows 0..15 are rows row_a .. row_a + va - 1 of W, tile rows
// 16..31 rows row_b .. row_b + vb - 1 (va >= 1, vb >= 0, at most 16 each).  Tile rows without a row of
// their own read the last row of their half again (the same cache lines: no traffic); what they sum
// is never stored.  A tile with fewer rows is how the host makes the number of workgroups fit the
// chip: a compute unit takes in about 25 GB/s whatever runs on it, so the time of a launch is what
// the fullest compute unit has to read, and 560 tiles on 256 compute units cost as much as 768.
struct TileRows {
  int row_a, row_b, va, vb;
  __device__ __forceinline__ int row(int tile_row) const {     // the row of W that tile row `tile_row` reads
    const bool second = tile_row >= 16 && vb > 0;
    return second ? row_b + min(tile_row - 16, vb - 1) : row_a + min(tile_row, va - 1);
  }
};

#define EPI_BF16 0     // out bf16 [M, N]
#define EPI_F32 1      // out float32 [M, N] (slab `blockIdx.y` when the k range is split over the grid)
#define EPI_SWIGLU 2   // W = [gate rows; up rows], out bf16 [M, N / 2]
#define MAX_SK_SLABS 8 // partial sums that a norm in front of a projection adds up

// The sums of one output tile when K is no multiple of 64 (any multiple of 8): operands go through
// registers, lane (i, h) reads W[row i][k0 + 32 h ..] and the activations alike; k beyond the range
// reads as zero.  Sums over k_begin .. k_end of W[wrow0][k] X[m][k] for the 32 tile rows (wrow0: this
// lane's row of W) and 32 MT tokens, each of the 4 waves over its slices, left in
// red[wave][token block][register][lane]; the caller sums the waves after the barrier at the end.
template <int MT>
__device__ __forceinline__ void skinny_stream(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ wrow0,
                                              int m0, int M, int k_begin, int k_end, float (*red)[MT][16][64]) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const bf16_t* xrow0[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) xrow0[t] = X + (size_t)min(m0 + 32 * t + col, M - 1) * ldx;
  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
  // this wave's slices start at k_begin + 64 (wave + 4 i)
  for (int k0 = k_begin + 64 * wave; k0 < k_end; k0 += 256) {
    u32x4 w[4], x[MT][4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int k = k0 + 32 * h + 8 * s;          // 8 consecutive k; K % 8 == 0, so all or nothing
      const bool ok = k < k_end;
      const u32x4 wv = *reinterpret_cast<const u32x4*>(wrow0 + (ok ? k : 0));
      w[s] = ok ? wv : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int t = 0; t < MT; t++) {
        const u32x4 xv = *reinterpret_cast<const u32x4*>(xrow0[t] + (ok ? k : 0));
        x[t][s] = ok ? xv : u32x4{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int t = 0; t < MT; t++)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[s]), __builtin_bit_cast(bf16x8, x[t][s]),
                                                         acc[t], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) red[wave][t][r][lane] = acc[t][r];
  __syncthreads();
}

// ---- the stream through LDS ----------------------------------------------------------------
// One slice of one wave in LDS: 4 groups of W (8 tile rows x 128 bytes each) and NX groups of X
// (8 tokens x 128 bytes).  A group is what one load instruction brings: lane l = (rho, pos) =
// (l / 8, l % 8) writes bytes 16 l .. 16 l + 15 of the group, and fetches chunk pos ^ rho of row
// rho of the group, so that the rows of a group lie in LDS with their 16-byte chunks xor-swizzled by
// the row and the operand reads below (32 rows, one chunk each) spread over the banks; groups are
// 16 bytes further apart than their size for the same reason.
#define GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LPTR(p) ((__attribute__((address_space(3))) void*)(p))
constexpr int SK_GROUP = 1024 + 16;
template <int NX> constexpr int sk_stage_bytes() { return (4 + NX) * SK_GROUP; }
// How full the grid makes the chip (FILL): SK_FEW, at most one workgroup per compute unit; SK_MANY, more than two
// per unit; 0 otherwise.
// Slices in flight per wave.  SK_FEW (the whole LDS is the workgroup's own): as many as fit, because such a launch
// is a chain of memory latencies, not a stream.  SK_MANY, up to 16 tokens: two, so that the stages are 42 to 50 KB
// and three workgroups share a compute unit instead of two (5,141 against 5,098 tokens a second at batch 8; with
// the normed row in LDS three workgroups gave 800 tokens a second at batch 1, two gave 747).
#define SK_FEW 1
#define SK_MANY 2
template <int NX, int FILL> constexpr int sk_depth() {
  return FILL == SK_FEW ? (NX <= 2 ? 6 : NX == 4 ? 4 : 3) : (NX >= 4 || FILL == SK_MANY) ? 2 : 3;
}
// waves per workgroup: two when a wave holds two blocks of tokens in LDS and the grid is large, so that
// three workgroups fit a compute unit, and with 17 to 32 tokens on a grid of more than two workgroups a unit, so
// that four do (33 KB each; 14,340 against 14,140 tokens a second at batch 32); four otherwise (SK_FEW: at most
// one workgroup per compute unit anyway)
template <int MT, int NX, int FILL> constexpr int sk_waves() {
  return ((MT == 2 && NX > 0 && FILL != SK_FEW) || (NX == 4 && FILL == SK_MANY)) ? 2 : 4;
}
// s_waitcnt for "at most n vector memory operations outstanding", nothing else waited for
constexpr int sk_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

template <int MT, int NX, int FILL>
constexpr int sk_smem_bytes() {
  constexpr int red = 4 * MT * 16 * 64 * 4;
  if (NX == 0) return red;
  constexpr int stages = sk_depth<NX, FILL>() * sk_waves<MT, NX, FILL>() * sk_stage_bytes<NX>();
  return stages > red ? stages : red;
}

// The sums of tile `tr`;
// tokens m0 .. m0 + 8 NX - 1 (clamped to M - 1) in MT blocks of 32.  The sums end up in
// red[v][token block][register][lane] at the start of smem, as skinny_stream leaves them: v = 0..3
// holds the slices k_begin + 64 (v + 4 i) whatever the number of waves (a wave of a two-wave
// workgroup keeps two sets of sums), so that a row's result does not depend on how many rows came
// with it.
//
// XS: the activations, one row, do not travel with the slices.  The row lies in LDS already, bfloat16 [k_end] at xs
// (the caller's `between`, which every wave runs after the first copies of W have been issued, puts it there;
// its `before` runs ahead of those copies, for loads that should not queue behind them); a stage then holds
// W only, and every column of the product is the row's.
struct SkNothing {
  __device__ __forceinline__ void operator()() const {}
};
template <int MT, int NX, int NWV, int DEPTH, bool XS = false, typename Before = SkNothing, typename Between = SkNothing>
__device__ __forceinline__ void skinny_stream_lds(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W,
                                                  int ldw, TileRows tr, int m0, int M, int k_begin,
                                                  int k_end, char* smem, const char* xs = nullptr,
                                                  Before before = Before(), Between between = Between()) {
  constexpr int STAGE = XS ? 4 * SK_GROUP : sk_stage_bytes<NX>(), LOADS = XS ? 4 : 4 + NX;
  static_assert(!XS || (MT == 1 && NX == 1), "activations that stay in LDS: one row");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int col = lane & 31, h = lane >> 5, rho = lane >> 3, pos = lane & 7;
  // sources of this lane's 16 bytes in each group, at k = 0
  const bf16_t* wsrc[4];
#pragma unroll
  for (int g = 0; g < 4; g++) wsrc[g] = W + (size_t)tr.row(8 * g + rho) * ldw + 8 * (pos ^ rho);
  const bf16_t* xsrc[NX];
#pragma unroll
  for (int g = 0; g < NX; g++) xsrc[g] = XS ? nullptr : X + (size_t)min(m0 + 8 * g + rho, M - 1) * ldx + 8 * (pos ^ rho);
  // where lane (col, h) finds chunk 4 h + s of tile row (or token) col, relative to the slice
  int rd[4];
#pragma unroll
  for (int s = 0; s < 4; s++) rd[s] = (col >> 3) * SK_GROUP + (col & 7) * 128 + (((4 * h + s) ^ (col & 7)) << 4);
  char* mine = smem + wave * STAGE;            // stage d of this wave: mine + d * NWV * STAGE
  constexpr int VW = 4 / NWV;                  // sets of sums per wave: slice i of the wave goes to set i % VW
  static_assert(DEPTH % VW == 0, "a stage must always feed the same set of sums");
  f32x16 acc[MT][VW];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int v = 0; v < VW; v++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[t][v][r] = 0.f;

  constexpr int STRIDE = 64 * NWV;             // this wave's slices start at k_begin + 64 (wave + NWV i)
  const int first = k_begin + 64 * wave;
  const bool any = first < k_end;
  const int n_slices = any ? (k_end - first + STRIDE - 1) / STRIDE : 0;
  const int rounds = (n_slices + DEPTH - 1) / DEPTH;
  const int last = first + (n_slices - 1) * STRIDE;
  auto issue = [&](int d, int slice) {         // beyond the wave's last slice the last one is copied again
    const int k0 = min(first + STRIDE * slice, last);
    char* dst = mine + d * NWV * STAGE;
#pragma unroll
    for (int g = 0; g < 4; g++) __builtin_amdgcn_global_load_lds(GPTR(wsrc[g] + k0), LPTR(dst + g * SK_GROUP), 16, 0, 0);
    if (!XS) {
#pragma unroll
      for (int g = 0; g < NX; g++)
        __builtin_amdgcn_global_load_lds(GPTR(xsrc[g] + k0), LPTR(dst + (4 + g) * SK_GROUP), 16, 0, 0);
    }
  };
  auto multiply = [&](int d, int slice) {
    const char* src = mine + d * NWV * STAGE;
    u32x4 a[4], b[MT][4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      a[s] = *reinterpret_cast<const u32x4*>(src + rd[s]);
      if (XS) {   // the one row, for every column alike (only column 0 is stored)
        b[0][s] = *reinterpret_cast<const u32x4*>(xs + 2 * (first + STRIDE * slice) + ((4 * h + s) << 4));
      } else {
#pragma unroll
        for (int t = 0; t < MT; t++) b[t][s] = *reinterpret_cast<const u32x4*>(src + (4 + 4 * t) * SK_GROUP + rd[s]);
      }
    }
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int t = 0; t < MT; t++)
        acc[t][d % VW] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[s]),
                                                                 __builtin_bit_cast(bf16x8, b[t][s]), acc[t][d % VW], 0, 0, 0);
  };
  before();
  __builtin_amdgcn_sched_barrier(0);
  if (any) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) issue(d, d);
    __builtin_amdgcn_sched_barrier(0);
  }
  between();                                   // every wave, with its first copies on their way
  if (any) {
    for (int r = 0; r + 1 < rounds; r++) {     // every slice of these rounds exists
#pragma unroll
      for (int d = 0; d < DEPTH; d++) {
        // DEPTH stages are in flight, stage d is the oldest: it has landed when at most the loads of
        // the DEPTH - 1 younger stages are outstanding.  The compiler does not order LDS reads after
        // these copies by itself.
        __builtin_amdgcn_s_waitcnt(sk_vmcnt((DEPTH - 1) * LOADS));
        __builtin_amdgcn_sched_barrier(0);
        multiply(d, r * DEPTH + d);             // its operand reads are complete when the products have issued
        __builtin_amdgcn_sched_barrier(0);
        issue(d, (r + 1) * DEPTH + d);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_waitcnt(sk_vmcnt(0));
    __builtin_amdgcn_sched_barrier(0);
    const int left = n_slices - (rounds - 1) * DEPTH;            // 1..DEPTH slices in the last round
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
      if (d < left) multiply(d, (rounds - 1) * DEPTH + d);
  }
  __syncthreads();                             // every wave is done with its stages: the sums take their place
  float(*red)[MT][16][64] = reinterpret_cast<float(*)[MT][16][64]>(smem);
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int v = 0; v < VW; v++)
#pragma unroll
      for (int r = 0; r < 16; r++) red[wave + NWV * v][t][r][lane] = acc[t][v][r];
  __syncthreads();
}

// The 32 tile rows' sums for this workgroup's tokens, through LDS (NX > 0) or registers (NX == 0).
template <int MT, bool TAIL, int NX, int FILL>
__device__ __forceinline__ float (*skinny_tile(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw,
                                               TileRows tr, int m0, int M, int k_begin, int k_end,
                                               char* smem))[MT][16][64] {
  float(*red)[MT][16][64] = reinterpret_cast<float(*)[MT][16][64]>(smem);
  if constexpr (NX > 0) {
    static_assert(!TAIL && NX <= 4 * MT, "the stream through LDS takes whole slices");
    skinny_stream_lds<MT, NX, sk_waves<MT, NX, FILL>(), sk_depth<NX, FILL>()>(X, ldx, W, ldw, tr, m0, M, k_begin, k_end, smem);
  } else {
    // Only a k tail must read as zero, because it is summed into outputs that are stored.
    skinny_stream<MT>(X, ldx, W + (size_t)tr.row(threadIdx.x & 31) * ldw, m0, M, k_begin, k_end, red);
  }
  return red;
}

// Which rows of W stand behind tile `tile` when a tile has `rows` of them (`rows` pairs for SwiGLU: gate rows
// in the first half of the tile, the matching up rows in the second).
template <int EPI>
__device__ __forceinline__ TileRows skinny_rows(int tile, int rows, int N) {
  TileRows tr;
  if (EPI == EPI_SWIGLU) {
    const int I = N / 2;
    tr.row_a = min(tile * rows, I - 1);
    tr.row_b = I + tr.row_a;
    tr.va = tr.vb = min(rows, I - tr.row_a);
  } else {
    tr.row_a = min(tile * rows, N - 1);
    tr.row_b = tr.row_a + 16;
    tr.va = min(min(rows, 16), N - tr.row_a);
    tr.vb = max(0, min(rows - 16, N - tr.row_b));
  }
  return tr;
}

// Thread (a, lane) finishes tile rows 8 a + 4 h + 0..3 of column `col` of tile `tile` of `rows` rows
// (pairs): the sum of the 4 sets of slices, then the epilogue.
template <int MT, int EPI>
__device__ __forceinline__ void skinny_finish(float (*red)[MT][16][64], int tile, int rows, int a, int m0, int M, int N,
                                              const float* __restrict__ bias, void* __restrict__ out, int ldo,
                                              long long slab_stride) {
  const int lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int t0 = 8 * a + 4 * h;                      // this thread's first tile row
  if (t0 >= rows) return;
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int m = m0 + 32 * t + col;
    if (m >= M) continue;
    if (EPI == EPI_SWIGLU) {
      if (a >= 2) continue;
      const int I = N / 2, gi = tile * rows + t0;
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
        if (t0 + b < rows && gi + b < I) store_f32(o + b, v[b]);
    } else {
      const int n = tile * rows + t0;
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
          if (t0 + b < rows && n + b < N) o[b] = v[b];
      } else {
        bf16_t* o = (bf16_t*)out + (size_t)m * ldo + n;
#pragma unroll
        for (int b = 0; b < 4; b++)
          if (t0 + b < rows && n + b < N) store_f32(o + b, v[b]);
      }
    }
  }
}

// FILL: SK_FEW, SK_MANY or 0 (see sk_depth)
template <int MT, int EPI, bool TAIL, int NX, int FILL = 0>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ X, int ldx,
                                                          const bf16_t* __restrict__ W, int ldw,
                                                          const float* __restrict__ bias, void* __restrict__ out,
                                                          int ldo, long long slab_stride, int M, int N, int K,
                                                          int k_per_wg, int rows) {
  __shared__ __attribute__((aligned(16))) char smem[sk_smem_bytes<MT, NX, FILL>()];
  const int wave = threadIdx.x >> 6;
  const int tile = blockIdx.x;
  const int m0 = blockIdx.z * 32 * MT;
  const int k_begin = blockIdx.y * k_per_wg, k_end = min(K, k_begin + k_per_wg);
  float(*red)[MT][16][64] = skinny_tile<MT, TAIL, NX, FILL>(X, ldx, W, ldw, skinny_rows<EPI>(tile, rows, N), m0, M, k_begin, k_end, smem);
  constexpr int NWV = sk_waves<MT, NX, FILL>();
  for (int a = wave; a < 4; a += NWV) skinny_finish<MT, EPI>(red, tile, rows, a, m0, M, N, bias, out, ldo, slab_stride);
}

// ---- one token: the norm in front of the projection inside the projection's launch -------------------
// A decode step of one request is a chain of launches of which each costs about 4.5 us before it has
// streamed a byte, the add + norm kernels in front of the q/k/v and gate/up projections among them.  With
// one row every workgroup of the projection can do that norm itself: it reads the row of the
// residual stream, the partial sums that the projection before left (pico_vllm/RMSNorm.py:22-31 for the
// norm, the sums in slab order as pico_add_rmsnorm forms them), reduces, and writes the normed row as
// bfloat16 into LDS, where it stays for all slices; only W streams.  Workgroup 0 also writes the new
// residual stream, to another buffer than the one the other workgroups still read.
struct SkNormIn {
  const float* resid;        // [M, K] float32, the residual stream before the sum
  const float* delta;        // `slabs` partial sums [M, K] float32, slab s at delta + s * slab_stride; null: nothing to add
  int slabs;
  long long slab_stride;
  const float* weight;       // [K] float32
  float eps;
  float* resid_out;          // [M, K] float32: resid + the slabs, written by workgroup 0
};
constexpr int SK_NORM_MAX_VPT = 4;                     // groups of four elements a thread: K <= 256 * 4 * 4
constexpr int SK_NORM_MAX_K = 256 * 4 * SK_NORM_MAX_VPT;
constexpr int SK_NORM_DEPTH = 3;                       // slices a wave keeps in flight in the projections of many tiles:
                                                       // 50 KB of stages and the row leave room for three workgroups a compute unit

// The one row: `load` requests the row, its partial sums and the norm's weight (before the first copies of W are
// issued: vector memory returns in order, and behind those copies this small read from the caches would wait
// for HBM); `finish` sums, norms and writes the row into xs as bfloat16 [K].
// All 256 threads of the workgroup take part in both.
// VPT: groups of four elements a thread holds (K <= 1024 VPT): what is loaded early waits in registers.
template <int VPT>
struct SkNormRow {
  float4 v[VPT], g[VPT], d[VPT][MAX_SK_SLABS];

  __device__ __forceinline__ void load(const SkNormIn& in, int K) {
#pragma unroll
    for (int j = 0; j < VPT; j++) {
      const int i = 4 * threadIdx.x + 1024 * j;
      v[j] = g[j] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int sl = 0; sl < MAX_SK_SLABS; sl++) d[j][sl] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < K) {
        v[j] = *reinterpret_cast<const float4*>(in.resid + i);
        g[j] = *reinterpret_cast<const float4*>(in.weight + i);
#pragma unroll
        for (int sl = 0; sl < MAX_SK_SLABS; sl++)
          if (sl < in.slabs) d[j][sl] = *reinterpret_cast<const float4*>(in.delta + sl * in.slab_stride + i);
      }
    }
  }

  __device__ __forceinline__ void finish(const SkNormIn& in, int K, char* xs, float* scratch, bool writer) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; j++) {
      const int i = 4 * threadIdx.x + 1024 * j;
#pragma unroll
      for (int sl = 0; sl < MAX_SK_SLABS; sl++) { v[j].x += d[j][sl].x; v[j].y += d[j][sl].y; v[j].z += d[j][sl].z; v[j].w += d[j][sl].w; }
      if (i < K) {
        if (writer) *reinterpret_cast<float4*>(in.resid_out + i) = v[j];
        ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
      }
    }
    ss = block_sum(ss, scratch);
    const float r = 1.0f / sqrtf(ss / (float)K + in.eps);
#pragma unroll
    for (int j = 0; j < VPT; j++) {
      const int i = 4 * threadIdx.x + 1024 * j;
      if (i < K) {
        *reinterpret_cast<uint2*>(xs + 2 * i) = make_uint2(pack2_bf16(v[j].x * r * g[j].x, v[j].y * r * g[j].y),
                                                   pack2_bf16(v[j].z * r * g[j].z, v[j].w * r * g[j].w));
      }
    }
    // workgroup 0 has stores on their way besides the copies: the counts that the stream waits with assume copies only
    if (writer) __builtin_amdgcn_s_waitcnt(sk_vmcnt(0));
    __syncthreads();
  }
};

// stages of the stream (4 waves, W only), then the normed row
template <int DEPTH> constexpr int sk_xs_offset() { return DEPTH * 4 * 4 * SK_GROUP; }
static int sk_xs_smem_bytes(int depth, int K) { return depth * 4 * 4 * SK_GROUP + 2 * K; }

template <int EPI, int VPT>
__global__ __launch_bounds__(256) void gemm_skinny_norm_kernel(SkNormIn in, const bf16_t* __restrict__ W, int ldw,
                                                               void* __restrict__ out, int ldo, int M, int N, int K,
                                                               int rows) {
  constexpr int DEPTH = SK_NORM_DEPTH;
  extern __shared__ __attribute__((aligned(16))) char dsmem[];
  __shared__ float scratch[16];
  char* xs = dsmem + sk_xs_offset<DEPTH>();
  const int wave = threadIdx.x >> 6, tile = blockIdx.x;
  SkNormRow<VPT> row;
  skinny_stream_lds<1, 1, 4, DEPTH, true>(nullptr, 0, W, ldw, skinny_rows<EPI>(tile, rows, N), 0, M, 0, K, dsmem, xs,
                                          [&]() { row.load(in, K); },
                                          [&]() { row.finish(in, K, xs, scratch, blockIdx.x == 0); });
  float(*red)[1][16][64] = reinterpret_cast<float(*)[1][16][64]>(dsmem);
  skinny_finish<1, EPI>(red, tile, rows, wave, 0, M, N, nullptr, out, ldo, 0);
}

// ---- 33 to 64 tokens, large grids: two tiles of W share the activations ---------------------------
// With 64 tokens a slice of activations is twice the bytes of a tile's slice of W, and every tile
// fetches it again from the L2: that traffic, not HBM, bounds the stream (the 55 MB gate/up matrix
// brings 110 MB of activations with it).  Here a workgroup owns 64 rows of W, two tiles, and four
// waves (r, p) = (wave / 2, wave % 2): wave (r, p) multiplies tile r by the slices of parity p, and
// the two waves of a parity share the activations of their slice, each copying half of them.  What
// is shared needs a barrier per step; a step is one slice per parity, two stages alternate.  Slice
// s of the k range still goes to set s % 4 of the sums, so a row's result is what the other
// kernels give.
constexpr int SK_PAIR_HALF = 16 * SK_GROUP;          // one parity of a stage: [W tile 0: 4 groups][W tile 1: 4][activations: 8]
constexpr int SK_PAIR_STAGE = 2 * SK_PAIR_HALF;
constexpr int SK_PAIR_SMEM = 2 * SK_PAIR_STAGE;      // 66,560 bytes: two workgroups share a compute unit; holds 2 x 32 KB of sums
static_assert(SK_PAIR_SMEM >= 2 * 4 * 2 * 16 * 64 * 4, "the sums of both tiles take the place of the stages");

// tr: the tile of this wave.  Leaves the sums of tile r in red[r][set][token block][register][lane] at the start of smem.
__device__ __forceinline__ void skinny_stream_pair(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W,
                                                   int ldw, TileRows tr, int m0, int M, int k_begin,
                                                   int k_end, char* smem) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = wave >> 1, p = wave & 1;
  const int col = lane & 31, h = lane >> 5, rho = lane >> 3, pos = lane & 7;
  const bf16_t* wsrc[4];
#pragma unroll
  for (int g = 0; g < 4; g++) wsrc[g] = W + (size_t)tr.row(8 * g + rho) * ldw + 8 * (pos ^ rho);
  const bf16_t* xsrc[4];                       // this wave copies the token groups 4 r .. 4 r + 3 of its parity's slice
#pragma unroll
  for (int g = 0; g < 4; g++) xsrc[g] = X + (size_t)min(m0 + 8 * (4 * r + g) + rho, M - 1) * ldx + 8 * (pos ^ rho);
  int rd[4];
#pragma unroll
  for (int s = 0; s < 4; s++) rd[s] = (col >> 3) * SK_GROUP + (col & 7) * 128 + (((4 * h + s) ^ (col & 7)) << 4);
  f32x16 acc[2][2];                            // [token block][set of the wave: slice i of the wave goes to set i % 2]
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int v = 0; v < 2; v++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[t][v][q] = 0.f;

  const int n_total = (k_end - k_begin) >> 6;  // whole slices: the caller has checked
  const int n_steps = (n_total + 1) >> 1;      // the same for every wave: the barriers below are met by all
  const int n_mine = (n_total + 1 - p) >> 1;   // slices k_begin + 64 (p + 2 i), i < n_mine
  auto issue = [&](int d, int i) {
    if (i >= n_mine) return;
    const int k0 = k_begin + 64 * (p + 2 * i);
    char* half = smem + d * SK_PAIR_STAGE + p * SK_PAIR_HALF;
#pragma unroll
    for (int g = 0; g < 4; g++)
      __builtin_amdgcn_global_load_lds(GPTR(wsrc[g] + k0), LPTR(half + (4 * r + g) * SK_GROUP), 16, 0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++)
      __builtin_amdgcn_global_load_lds(GPTR(xsrc[g] + k0), LPTR(half + (8 + 4 * r + g) * SK_GROUP), 16, 0, 0);
  };
  auto multiply = [&](auto dc, int i) {
    constexpr int d = decltype(dc)::value;     // stage and set of the sums alike
    if (i >= n_mine) return;
    const char* half = smem + d * SK_PAIR_STAGE + p * SK_PAIR_HALF;
    u32x4 a[4], b[2][4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      a[s] = *reinterpret_cast<const u32x4*>(half + 4 * r * SK_GROUP + rd[s]);
#pragma unroll
      for (int t = 0; t < 2; t++) b[t][s] = *reinterpret_cast<const u32x4*>(half + (8 + 4 * t) * SK_GROUP + rd[s]);
    }
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int t = 0; t < 2; t++)
        acc[t][d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[s]), __builtin_bit_cast(bf16x8, b[t][s]),
                                                            acc[t][d], 0, 0, 0);
  };
  issue(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  for (int i = 0; i < n_steps; i += 2) {
    // The copies of step i have landed for this wave, after the barrier for all; every wave has also
    // issued the products of step i - 1 by then, so its operand reads of the other stage are complete
    // and the stage can be filled again.  The compiler does not order LDS reads after these copies by itself.
    __builtin_amdgcn_s_waitcnt(sk_vmcnt(0));
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    issue(1, i + 1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(std::integral_constant<int, 0>{}, i);
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < n_steps) {
      __builtin_amdgcn_s_waitcnt(sk_vmcnt(0));
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      issue(0, i + 2);
      __builtin_amdgcn_sched_barrier(0);
      multiply(std::integral_constant<int, 1>{}, i + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __syncthreads();                             // every wave is done with the stages: the sums take their place
  float(*red)[2][16][64] = reinterpret_cast<float(*)[2][16][64]>(smem) + 4 * r;
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int v = 0; v < 2; v++)
#pragma unroll
      for (int q = 0; q < 16; q++) red[p + 2 * v][t][q][lane] = acc[t][v][q];
  __syncthreads();
}

template <int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_pair_kernel(const bf16_t* __restrict__ X, int ldx,
                                                               const bf16_t* __restrict__ W, int ldw,
                                                               const float* __restrict__ bias, void* __restrict__ out,
                                                               int ldo, long long slab_stride, int M, int N, int K,
                                                               int k_per_wg, int rows) {
  __shared__ __attribute__((aligned(16))) char smem[SK_PAIR_SMEM];
  const int wave = threadIdx.x >> 6;
  const int tile = 2 * blockIdx.x + (wave >> 1);     // of this wave while it streams
  const int m0 = blockIdx.z * 64;
  const int k_begin = blockIdx.y * k_per_wg, k_end = min(K, k_begin + k_per_wg);
  skinny_stream_pair(X, ldx, W, ldw, skinny_rows<EPI>(tile, rows, N), m0, M, k_begin, k_end, smem);
  float(*red)[2][16][64] = reinterpret_cast<float(*)[2][16][64]>(smem);
  for (int item = wave; item < 8; item += 4)         // (tile of the pair, a)
    skinny_finish<2, EPI>(red + 4 * (item >> 2), 2 * blockIdx.x + (item >> 2), rows, item & 3, m0, M, N, bias, out, ldo, slab_stride);
}

// How many rows of W (pairs of rows for the SwiGLU and rotation epilogues, `unit` = 2 rows) a tile gets:
// the time of a launch goes with what the fullest compute unit reads, its workgroups' rows of W and the
// activations that each workgroup reads again, so take the height with the least of it (a tile taller than
// 32 rows, whose blocks share the activations, would read less still, but left with one workgroup of few
// slices in flight per compute unit it measured slower); ties go to the taller tile.  total: rows (pairs) of the matrix; k_splits: ranges
// of k, each a workgroup of its own; x_rows: rows of activations a workgroup fetches per slice.
// Compute units of the current device, asked once per device; 256 (an MI355X) where no device answers (a build
// check without a GPU).
static int sk_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
#define SK_COMPUTE_UNITS sk_compute_units()
static int skinny_tile_height(long long total, int unit, int k_splits, int x_rows, double* cost_out = nullptr,
                              int tiles_per_wg = 1, int step = 1) {
  int best = 0;
  double best_cost = 0;
  const int cus = SK_COMPUTE_UNITS;
  for (int h = 32 / unit; h >= 1; h -= step) {       // rows or pairs per tile
    const long long wgs = (total + h * tiles_per_wg - 1) / (h * tiles_per_wg) * k_splits;
    // whole rounds of workgroups while they are few; many rounds run into one another
    const double rounds = wgs <= 4 * cus ? (double)((wgs + cus - 1) / cus) : (double)wgs / cus;
    const double cost = rounds * (h * unit * tiles_per_wg + x_rows);
    if (best == 0 || cost < best_cost) best = h, best_cost = cost;
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

// Into how many ranges of whole 256-wide steps the k of a small matrix [N, K] is cut, each range a
// workgroup of its own that leaves a float32 slab of partial sums: the cut for which the fullest
// compute unit reads least (ties: fewer slabs).  It depends on the matrix alone, never on the number
// of tokens, so that a token's sums are formed in the same order whatever comes with it.
extern "C" int pico_gemm_skinny_k_splits(int N, int K, int max_splits) {
  int best = 1;
  double best_cost = 0;
  for (int want = 1; want <= max_splits; want++) {
    const int per = ((K + want - 1) / want + 255) / 256 * 256;
    if ((K + per - 1) / per != want) continue;       // ranges would be empty
    double cost;
    skinny_tile_height(N, 1, want, 8, &cost);
    cost *= per;
    if (want == 1 || cost < best_cost) best = want, best_cost = cost;
  }
  return best;
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
  const int k_per_wg = ((K + k_splits - 1) / k_splits + 255) / 256 * 256;
  const int ky = (K + k_per_wg - 1) / k_per_wg;
  PICO_REQUIRE(ky == k_splits, "pico_gemm_skinny: K=%d cannot be cut into %d ranges of whole 256-wide steps (got %d)", K, k_splits, ky);
  const bool tail = K % 64 != 0;
  // few rows and whole slices: the stream through LDS, with as many 8-token groups as hold tokens
  const int nx = tail ? 0 : (mt == 2 ? 8 : M <= 8 ? 1 : M <= 16 ? 2 : 4);
  const int unit = epilogue == EPI_SWIGLU ? 2 : 1;
  const int total = epilogue == EPI_SWIGLU ? N / 2 : N;
  // the tile height that fills the chip best; 33 to 64 tokens and whole slices: also whether two tiles of
  // W per workgroup, which share the activations, do better than one
  double cost1, cost2 = 0;
  int rows = skinny_tile_height(total, unit, ky, mt == 2 ? 64 : M <= 8 ? 8 : M <= 16 ? 16 : 32, &cost1);
  const int rows2 = nx == 8 ? skinny_tile_height(total, unit, ky, 64, &cost2, 2) : 0;
  const bool pair = nx == 8 && cost2 < cost1;
  if (pair) rows = rows2;
  const int tiles = (total + rows - 1) / rows;
  dim3 grid(tiles, ky, (M + 32 * mt - 1) / (32 * mt));
  PICO_REQUIRE(grid.z <= 65535 && grid.y <= 65535, "pico_gemm_skinny: too many blocks");
  const float* b0 = bias;
  if (pair) {
    dim3 pgrid((tiles + 1) / 2, ky, grid.z);
#define LAUNCHP(EPI) \
  gemm_skinny_pair_kernel<EPI><<<pgrid, 256, 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, ldw, b0, out, ldo, slab_stride, M, N, K, k_per_wg, rows)
    if (epilogue == EPI_BF16) LAUNCHP(EPI_BF16);
    else if (epilogue == EPI_F32) LAUNCHP(EPI_F32);
    else LAUNCHP(EPI_SWIGLU);
#undef LAUNCHP
    PICO_LAUNCH_CHECK();
    return 0;
  }
  // 33 to 64 tokens and at most one workgroup per compute unit (the O and down projections): four waves and
  // three slices each in flight instead of two and two (19.9 against 19.5 thousand tokens a second at batch
  // 64); with fewer tokens the same made the step slower (707 against 721 tokens a second at batch 1)
  const long long workgroups = (long long)grid.x * grid.y * grid.z;
  const bool few = nx == 8 && workgroups <= SK_COMPUTE_UNITS;
  // up to 32 tokens and more than two workgroups per compute unit: smaller workgroups (shallower stages up to 16
  // tokens, two waves beyond), three or four of them a unit
  const bool many = workgroups > 2 * SK_COMPUTE_UNITS;
#define LAUNCH4(MT, EPI, TAIL, NX, FILL) \
  gemm_skinny_kernel<MT, EPI, TAIL, NX, FILL><<<grid, 64 * sk_waves<MT, NX, FILL>(), 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, ldw, b0, out, ldo, slab_stride, M, N, K, k_per_wg, rows)
#define LAUNCH(EPI)                                               \
  do {                                                            \
    if (nx == 1 && many) LAUNCH4(1, EPI, false, 1, SK_MANY);      \
    else if (nx == 1) LAUNCH4(1, EPI, false, 1, 0);               \
    else if (nx == 2 && many) LAUNCH4(1, EPI, false, 2, SK_MANY); \
    else if (nx == 2) LAUNCH4(1, EPI, false, 2, 0);               \
    else if (nx == 4 && many) LAUNCH4(1, EPI, false, 4, SK_MANY); \
    else if (nx == 4) LAUNCH4(1, EPI, false, 4, 0);               \
    else if (nx == 8 && few) LAUNCH4(2, EPI, false, 8, SK_FEW);   \
    else if (nx == 8) LAUNCH4(2, EPI, false, 8, 0);               \
    else if (mt == 1) LAUNCH4(1, EPI, true, 0, 0);                \
    else LAUNCH4(2, EPI, true, 0, 0);                             \
  } while (0)
  if (epilogue == EPI_BF16) LAUNCH(EPI_BF16);
  else if (epilogue == EPI_F32) LAUNCH(EPI_F32);
  else LAUNCH(EPI_SWIGLU);
#undef LAUNCH4
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

static int sk_check_norm(const char* who, const float* resid, const float* delta, int slabs, long long slab_stride,
                         const float* norm_w, float eps, const float* resid_out, int M, int K) {
  PICO_REQUIRE(M == 1, "%s: one row, got %d", who, M);
  PICO_REQUIRE(K > 0 && K % 64 == 0 && K <= SK_NORM_MAX_K, "%s: K = %d must be a multiple of 64 up to %d", who, K, SK_NORM_MAX_K);
  PICO_REQUIRE(resid && norm_w && resid_out && resid_out != resid, "%s: the residual stream needs a buffer of its own to go to", who);
  PICO_REQUIRE(eps > 0.f, "%s: eps must be positive", who);
  PICO_REQUIRE(delta ? (slabs >= 1 && slabs <= MAX_SK_SLABS && slab_stride >= (long long)M * K && slab_stride % 4 == 0) : slabs == 0,
               "%s: 1 to %d slabs of at least M * K floats each, or none (got %d, stride %lld)", who, MAX_SK_SLABS, slabs, slab_stride);
  PICO_REQUIRE((uintptr_t)resid % 16 == 0 && (uintptr_t)delta % 16 == 0 && (uintptr_t)norm_w % 16 == 0 && (uintptr_t)resid_out % 16 == 0,
               "%s: the norm's operands must be 16-byte aligned", who);
  return 0;
}

// A kernel may be launched with `bytes` of dynamic LDS once it has been allowed that much; `allowed` is the
// kernel's own record of it (one per instantiation, at the call site).
template <typename Kernel>
static int sk_raise_lds(Kernel kernel, int bytes, int* allowed, const char* who) {
  PICO_REQUIRE(bytes <= 160 * 1024, "%s: %d bytes of LDS are more than a compute unit has", who, bytes);
  if (bytes <= *allowed) return 0;
  if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    pico_set_error("%s: %d bytes of LDS refused", who, bytes);
    return -1;
  }
  *allowed = bytes;
  return 0;
}

// out = epilogue(norm(resid + slabs) W^T) for one row, the norm as pico_add_rmsnorm
// computes it; resid_out [M, K] gets resid + slabs.  epilogue: EPI_BF16, EPI_F32 (one slab) or EPI_SWIGLU.
extern "C" int pico_gemm_skinny_norm(const float* resid, const float* delta, int slabs, long long slab_stride,
                                     const float* norm_w, float eps, float* resid_out, const void* W, int ldw, void* out,
                                     int ldo, int epilogue, int M, int N, int K, hipStream_t stream) {
  if (sk_check_norm("pico_gemm_skinny_norm", resid, delta, slabs, slab_stride, norm_w, eps, resid_out, M, K)) return -1;
  PICO_REQUIRE(N > 0 && ldw % 8 == 0 && ldw >= K && (uintptr_t)W % 16 == 0, "pico_gemm_skinny_norm: W must be 16-byte aligned with a row stride that is a multiple of 8");
  PICO_REQUIRE(epilogue >= 0 && epilogue <= 2, "pico_gemm_skinny_norm: unknown epilogue %d", epilogue);
  PICO_REQUIRE(epilogue != EPI_SWIGLU || N % 2 == 0, "pico_gemm_skinny_norm: SwiGLU needs an even N");
  const int n_out = epilogue == EPI_SWIGLU ? N / 2 : N;
  PICO_REQUIRE(ldo >= n_out, "pico_gemm_skinny_norm: output row stride too small");
  const int unit = epilogue == EPI_SWIGLU ? 2 : 1;
  const int rows = skinny_tile_height(n_out, unit, 1, 8);
  const int tiles = (n_out + rows - 1) / rows;
  const int smem = sk_xs_smem_bytes(SK_NORM_DEPTH, K);
  const SkNormIn in = {resid, delta, slabs, slab_stride, norm_w, eps, resid_out};
#define LAUNCHV(EPI, VPT)                                                                                  \
  do {                                                                                                    \
    static int allowed = 0;                                                                               \
    if (sk_raise_lds(gemm_skinny_norm_kernel<EPI, VPT>, smem, &allowed, "pico_gemm_skinny_norm")) return -1; \
    gemm_skinny_norm_kernel<EPI, VPT><<<dim3(tiles), 256, smem, stream>>>(in, (const bf16_t*)W, ldw, out, ldo, M, N, K, rows); \
  } while (0)
#define LAUNCHN(EPI)            \
  do {                          \
    if (K <= 2048) LAUNCHV(EPI, 2); \
    else LAUNCHV(EPI, 4);       \
  } while (0)
  if (epilogue == EPI_BF16) LAUNCHN(EPI_BF16);
  else if (epilogue == EPI_F32) LAUNCHN(EPI_F32);
  else LAUNCHN(EPI_SWIGLU);
#undef LAUNCHN
#undef LAUNCHV
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The q/k/v projection of a decode step with everything that follows it before attention:
// bias, rotate-half position encoding of q and k (pico_vllm/kernels/fused_rope_kvcache_store.py:51-101
// fuses the rotation with the store; here both ride on the projection) and the store of k and v
// into the paged cache.  W = [q heads | k heads | v heads] x d rows.  A tile of a q or k head
// holds `pairs` (16, 8 or 4: what fills the chip best) rows j .. of the head and the rows j + d/2 ..
// they are rotated with, so a pair is local to a lane as gate and up are in the SwiGLU epilogue; a
// tile of a v head holds 2 `pairs` consecutive rows.  Needs rot == d and d % 32 == 0.
//   cos_sin [M][d / 2][2] float32: cosine and sine of every token's angles (pico_rope_table);
//   q_out [M, ldq] bfloat16 gets the rotated q heads at columns head * d + dim;
//   K pages [page][kv head][slot][d], V pages [page][kv head][d][slot], P = 1 << pshift slots;
//   slots[m] = page * P + slot of token m, negative: store nothing.
// ---------------------------------------------------------------------------
// XS: the activations are put into LDS at `xs` by `between` (a norm in front of the projection) and stay there.
template <int MT, bool TAIL, int NX, bool XS = false, typename Before = SkNothing, typename Between = SkNothing>
__device__ __forceinline__ void skinny_rope_body(
    const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw, const float* __restrict__ bias,
    bf16_t* __restrict__ q_out, int ldq, const float2* __restrict__ cos_sin, const int* __restrict__ slots,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int M, int K,
    int nq, int nkv, int d, int pshift, int num_pages, int pairs, char* smem, const char* xs = nullptr,
    Before before = Before(), Between between = Between()) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int half = d >> 1, tiles_per_head = half / pairs;
  const int head = blockIdx.x / tiles_per_head, tp = blockIdx.x % tiles_per_head;
  const int m0 = blockIdx.z * 32 * MT;
  const bool rotated = head < nq + nkv;
  TileRows tr;
  if (rotated) {                      // `pairs` dimensions j and the ones they are rotated with
    tr.row_a = head * d + pairs * tp;
    tr.row_b = tr.row_a + half;
    tr.va = tr.vb = pairs;
  } else {                            // 2 `pairs` consecutive dimensions
    tr.row_a = head * d + 2 * pairs * tp;
    tr.row_b = tr.row_a + 16;
    tr.va = min(2 * pairs, 16);
    tr.vb = 2 * pairs - tr.va;
  }
  // What the epilogue needs besides the sums is read now, so that the stream hides the latency: thread
  // (wave a, lane (col, h)) finishes tile rows 8 a + 4 h + 0..3 of token block t's column `col`.
  static_assert(sk_waves<MT, NX, SK_FEW>() == 4, "one wave per 8 tile rows");
  const int a = wave, t0 = 8 * a + 4 * h;
  const bool mine = rotated ? (a < 2 && t0 < pairs) : t0 < 2 * pairs;
  const int e0 = rotated ? pairs * tp + t0 : 2 * pairs * tp + t0;      // first of this thread's four head dimensions
  float b1[4] = {0.f, 0.f, 0.f, 0.f}, b2[4] = {0.f, 0.f, 0.f, 0.f};
  float2 cs[MT][4];
  int slot[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) {
    slot[t] = -1;
#pragma unroll
    for (int b = 0; b < 4; b++) cs[t][b] = make_float2(1.f, 0.f);
  }
  if (mine) {
    if (bias) {
#pragma unroll
      for (int b = 0; b < 4; b++) {
        b1[b] = bias[head * d + e0 + b];
        if (rotated) b2[b] = bias[head * d + e0 + b + half];
      }
    }
#pragma unroll
    for (int t = 0; t < MT; t++) {
      const int m = m0 + 32 * t + col;
      if (m >= M) continue;
      if (head >= nq) slot[t] = slots[m];
      if (rotated) {
#pragma unroll
        for (int b = 0; b < 4; b++) cs[t][b] = cos_sin[(size_t)m * half + e0 + b];
      }
    }
  }
  float(*red)[MT][16][64];
  if constexpr (XS) {
    skinny_stream_lds<1, 1, 4, sk_depth<1, SK_FEW>(), true>(nullptr, 0, W, ldw, tr, m0, M, 0, K, smem, xs, before, between);
    red = reinterpret_cast<float(*)[MT][16][64]>(smem);
  } else {
    red = skinny_tile<MT, TAIL, NX, SK_FEW>(X, ldx, W, ldw, tr, m0, M, 0, K, smem);
  }
  if (!mine) return;

#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int m = m0 + 32 * t + col;
    if (m >= M) continue;
    const int page = slot[t] >> pshift;
    if (head >= nq && (slot[t] < 0 || page >= num_pages)) continue;   // padding row; the host has checked the rest
    if (rotated) {
      float y1[4], y2[4];
#pragma unroll
      for (int b = 0; b < 4; b++) {
        float x1 = 0.f, x2 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
          x1 += red[w][t][4 * a + b][lane];
          x2 += red[w][t][4 * (a + 2) + b][lane];
        }
        // rounded as the projection's output is when it goes through memory, so that a token gets
        // the same key whether it came in a small step (here) or in a large one
        x1 = bf16_to_f32(f32_to_bf16(x1 + b1[b]));
        x2 = bf16_to_f32(f32_to_bf16(x2 + b2[b]));
        const float c = cs[t][b].x, sn = cs[t][b].y;
        y1[b] = x1 * c - x2 * sn;
        y2[b] = x2 * c + x1 * sn;
      }
      bf16_t* o = head < nq ? q_out + (size_t)m * ldq + head * d + e0
                            : k_cache + ((((size_t)page * nkv + (head - nq)) << pshift) + (slot[t] & ((1 << pshift) - 1))) * d + e0;
      *reinterpret_cast<uint2*>(o) = make_uint2(pack2_bf16(y1[0], y1[1]), pack2_bf16(y1[2], y1[3]));
      *reinterpret_cast<uint2*>(o + half) = make_uint2(pack2_bf16(y2[0], y2[1]), pack2_bf16(y2[2], y2[3]));
    } else {
      bf16_t* o = v_cache + ((((size_t)page * nkv + (head - nq - nkv)) * d + e0) << pshift) + (slot[t] & ((1 << pshift) - 1));
#pragma unroll
      for (int b = 0; b < 4; b++) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) v += red[w][t][4 * a + b][lane];
        o[(size_t)b << pshift] = f32_to_bf16(v + b1[b]);
      }
    }
  }
}

template <int MT, bool TAIL, int NX>
__global__ __launch_bounds__(256) void gemm_skinny_rope_kernel(
    const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw, const float* __restrict__ bias,
    bf16_t* __restrict__ q_out, int ldq, const float2* __restrict__ cos_sin, const int* __restrict__ slots,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int M, int K,
    int nq, int nkv, int d, int pshift, int num_pages, int pairs) {
  // the grid of this projection is small (one workgroup per 32 of (nq + 2 nkv) d rows): four waves always
  __shared__ __attribute__((aligned(16))) char smem[sk_smem_bytes<MT, NX, SK_FEW>()];
  skinny_rope_body<MT, TAIL, NX>(X, ldx, W, ldw, bias, q_out, ldq, cos_sin, slots, k_cache, v_cache, M, K, nq, nkv, d, pshift,
                                 num_pages, pairs, smem);
}

// the same with the norm of the one row in front (SkNormIn), the activations staying in LDS
template <int VPT>
__global__ __launch_bounds__(256) void gemm_skinny_rope_norm_kernel(
    SkNormIn in, const bf16_t* __restrict__ W, int ldw, const float* __restrict__ bias,
    bf16_t* __restrict__ q_out, int ldq, const float2* __restrict__ cos_sin, const int* __restrict__ slots,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int M, int K,
    int nq, int nkv, int d, int pshift, int num_pages, int pairs) {
  extern __shared__ __attribute__((aligned(16))) char dsmem[];
  __shared__ float scratch[16];
  char* xs = dsmem + sk_xs_offset<sk_depth<1, SK_FEW>()>();
  SkNormRow<VPT> row;
  skinny_rope_body<1, false, 1, true>(nullptr, 0, W, ldw, bias, q_out, ldq, cos_sin, slots, k_cache, v_cache, M, K, nq, nkv, d,
                                      pshift, num_pages, pairs, dsmem, xs, [&]() { row.load(in, K); },
                                      [&]() { row.finish(in, K, xs, scratch, blockIdx.x == 0); });
}

extern "C" int pico_gemm_skinny_rope(const void* X, int ldx, const void* W, int ldw, const float* bias, void* q_out,
                                     int ldq, const float* cos_sin, const int* slots,
                                     void* k_cache, void* v_cache, int M, int K, int nq, int nkv, int d, int P,
                                     int num_pages, hipStream_t stream) {
  PICO_REQUIRE(cos_sin != nullptr && (uintptr_t)cos_sin % 8 == 0, "pico_gemm_skinny_rope: no table of cosines and sines");
  PICO_REQUIRE(M > 0 && K > 0 && nq > 0 && nkv > 0 && num_pages > 0, "pico_gemm_skinny_rope: bad sizes");
  PICO_REQUIRE(d >= 32 && d % 32 == 0, "pico_gemm_skinny_rope: head size %d is not a multiple of 32", d);
  PICO_REQUIRE(P >= 1 && (P & (P - 1)) == 0, "pico_gemm_skinny_rope: page size %d is not a power of two", P);
  PICO_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K,
               "pico_gemm_skinny_rope: K and the row strides must be multiples of 8 (K=%d ldx=%d ldw=%d)", K, ldx, ldw);
  PICO_REQUIRE((uintptr_t)X % 16 == 0 && (uintptr_t)W % 16 == 0, "pico_gemm_skinny_rope: operands must be 16-byte aligned");
  PICO_REQUIRE(ldq >= nq * d && ldq % 4 == 0 && (uintptr_t)q_out % 8 == 0 && (uintptr_t)k_cache % 8 == 0,
               "pico_gemm_skinny_rope: q and the cache must be 8-byte aligned, the q row stride a multiple of 4");
  const int mt = M <= 32 ? 1 : 2;
  int pshift = 0;
  while ((1 << pshift) < P) pshift++;
  // 16, 12, 8 or 4 pairs a tile; 12 would not divide d / 2
  int pairs = skinny_tile_height((long long)(nq + 2 * nkv) * (d / 2), 2, 1, mt == 2 ? 64 : M <= 8 ? 8 : M <= 16 ? 16 : 32, nullptr, 1, 4);
  if (pairs == 12) pairs = 16;
  dim3 grid((nq + 2 * nkv) * (d / 2 / pairs), 1, (M + 32 * mt - 1) / (32 * mt));
  PICO_REQUIRE(grid.z <= 65535, "pico_gemm_skinny_rope: too many rows");
  const bool tail = K % 64 != 0;
  const int nx = tail ? 0 : (mt == 2 ? 8 : M <= 8 ? 1 : M <= 16 ? 2 : 4);
#define LAUNCH(MT, TAIL, NX) \
  gemm_skinny_rope_kernel<MT, TAIL, NX><<<grid, 64 * sk_waves<MT, NX, SK_FEW>(), 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, ldw, bias, \
      (bf16_t*)q_out, ldq, (const float2*)cos_sin, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, M, K, nq, nkv, d, pshift, num_pages, pairs)
  if (nx == 1) LAUNCH(1, false, 1);
  else if (nx == 2) LAUNCH(1, false, 2);
  else if (nx == 4) LAUNCH(1, false, 4);
  else if (nx == 8) LAUNCH(2, false, 8);
  else if (mt == 1) LAUNCH(1, true, 0);
  else LAUNCH(2, true, 0);
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

// pico_gemm_skinny_rope with the norm of the rows in front: X = norm(resid + slabs) as pico_add_rmsnorm computes it
// (one row); resid_out [1, K] gets resid + slabs.
extern "C" int pico_gemm_skinny_rope_norm(const float* resid, const float* delta, int slabs, long long slab_stride,
                                          const float* norm_w, float eps, float* resid_out, const void* W, int ldw,
                                          const float* bias, void* q_out, int ldq, const float* cos_sin, const int* slots,
                                          void* k_cache, void* v_cache, int M, int K, int nq, int nkv, int d, int P,
                                          int num_pages, hipStream_t stream) {
  if (sk_check_norm("pico_gemm_skinny_rope_norm", resid, delta, slabs, slab_stride, norm_w, eps, resid_out, M, K)) return -1;
  PICO_REQUIRE(cos_sin != nullptr && (uintptr_t)cos_sin % 8 == 0, "pico_gemm_skinny_rope_norm: no table of cosines and sines");
  PICO_REQUIRE(nq > 0 && nkv > 0 && num_pages > 0, "pico_gemm_skinny_rope_norm: bad sizes");
  PICO_REQUIRE(d >= 32 && d % 32 == 0, "pico_gemm_skinny_rope_norm: head size %d is not a multiple of 32", d);
  PICO_REQUIRE(P >= 1 && (P & (P - 1)) == 0, "pico_gemm_skinny_rope_norm: page size %d is not a power of two", P);
  PICO_REQUIRE(ldw % 8 == 0 && ldw >= K && (uintptr_t)W % 16 == 0, "pico_gemm_skinny_rope_norm: W must be 16-byte aligned with a row stride that is a multiple of 8");
  PICO_REQUIRE(ldq >= nq * d && ldq % 4 == 0 && (uintptr_t)q_out % 8 == 0 && (uintptr_t)k_cache % 8 == 0,
               "pico_gemm_skinny_rope_norm: q and the cache must be 8-byte aligned, the q row stride a multiple of 4");
  int pshift = 0;
  while ((1 << pshift) < P) pshift++;
  int pairs = skinny_tile_height((long long)(nq + 2 * nkv) * (d / 2), 2, 1, 8, nullptr, 1, 4);
  if (pairs == 12) pairs = 16;
  const int smem = sk_xs_smem_bytes(sk_depth<1, SK_FEW>(), K);
  const SkNormIn in = {resid, delta, slabs, slab_stride, norm_w, eps, resid_out};
#define LAUNCHR(VPT)                                                                                              \
  do {                                                                                                            \
    static int allowed = 0;                                                                                       \
    if (sk_raise_lds(gemm_skinny_rope_norm_kernel<VPT>, smem, &allowed, "pico_gemm_skinny_rope_norm")) return -1; \
    gemm_skinny_rope_norm_kernel<VPT><<<dim3((nq + 2 * nkv) * (d / 2 / pairs)), 256, smem, stream>>>(            \
        in, (const bf16_t*)W, ldw, bias, (bf16_t*)q_out, ldq, (const float2*)cos_sin, slots, (bf16_t*)k_cache,    \
        (bf16_t*)v_cache, M, K, nq, nkv, d, pshift, num_pages, pairs);                                            \
  } while (0)
  if (K <= 2048) LAUNCHR(2);
  else LAUNCHR(4);
#undef LAUNCHR
  PICO_LAUNCH_CHECK();
  return 0;
}
