// Sampling from float32 logits, one workgroup per row, with per-row parameters:
//   temperature == 0        argmax, lowest index on a tie            (pico_vllm/sampler.py:8)
//   top_p >= 1              draw from softmax(logits / T)             (sampler.py:16-17)
//   top_p <  1              keep the tokens whose preceding cumulative mass, in descending
//                           order of probability, is < top_p (the token that crosses stays),
//                           renormalise, draw                          (sampler.py:25-36)
// The draw is the inverse CDF in vocabulary order at the uniform number u[row] that the
// host supplies (the reference calls torch.multinomial; only the distribution is shared).
// The kept set of top-p is found without sorting: with e_i = exp((x_i - max) / T) and
// f(t) = sum of e_i > t, the kept tokens are those with e_i > t*, t* being the smallest
// float with f(t*) < top_p * sum(e), and of the tokens with e_i == t* exactly (the token that
// crosses, and any tied with it) the first ceil((top_p * sum - f(t*)) / t*) in vocabulary order:
// a sort keeps a prefix of tied tokens, not all of them (sampler.py:25-32; which of them is the
// sort's choice there, the lowest indices here, as a stable sort would).  t* comes from
// bisection over the float's bit pattern.
// All sums run in a fixed order, so a row's result depends on its inputs only.
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ float masked_sum(const float* __restrict__ x, int V, float mx, float inv_t, float thr,
                                            bool inclusive, float* scratch) {
  float s = 0.f;
  for (int i0 = threadIdx.x; i0 < V; i0 += 8 * SAMPLE_THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int i = i0 + j * SAMPLE_THREADS;
      v[j] = i < V ? x[i] : -INFINITY;           // exp(-inf) = 0 adds nothing
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float e = expf((v[j] - mx) * inv_t);
      if (inclusive ? (e >= thr) : (e > thr)) s += e;
    }
  }
  return block_sum(s, scratch);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int V,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ top_p,
                                                                const float* __restrict__ u, int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ double part[SAMPLE_THREADS];  // chunk sums in double: the CDF of 150k terms stays exact to ~1e-7
  __shared__ int idx_scratch[16];
  __shared__ int chosen_chunk;
  __shared__ double chosen_before;
  __shared__ double chosen_target;
  __shared__ int ties_before[SAMPLE_THREADS];   // tokens with e == thr in the chunks before a thread's own
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const float temp = temperature[row];

  // max and its first index
  float mx = -INFINITY;
  int mi = 0x7fffffff;
  // eight loads in flight per thread; indices rise within a thread, so ">" keeps the first maximum
  for (int i0 = tid; i0 < V; i0 += 8 * SAMPLE_THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int i = i0 + j * SAMPLE_THREADS;
      v[j] = i < V ? x[i] : -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (v[j] > mx) { mx = v[j]; mi = i0 + j * SAMPLE_THREADS; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(mx, off, 64);
    const int oi = __shfl_xor(mi, off, 64);
    if (ov > mx || (ov == mx && oi < mi)) { mx = ov; mi = oi; }
  }
  if ((tid & 63) == 0) { scratch[tid >> 6] = mx; idx_scratch[tid >> 6] = mi; }
  __syncthreads();
  mx = scratch[0]; mi = idx_scratch[0];
  for (int w = 1; w < SAMPLE_THREADS / 64; w++) {
    const float ov = scratch[w]; const int oi = idx_scratch[w];
    if (ov > mx || (ov == mx && oi < mi)) { mx = ov; mi = oi; }
  }
  __syncthreads();
  if (!(temp > 0.f)) {
    if (tid == 0) out[row] = mi;
    return;
  }
  const float inv_t = 1.0f / temp;
  const float tp = top_p[row];
  float thr = 0.f;  // keep e > thr, and the first `ties_kept` tokens with e == thr
  int ties_kept = 0x7fffffff;
  // thread i owns a contiguous chunk of the vocabulary
  const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int b = min(tid * chunk, V), e_ = min(b + chunk, V);
  int my_ties_before = 0;
  if (tp < 1.0f) {
    const float total = masked_sum(x, V, mx, inv_t, -1.f, false, scratch);
    const float target = tp * total;
    uint32_t lo = 0u, hi = 0x3f800000u;  // f(lo) >= target, f(hi) = 0 < target
    while (hi - lo > 1u) {
      const uint32_t mid = lo + (hi - lo) / 2u;
      const float f = masked_sum(x, V, mx, inv_t, __uint_as_float(mid), false, scratch);
      if (f < target) hi = mid; else lo = mid;
    }
    thr = __uint_as_float(hi);
    // the mass above the threshold is below the target; tied tokens are taken, in vocabulary order, while
    // the mass before them still is
    const float above = masked_sum(x, V, mx, inv_t, thr, false, scratch);
    ties_kept = max(1, (int)ceilf((target - above) / thr));
    int mine = 0;
    for (int i = b; i < e_; i++) mine += expf((x[i] - mx) * inv_t) == thr;
    ties_before[tid] = mine;
    __syncthreads();
    if (tid == 0) {
      int run = 0;
      for (int i = 0; i < SAMPLE_THREADS; i++) { const int n = ties_before[i]; ties_before[i] = run; run += n; }
    }
    __syncthreads();
    my_ties_before = ties_before[tid];
  }
  // inverse CDF over the kept tokens in vocabulary order
  double s = 0.0;
  {
    int tie = my_ties_before;
    for (int i = b; i < e_; i++) {
      const float e = expf((x[i] - mx) * inv_t);
      if (e > thr || (e == thr && tie++ < ties_kept)) s += (double)e;
    }
  }
  part[tid] = s;
  __syncthreads();
  if (tid == 0) {
    double kept = 0.0;
    for (int i = 0; i < SAMPLE_THREADS; i++) kept += part[i];
    const double target = (double)u[row] * kept;
    double run = 0.0;
    int c = -1, last_nonzero = 0;
    double before_last = 0.0;
    for (int i = 0; i < SAMPLE_THREADS; i++) {
      if (part[i] > 0.0) { last_nonzero = i; before_last = run; }
      if (run + part[i] > target) { c = i; break; }
      run += part[i];
    }
    if (c < 0) { c = last_nonzero; run = before_last; }
    chosen_chunk = c;
    chosen_before = run;
    chosen_target = target;
  }
  __syncthreads();
  if (tid == chosen_chunk) {
    const double target = chosen_target;
    double run = chosen_before;
    int pick = -1, last_kept = mi, tie = my_ties_before;
    for (int i = b; i < e_; i++) {
      const float e = expf((x[i] - mx) * inv_t);
      if (e > thr || (e == thr && tie++ < ties_kept)) {
        last_kept = i;
        run += (double)e;
        if (run > target) { pick = i; break; }
      }
    }
    out[row] = pick >= 0 ? pick : last_kept;
  }
}

extern "C" int pico_sample(const float* logits, int ld, int R, int V, const float* temperature, const float* top_p,
                           const float* u, int* out, hipStream_t stream) {
  PICO_REQUIRE(R >= 0 && V > 0 && ld >= V, "pico_sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  if (R == 0) return 0;
  sample_kernel<<<R, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, top_p, u, out);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Greedy rows only: the argmax in two launches.  One workgroup per row reads the row no faster than
// one compute unit takes data in (19 us for 151,936 logits); ARGMAX_CHUNKS workgroups per row find the
// first maximum of a chunk each, a second launch picks among them (the lowest index on a tie, as above).
// ---------------------------------------------------------------------------
#define ARGMAX_CHUNKS 32

__device__ __forceinline__ void keep_first_max(float& mx, int& mi, float ov, int oi) {
  if (ov > mx || (ov == mx && oi < mi)) { mx = ov; mi = oi; }
}

__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits, int ld, int V,
                                                          float* __restrict__ part_val, int* __restrict__ part_idx) {
  __shared__ float vals[4];
  __shared__ int idxs[4];
  const int row = blockIdx.x, c = blockIdx.y, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int len = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
  const int begin = min(V, c * len), end = min(V, begin + len);
  float mx = -INFINITY;
  int mi = 0x7fffffff;
  // four loads in flight per thread; indices rise within a thread, so ">" keeps the first maximum
  for (int i0 = begin + tid; i0 < end; i0 += 4 * 256) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int i = i0 + j * 256;
      v[j] = i < end ? x[i] : -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (v[j] > mx) { mx = v[j]; mi = i0 + j * 256; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) keep_first_max(mx, mi, __shfl_xor(mx, off, 64), __shfl_xor(mi, off, 64));
  if ((tid & 63) == 0) { vals[tid >> 6] = mx; idxs[tid >> 6] = mi; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 4; w++) keep_first_max(mx, mi, vals[w], idxs[w]);
    part_val[row * ARGMAX_CHUNKS + c] = mx;
    part_idx[row * ARGMAX_CHUNKS + c] = mi;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                                                          int* __restrict__ out) {
  const int row = blockIdx.x, lane = threadIdx.x;
  float mx = lane < ARGMAX_CHUNKS ? part_val[row * ARGMAX_CHUNKS + lane] : -INFINITY;
  int mi = lane < ARGMAX_CHUNKS ? part_idx[row * ARGMAX_CHUNKS + lane] : 0x7fffffff;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) keep_first_max(mx, mi, __shfl_xor(mx, off, 64), __shfl_xor(mi, off, 64));
  if (lane == 0) out[row] = mi;
}

// part_val, part_idx: workspace of R * pico_argmax_chunks() entries each
extern "C" int pico_argmax_chunks() { return ARGMAX_CHUNKS; }

extern "C" int pico_argmax(const float* logits, int ld, int R, int V, float* part_val, int* part_idx, int* out,
                           hipStream_t stream) {
  PICO_REQUIRE(R >= 0 && V > 0 && ld >= V, "pico_argmax: bad sizes R=%d V=%d ld=%d", R, V, ld);
  PICO_REQUIRE(R <= 65535, "pico_argmax: too many rows");
  if (R == 0) return 0;
  argmax_part_kernel<<<dim3(R, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, ld, V, part_val, part_idx);
  argmax_final_kernel<<<R, 64, 0, stream>>>(part_val, part_idx, out);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The same two launches with the chunk maxima in memory of the library's own (no_alloc.h).
// ---------------------------------------------------------------------------
#include "no_alloc.h"

#include <mutex>

#define NOALLOC_ENTRIES (PICO_NOALLOC_MAX_ROWS * ARGMAX_CHUNKS)
#define NOALLOC_MAX_DEVICES 64

// [values: NOALLOC_ENTRIES floats][indices: NOALLOC_ENTRIES ints].  In host code this name is only a handle
// for hipGetSymbolAddress; the address that kernels and copies take is g_scratch_ptr[device].
static __device__ __align__(256) unsigned char scratch[NOALLOC_ENTRIES * (sizeof(float) + sizeof(int))];

static void* g_scratch_ptr[NOALLOC_MAX_DEVICES];     // per device: where that GPU's copy of the array lies
static std::mutex g_scratch_mutex;

// The address of the current device's copy, looked up once per device with that device current.
static int noalloc_scratch(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  PICO_REQUIRE(e == hipSuccess, "pico_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
  PICO_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES, "pico_noalloc: device %d is beyond the %d this library keeps", dev,
               NOALLOC_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    PICO_REQUIRE(e == hipSuccess && p != nullptr, "pico_noalloc: hipGetSymbolAddress failed on device %d: %s", dev,
                 hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int pico_noalloc_max_rows() { return PICO_NOALLOC_MAX_ROWS; }

extern "C" int pico_noalloc_init() {
  void* p = nullptr;
  return noalloc_scratch(&p);
}

extern "C" int pico_argmax_noalloc(const float* logits, int ld, int R, int V, int* out, hipStream_t stream) {
  PICO_REQUIRE(R >= 0 && V > 0 && ld >= V, "pico_argmax_noalloc: bad sizes R=%d V=%d ld=%d", R, V, ld);
  PICO_REQUIRE(R <= PICO_NOALLOC_MAX_ROWS, "pico_argmax_noalloc: %d rows, the library's own memory holds %d; "
               "use pico_argmax with a workspace", R, PICO_NOALLOC_MAX_ROWS);
  PICO_REQUIRE(logits != nullptr && out != nullptr, "pico_argmax_noalloc: null pointer");
  if (R == 0) return 0;
  void* base = nullptr;
  if (noalloc_scratch(&base) != 0) return -1;
  float* part_val = reinterpret_cast<float*>(base);
  int* part_idx = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(base) + NOALLOC_ENTRIES * sizeof(float));
  // the first launch writes entries [0, R * ARGMAX_CHUNKS), the second reads exactly those: nothing to clear
  argmax_part_kernel<<<dim3(R, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, ld, V, part_val, part_idx);
  argmax_final_kernel<<<R, 64, 0, stream>>>(part_val, part_idx, out);
  PICO_LAUNCH_CHECK();
  return 0;
}
