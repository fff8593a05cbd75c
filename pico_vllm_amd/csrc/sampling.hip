// Sampling from float32 logits with per-row parameters:
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
// sort's choice there, the lowest indices here, as a stable sort would).
//
// A row is read by SAMPLE_CHUNKS workgroups, one per chunk of the vocabulary (one workgroup reads a row no
// faster than one compute unit takes data in: 19 us for 151,936 logits), in a chain of launches whose
// workgroups never wait for one another: what a launch needs of the launch before it lies in memory.
//   1. the first maximum of every chunk (argmax_part_kernel);
//   2. for rows with top_p < 1, five rounds that narrow t* in the order of the float's bit pattern (e lies in
//      (0, 1], where that order is the order of the values): a round lays 63 thresholds evenly between the
//      bounds lo < t* <= hi, every workgroup sorts the e of its chunk into the 64 classes between them and
//      sums each class; the next launch adds the classes of all chunks, finds between which two thresholds
//      f drops below the target and takes those as its bounds: 2^30 patterns shrink by 64 a round;
//   3. per chunk, the sum of e > t* in double and the number of e == t*;
//   4. one workgroup a row picks the chunk, then the thread, then the token at which the running sum of the
//      kept e passes u times their total, ties counted in vocabulary order.
// All sums run in a fixed order, so a row's result depends on its inputs only.  e is the hardware's exponential
// (__expf: 2^(x log2 e)) in every launch alike: what a token weighs must be the same bits wherever it is asked.
#include "common.h"

#define SAMPLE_CHUNKS 32            // as ARGMAX_CHUNKS below: the two share the first launch
#define ARGMAX_CHUNKS 32
#define SAMPLE_THREADS 256
#define SAMPLE_ROUND_THREADS 128    // of a round's workgroups: 64 classes a thread in LDS, 32 KB
#define SAMPLE_K 63                 // thresholds a round
#define SAMPLE_CLASSES (SAMPLE_K + 1)
#define SAMPLE_ROUNDS 5             // ceil(2^30 / 64^5) = 1
#define SAMPLE_PIECE 32             // the elements of the chosen chunk that a thread of the last launch holds in registers
#define SAMPLE_ONE 0x3f800000u      // the bit pattern of 1.0f: no e is above it

struct SampleChunk {
  int begin, end;
};
__device__ __forceinline__ SampleChunk sample_chunk(int V, int c) {
  const int len = (V + SAMPLE_CHUNKS - 1) / SAMPLE_CHUNKS;
  const int begin = min(V, c * len);
  return {begin, min(V, begin + len)};
}

// the row's maximum from the chunks' maxima; every lane of every wave gets it
__device__ __forceinline__ float sample_row_max(const float* __restrict__ part_val, int row) {
  const int lane = threadIdx.x & 63;
  return wave_max(lane < SAMPLE_CHUNKS ? part_val[row * SAMPLE_CHUNKS + lane] : -INFINITY);
}

// threshold j of a round with bounds lo < t* <= hi (patterns), w = hi - lo: lo + (j + 1) step with step = ceil(w / 64).
// (The last ones may lie beyond hi, where f is below the target as it is at hi: the bounds still close in by 64 a round.)
__device__ __forceinline__ uint32_t sample_step(uint32_t w) { return (w + SAMPLE_CLASSES - 1) / SAMPLE_CLASSES; }
__device__ __forceinline__ uint32_t sample_threshold(uint32_t lo, uint32_t w, int j) {
  return lo + (uint32_t)(j + 1) * sample_step(w);
}

// What a workgroup keeps of the search from launch to launch, every workgroup its own copy: lo, hi, f(hi), the target.

// lane m of the first wave: class m of the row, the chunks' sums added in the order of the chunks
__device__ __forceinline__ float sample_class_total(const float* __restrict__ classes) {
  float t = 0.f;
  if (threadIdx.x < 64) {
    float v[SAMPLE_CHUNKS];                  // all loads in flight at once
#pragma unroll
    for (int c = 0; c < SAMPLE_CHUNKS; c++) v[c] = classes[c * SAMPLE_CLASSES + threadIdx.x];
#pragma unroll
    for (int c = 0; c < SAMPLE_CHUNKS; c++) t += v[c];
  }
  return t;
}

// The bounds after the round whose class totals the first wave holds in `t`; all threads get them.
__device__ void sample_decide(float t, uint4 st, float tp, uint32_t& lo, uint32_t& hi, float& f_hi, float& target,
                              uint32_t* result) {
  static_assert(SAMPLE_CLASSES == 64, "lane m of the first wave holds class m");
  lo = st.x; hi = st.y;
  f_hi = __uint_as_float(st.z); target = __uint_as_float(st.w);
  const uint32_t w = hi - lo;
  if (w <= 1u) return;                       // found already
  const int tid = threadIdx.x;
  if (tid < 64) {
    if (!(target > 0.f)) target = tp * wave_sum(t);          // the first round: the classes hold every e of the row
    // classes m .. 63 together, in every lane m (a fixed tree of additions)
    float above = t;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float o = __shfl_down(above, off, 64);
      if (tid + off < 64) above += o;
    }
    // f(t_j) = classes j + 1 .. 63 together; the first j at which it is below the target
    const float f_j = __shfl_down(above, 1, 64);
    const unsigned long long below = __ballot(tid < SAMPLE_K && f_j < target);
    const int first = below ? __ffsll((long long)below) - 1 : SAMPLE_K;
    const float f_new = first < SAMPLE_K ? __shfl(f_j, first, 64) : f_hi;
    if (tid == 0) {
      result[0] = first > 0 ? sample_threshold(lo, w, first - 1) : lo;
      result[1] = first < SAMPLE_K ? sample_threshold(lo, w, first) : hi;
      result[2] = __float_as_uint(f_new); result[3] = __float_as_uint(target);
    }
  }
  __syncthreads();
  lo = result[0]; hi = result[1];
  f_hi = __uint_as_float(result[2]); target = __uint_as_float(result[3]);
  __syncthreads();                           // result may be written again
}

__global__ __launch_bounds__(SAMPLE_ROUND_THREADS) void sample_round_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const float* __restrict__ top_p, const float* __restrict__ part_val, const float* __restrict__ prev,
    float* __restrict__ next, uint32_t* __restrict__ state, int first) {
  __shared__ float hist[SAMPLE_CLASSES][SAMPLE_ROUND_THREADS];   // a column per thread: no two threads share an entry
  __shared__ float halves[2][SAMPLE_CLASSES];
  __shared__ uint32_t result[4];
  const int row = blockIdx.x, c = blockIdx.y, tid = threadIdx.x;
  // everything the workgroup needs from memory is asked for at once, whatever it turns out to need: what the launch
  // before wrote comes from memory, a microsecond or two away, and asking one after the other would add them up
  const float temp = temperature[row], tp = top_p[row];
  uint32_t* st = state + ((size_t)row * SAMPLE_CHUNKS + c) * 4;
  const uint4 kept = first ? make_uint4(0u, SAMPLE_ONE, 0u, 0u) : *reinterpret_cast<const uint4*>(st);
  const float t = first ? 0.f : sample_class_total(prev + (size_t)row * SAMPLE_CHUNKS * SAMPLE_CLASSES);
  const float mx = sample_row_max(part_val, row);
  const float* x = logits + (size_t)row * ld;
  const SampleChunk ch = sample_chunk(V, c);
  // eight loads in flight per thread, those of the next eight tokens issued before these are classed
  auto fetch = [&](int i0, float* v) {
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int i = i0 + k * SAMPLE_ROUND_THREADS;
      v[k] = i < ch.end ? x[i] : -INFINITY;                // exp(-inf) = 0 adds nothing to its class
    }
  };
  float v[8], ahead[8];
  fetch(ch.begin + tid, v);
  if (!(temp > 0.f) || !(tp < 1.0f)) return;
  uint32_t lo = 0u, hi = SAMPLE_ONE;
  float f_hi = 0.f, target = 0.f;
  if (!first) sample_decide(t, kept, tp, lo, hi, f_hi, target, result);
  if (tid == 0) {
    st[0] = lo; st[1] = hi;
    st[2] = __float_as_uint(f_hi); st[3] = __float_as_uint(target);
  }
  const uint32_t w = hi - lo;
  if (w <= 1u) return;
  const float inv_t = 1.0f / temp;
#pragma unroll 8
  for (int m = 0; m < SAMPLE_CLASSES; m++) hist[m][tid] = 0.f;
  const uint32_t step = sample_step(w);
  const float per_step = 1.0f / (float)step;
  for (int i0 = ch.begin + tid; i0 < ch.end; i0 += 8 * SAMPLE_ROUND_THREADS) {
    fetch(i0 + 8 * SAMPLE_ROUND_THREADS, ahead);
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const float e = __expf((v[k] - mx) * inv_t);
      const uint32_t b = __float_as_uint(e);
      // the class of e: how many thresholds lie strictly below it
      // (threshold j is below e if (j + 1) step < b - lo: floor((b - lo - 1) / step) of them, 63 at most)
      uint32_t m = 0;
      if (b > lo) {
        const uint32_t d = b - lo - 1u;
        m = min((uint32_t)((float)d * per_step), (uint32_t)SAMPLE_CLASSES);      // a guess that is off by one at most
        if ((m + 1u) * step <= d) m++;
        if (m * step > d) m--;
        m = min(m, (uint32_t)SAMPLE_K);
      }
      hist[m][tid] += e;
    }
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = ahead[k];
  }
  __syncthreads();
  // Thread (m, half) adds the entries of class m of one half of the threads, one after the other (no exchange between
  // lanes: 32 reductions over a wave would be 32 chains of six exchanges); it starts at column m so that the lanes of a
  // wave read different banks.
  static_assert(SAMPLE_ROUND_THREADS == 128 && SAMPLE_CLASSES == 64, "two halves of 64 threads, a class a lane");
  const int m = tid & 63, half = tid >> 6;
  float sum = 0.f;
#pragma unroll 16
  for (int j = 0; j < 64; j++) sum += hist[m][half * 64 + ((j + m) & 63)];
  halves[half][m] = sum;
  __syncthreads();
  if (tid < SAMPLE_CLASSES)
    next[((size_t)row * SAMPLE_CHUNKS + c) * SAMPLE_CLASSES + tid] = halves[0][tid] + halves[1][tid];
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// The terms e = exp((x - max) / t) of the elements begin + thread, begin + thread + SAMPLE_THREADS, ... of a chunk, in
// that order, eight loads in flight a thread: one load at a time, each used at once, is a chain of memory latencies
// (6 us for the 19 elements a thread has of a chunk of 151,936 logits).
template <class Use>
__device__ __forceinline__ void sample_each_term(const float* __restrict__ x, int begin, int end, float mx, float inv_t, Use use) {
  for (int i0 = begin + (int)threadIdx.x; i0 < end; i0 += 8 * SAMPLE_THREADS) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int i = i0 + k * SAMPLE_THREADS;
      v[k] = i < end ? x[i] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int i = i0 + k * SAMPLE_THREADS;
      if (i < end) use(i, __expf((v[k] - mx) * inv_t));
    }
  }
}

// per chunk: the sum of e > t* (double) and the number of e == t*; the row's t* and how many ties it keeps
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_chunk_sums_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const float* __restrict__ top_p, const float* __restrict__ part_val, const float* __restrict__ prev,
    const uint32_t* __restrict__ state, double* __restrict__ fin_s, int* __restrict__ fin_n, uint32_t* __restrict__ fin_par) {
  __shared__ uint32_t result[4];
  __shared__ double ws[SAMPLE_THREADS / 64];
  __shared__ int wn[SAMPLE_THREADS / 64];
  const int row = blockIdx.x, c = blockIdx.y, tid = threadIdx.x;
  const float temp = temperature[row], tp = top_p != nullptr ? top_p[row] : 1.0f;
  if (!(temp > 0.f)) return;
  float thr = 0.f;                            // keep e > thr, and the first `ties_kept` tokens with e == thr
  int ties_kept = 0x7fffffff;
  if (tp < 1.0f) {
    uint32_t lo, hi;
    float f_hi, target;
    sample_decide(sample_class_total(prev + (size_t)row * SAMPLE_CHUNKS * SAMPLE_CLASSES),
                  *reinterpret_cast<const uint4*>(state + ((size_t)row * SAMPLE_CHUNKS + c) * 4), tp, lo, hi, f_hi, target, result);
    thr = __uint_as_float(hi);
    // the mass above the threshold is below the target; tied tokens are taken, in vocabulary order, while
    // the mass before them still is
    ties_kept = max(1, (int)ceilf((target - f_hi) / thr));
  }
  const float mx = sample_row_max(part_val, row), inv_t = 1.0f / temp;
  const float* x = logits + (size_t)row * ld;
  const SampleChunk ch = sample_chunk(V, c);
  double s = 0.0;
  int n = 0;
  sample_each_term(x, ch.begin, ch.end, mx, inv_t, [&](int, float e) {
    if (e > thr) s += (double)e;
    n += e == thr;
  });
  s = wave_sum_f64(s);
  n = wave_sum_i32(n);
  if ((tid & 63) == 0) { ws[tid >> 6] = s; wn[tid >> 6] = n; }
  __syncthreads();
  if (tid == 0) {
    for (int k = 1; k < SAMPLE_THREADS / 64; k++) { s += ws[k]; n += wn[k]; }
    const size_t at = (size_t)row * SAMPLE_CHUNKS + c;
    fin_s[at] = s;
    fin_n[at] = n;
    fin_par[2 * at] = __float_as_uint(thr);
    fin_par[2 * at + 1] = (uint32_t)ties_kept;
  }
}

// exclusive prefix sums over the workgroup's threads, in a fixed order; `total` gets the sum of all
__device__ __forceinline__ double block_prefix_f64(double v, double* wave_tot, double& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const double o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
  }
  __syncthreads();
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  double before = 0.0;
  total = 0.0;
  for (int k = 0; k < SAMPLE_THREADS / 64; k++) {
    if (k < wave) before += wave_tot[k];
    total += wave_tot[k];
  }
  return before + incl - v;
}
__device__ __forceinline__ int block_prefix_i32(int v, int* wave_tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
  }
  __syncthreads();
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  int before = 0;
  for (int k = 0; k < wave; k++) before += wave_tot[k];
  return before + incl - v;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_pick_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const float* __restrict__ u, const float* __restrict__ part_val, const int* __restrict__ part_idx,
    const double* __restrict__ fin_s, const int* __restrict__ fin_n, const uint32_t* __restrict__ fin_par,
    int* __restrict__ out) {
  __shared__ double wave_tot[SAMPLE_THREADS / 64];
  __shared__ int wave_cnt[SAMPLE_THREADS / 64];
  __shared__ int chosen_chunk, chosen_ties_before;
  __shared__ int wave_first[SAMPLE_THREADS / 64], wave_last[SAMPLE_THREADS / 64];
  __shared__ int chunk_n[SAMPLE_CHUNKS];
  __shared__ double chunk_s[SAMPLE_CHUNKS];
  __shared__ double chosen_before, chosen_target;
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
  // the row's first maximum: what a greedy row gives, and what a draw falls back on
  float mx = lane < SAMPLE_CHUNKS ? part_val[row * SAMPLE_CHUNKS + lane] : -INFINITY;
  int mi = lane < SAMPLE_CHUNKS ? part_idx[row * SAMPLE_CHUNKS + lane] : 0x7fffffff;
  wave_first_max(mx, mi);
  const float temp = temperature[row], u_row = u[row];    // (asked for here: where it is used, one thread would wait for it)
  if (!(temp > 0.f)) {
    if (tid == 0) out[row] = mi;
    return;
  }
  const size_t base = (size_t)row * SAMPLE_CHUNKS;
  const float thr = __uint_as_float(fin_par[2 * base]);
  const int ties_kept = (int)fin_par[2 * base + 1];
  if (tid < SAMPLE_CHUNKS) {
    chunk_n[tid] = fin_n[base + tid];
    chunk_s[tid] = fin_s[base + tid];
  }
  __syncthreads();
  if (tid == 0) {
    // what every chunk keeps: its e > thr, and of its ties those that still are among the first `ties_kept`
    double kept[SAMPLE_CHUNKS], total = 0.0;
    int before[SAMPLE_CHUNKS], ties = 0;
    for (int c = 0; c < SAMPLE_CHUNKS; c++) {
      const int n = chunk_n[c];
      before[c] = ties;
      const int taken = min(n, max(0, ties_kept - min(ties, ties_kept)));
      kept[c] = chunk_s[c] + (double)thr * (double)taken;
      total += kept[c];
      ties += n;
    }
    const double target = (double)u_row * total;
    double run = 0.0, before_last = 0.0;
    int c = -1, last_nonzero = 0;
    for (int i = 0; i < SAMPLE_CHUNKS; i++) {
      if (kept[i] > 0.0) { last_nonzero = i; before_last = run; }
      if (run + kept[i] > target) { c = i; break; }
      run += kept[i];
    }
    if (c < 0) { c = last_nonzero; run = before_last; }
    chosen_chunk = c;
    chosen_before = run;
    chosen_target = target;
    chosen_ties_before = before[c];
  }
  __syncthreads();
  const SampleChunk ch = sample_chunk(V, chosen_chunk);
  const float inv_t = 1.0f / temp;
  const float* x = logits + (size_t)row * ld;
  // A thread owns a contiguous piece of the chunk and goes through it three times.  One element after the other from
  // memory, each pass is a chain of latencies (2 to 2.6 us each for the 19 elements a thread has of a chunk of
  // 151,936 logits): a piece of up to SAMPLE_PIECE elements (vocabularies up to 262,144) is asked for at once and
  // its terms wait in registers.
  auto term = [&](int i) { return __expf((x[i] - mx) * inv_t); };
  const int piece = (ch.end - ch.begin + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int b = min(ch.end, ch.begin + tid * piece), e_ = min(ch.end, b + piece);
  const bool held = piece <= SAMPLE_PIECE;                                 // the same for all threads
  float mine[SAMPLE_PIECE];
  if (held) {
#pragma unroll
    for (int k = 0; k < SAMPLE_PIECE; k++) mine[k] = b + k < e_ ? x[b + k] : 0.f;
#pragma unroll
    for (int k = 0; k < SAMPLE_PIECE; k++) mine[k] = __expf((mine[k] - mx) * inv_t);
  }
  // use(i, e) for the elements of the piece in their order, until it returns false
  auto each = [&](auto use) {
    if (held) {
#pragma unroll
      for (int k = 0; k < SAMPLE_PIECE; k++) {
        if (b + k >= e_ || !use(b + k, mine[k])) break;
      }
    } else {
      for (int i = b; i < e_; i++)
        if (!use(i, term(i))) break;
    }
  };
  int my_ties = 0;
  each([&](int, float e) { my_ties += e == thr; return true; });
  const int ties_before = chosen_ties_before + block_prefix_i32(my_ties, wave_cnt);
  double s = 0.0;
  {
    int tie = ties_before;
    each([&](int, float e) {
      if (e > thr || (e == thr && tie++ < ties_kept)) s += (double)e;
      return true;
    });
  }
  double chunk_total;
  const double before = chosen_before + block_prefix_f64(s, wave_tot, chunk_total);
  const double target = chosen_target;
  // the first thread whose piece reaches the target, and the last that keeps anything (a vote in each wave, then
  // the waves side by side: every thread asking for one word of LDS at once takes 4 us)
  {
    const unsigned long long keeps = __ballot(s > 0.0), reaches = __ballot(s > 0.0 && before + s > target);
    if (lane == 0) {
      wave_last[tid >> 6] = keeps ? (tid | 63) - __clzll(keeps) : -1;
      wave_first[tid >> 6] = reaches ? tid + __ffsll(reaches) - 1 : 0x7fffffff;
    }
  }
  __syncthreads();
  int first = 0x7fffffff, last = -1;
#pragma unroll
  for (int w = 0; w < SAMPLE_THREADS / 64; w++) {
    first = min(first, wave_first[w]);
    last = max(last, wave_last[w]);
  }
  const int who = first != 0x7fffffff ? first : last;
  if (who < 0) {                              // nothing kept in the chunk (cannot be, but a token must come out)
    if (tid == 0) out[row] = mi;
    return;
  }
  if (tid == who) {
    double run = before;
    int pick = -1, last_kept = mi, tie = ties_before;
    each([&](int i, float e) {
      if (e > thr || (e == thr && tie++ < ties_kept)) {
        if (e > 0.f) last_kept = i;           // a token whose probability underflowed to zero is never the fallback
        run += (double)e;
        if (run > target) { pick = i; return false; }
      }
      return true;
    });
    out[row] = pick >= 0 ? pick : last_kept;
  }
}

// ---------------------------------------------------------------------------
// Greedy rows only: the argmax in two launches.  One workgroup per row reads the row no faster than
// one compute unit takes data in (19 us for 151,936 logits); ARGMAX_CHUNKS workgroups per row find the
// first maximum of a chunk each, a second launch picks among them (the lowest index on a tie, as above).
// ---------------------------------------------------------------------------
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
  wave_first_max(mx, mi);
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
  wave_first_max(mx, mi);
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

// work: pico_sample_workspace_words(R) 4-byte words, 16-byte aligned.  top_p_rows == 0: no row has top_p < 1 (every
// row is treated so), and the rounds that look for the threshold are not launched.
extern "C" long long pico_sample_workspace_words(int R) {
  return (long long)R * SAMPLE_CHUNKS * (2 + 1 + 1 + 2 * SAMPLE_CLASSES + 4 + 1 + 2);
}

extern "C" int pico_sample(const float* logits, int ld, int R, int V, const float* temperature, const float* top_p,
                           const float* u, int* out, void* work, int top_p_rows, hipStream_t stream) {
  static_assert(SAMPLE_CHUNKS == ARGMAX_CHUNKS, "the first launch is the argmax's");
  PICO_REQUIRE(R >= 0 && V > 0 && ld >= V, "pico_sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  PICO_REQUIRE(R <= 65535, "pico_sample: too many rows");
  if (R == 0) return 0;
  // (the rounds read their state with 16-byte loads; every part of the workspace is a multiple of 16 bytes long)
  PICO_REQUIRE(work != nullptr && (uintptr_t)work % 16 == 0, "pico_sample: the workspace is missing or not 16-byte aligned");
  const size_t n = (size_t)R * SAMPLE_CHUNKS;
  double* fin_s = (double*)work;
  float* part_val = (float*)(fin_s + n);
  int* part_idx = (int*)(part_val + n);
  float* classes[2] = {(float*)(part_idx + n), (float*)(part_idx + n) + n * SAMPLE_CLASSES};
  uint32_t* state = (uint32_t*)(classes[1] + n * SAMPLE_CLASSES);
  int* fin_n = (int*)(state + 4 * n);
  uint32_t* fin_par = (uint32_t*)(fin_n + n);
  const dim3 grid(R, SAMPLE_CHUNKS);
  argmax_part_kernel<<<grid, 256, 0, stream>>>(logits, ld, V, part_val, part_idx);
  const float* asked = top_p_rows ? top_p : nullptr;
  if (top_p_rows)
    for (int r = 0; r < SAMPLE_ROUNDS; r++)
      sample_round_kernel<<<grid, SAMPLE_ROUND_THREADS, 0, stream>>>(logits, ld, V, temperature, top_p, part_val,
                                                                    classes[(r + 1) & 1], classes[r & 1], state, r == 0);
  sample_chunk_sums_kernel<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, asked, part_val,
                                                               classes[(SAMPLE_ROUNDS - 1) & 1], state, fin_s, fin_n, fin_par);
  sample_pick_kernel<<<R, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, u, part_val, part_idx, fin_s, fin_n,
                                                      fin_par, out);
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
