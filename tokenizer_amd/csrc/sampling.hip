// Greedy pick on the device: the first maximum wins, as a scan with `>` from -inf does.
#include "common.h"

#define ARGMAX_THREADS 256

__device__ __forceinline__ bool better(float v, int at, float best, int best_at) {
  return v > best || (v == best && at < best_at);
}

// Block-wide (maximum, lowest index of it); the result is valid in thread 0.
__device__ __forceinline__ void block_best(float& best, int& at, float* best_s, int* at_s) {
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, WAVE);
    const int oa = __shfl_xor(at, off, WAVE);
    if (better(ob, oa, best, at)) { best = ob; at = oa; }
  }
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  if (lane == 0) { best_s[wave] = best; at_s[wave] = at; }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < ARGMAX_THREADS / WAVE; ++w)
      if (better(best_s[w], at_s[w], best, at)) { best = best_s[w]; at = at_s[w]; }
}

// Stage one: each row is cut into `chunks` pieces, one workgroup per piece; a piece's (maximum, index)
// goes to partial_v / partial_i [n_rows, chunks].  NaN never wins.
__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_pieces(const float* __restrict__ logits, float* __restrict__ partial_v, int* __restrict__ partial_i,
              int vocab, int chunks) {
  __shared__ float best_s[ARGMAX_THREADS / WAVE];
  __shared__ int at_s[ARGMAX_THREADS / WAVE];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float* src = logits + (size_t)row * vocab;
  const int per = (vocab + chunks - 1) / chunks;
  const int begin = chunk * per, end = min(vocab, begin + per);
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += ARGMAX_THREADS) {
    const float v = src[i];
    if (v > best) { best = v; at = i; }          // ascending i per thread: its first maximum stays
  }
  block_best(best, at, best_s, at_s);
  if (threadIdx.x == 0) {
    partial_v[(size_t)row * chunks + chunk] = best;
    partial_i[(size_t)row * chunks + chunk] = at;
  }
}

// Stage two: one workgroup per row reduces the pieces; a row without any maximum gives index 0.
__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_rows(const float* __restrict__ partial_v, const int* __restrict__ partial_i, int* __restrict__ out,
            int chunks) {
  __shared__ float best_s[ARGMAX_THREADS / WAVE];
  __shared__ int at_s[ARGMAX_THREADS / WAVE];
  const int row = blockIdx.x;
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += ARGMAX_THREADS) {
    const float v = partial_v[(size_t)row * chunks + c];
    const int a = partial_i[(size_t)row * chunks + c];
    if (better(v, a, best, at)) { best = v; at = a; }
  }
  block_best(best, at, best_s, at_s);
  if (threadIdx.x == 0) out[row] = (at == 0x7fffffff) ? 0 : at;
}

extern "C" int ta_argmax(const void* logits, void* out, void* partial_v, void* partial_i, int n_rows, int vocab,
                         int chunks, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (chunks < 1 || vocab < 1) return -1;
  dim3 grid(chunks, n_rows);
  argmax_pieces<<<grid, ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)partial_v, (int*)partial_i,
                                                    vocab, chunks);
  int status = LAUNCH_STATUS();
  if (status) return status;
  argmax_rows<<<n_rows, ARGMAX_THREADS, 0, stream>>>((const float*)partial_v, (const int*)partial_i, (int*)out, chunks);
  return LAUNCH_STATUS();
}

// ------------------------------------------------------------------------------------------------
// Temperature / nucleus sampling without a sort.
//
// The reference orders the tokens by falling logit (lower index first among equals), keeps the shortest
// prefix whose probability reaches top_p, and walks that prefix with a uniform number until the mass is
// used up.  Both questions are "where does the running mass, in that order, cross a value": answered here
// by narrowing an order-preserving 32-bit key of the logit four bits at a time, each round summing the
// weights exp((l - max) / T) of the sixteen candidate ranges (fixed summation order, so the result does not
// change from run to run), and then counting indices among the tokens whose logit equals the crossing one.
#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t order_key(float v) {
  // Larger float -> larger key; NaN is treated as the smallest value.
  if (v != v) return 0u;
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Sums `vals[0..n)` over the block; every thread gets all n results in `vals`.  n <= 16.
__device__ __forceinline__ void block_sums(float* vals, int n, float (*scratch)[16]) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  for (int i = 0; i < n; ++i) vals[i] = wave_sum(vals[i]);
  __syncthreads();
  if (lane == 0)
    for (int i = 0; i < n; ++i) scratch[wave][i] = vals[i];
  __syncthreads();
  for (int i = 0; i < n; ++i) {
    float total = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / WAVE; ++w) total += scratch[w][i];
    vals[i] = total;
  }
}

struct Crossing {
  uint32_t key;     // key of the token at which the running mass crosses the target
  float above;      // mass of all tokens with a larger key
  float each;       // weight of one token with this key
  int rank;         // how many tokens with this key (in index order) lie before the crossing one
};

// Finds where the mass, taken in falling key order, first exceeds `target` (target < total mass).
__device__ Crossing find_crossing(const float* __restrict__ row, int vocab, float max_logit, float inv_t,
                                  float target, float (*scratch)[16]) {
  uint32_t prefix = 0;
  float above = 0.f;
  for (int shift = 28; shift >= 0; shift -= 4) {
    float part[16];
#pragma unroll
    for (int n = 0; n < 16; ++n) part[n] = 0.f;
    const uint32_t mask = (shift == 28) ? 0u : (0xffffffffu << (shift + 4));
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
      const float v = row[i];
      const uint32_t key = order_key(v);
      if ((key & mask) != prefix) continue;
      const float w = (v != v) ? 0.f : expf((v - max_logit) * inv_t);
      const uint32_t nib = (key >> shift) & 15u;
#pragma unroll
      for (int n = 0; n < 16; ++n) part[n] += (nib == (uint32_t)n) ? w : 0.f;
    }
    block_sums(part, 16, scratch);
    // Walk the ranges from the largest keys down.  If rounding leaves the target at or past the whole mass,
    // the crossing is in the last range that holds anything.
    int pick = -1, last = 0;
    float run = above, run_at_last = above;
    for (int n = 15; n >= 0; --n) {
      if (part[n] > 0.f) { last = n; run_at_last = run; }
      if (target < run + part[n]) { pick = n; break; }
      run += part[n];
    }
    if (pick < 0) { pick = last; run = run_at_last; }
    above = run;
    prefix |= (uint32_t)pick << shift;
  }
  Crossing c;
  c.key = prefix;
  c.above = above;
  c.each = 0.f;
  c.rank = 0;
  return c;
}

// One workgroup per row.  temperature > 0.  out[row] = sampled index.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const float* __restrict__ uniform, int* __restrict__ out, int vocab) {
  __shared__ float scratch[SAMPLE_THREADS / WAVE][16];
  __shared__ int count_s[SAMPLE_THREADS];
  __shared__ int found_s;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float inv_t = 1.0f / temperature[r];
  // maximum
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) mx = fmaxf(mx, row[i]);   // fmaxf skips NaN
  mx = wave_max(mx);
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE][0] = mx;
  __syncthreads();
  for (int w = 0; w < SAMPLE_THREADS / WAVE; ++w) mx = fmaxf(mx, scratch[w][0]);
  // total mass
  float total[1] = {0.f};
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
    const float v = row[i];
    total[0] += (v != v) ? 0.f : expf((v - mx) * inv_t);
  }
  block_sums(total, 1, scratch);
  const float mass = total[0];
  uint32_t pick_key;
  int pick_rank;
  if (!(mx > -INFINITY) || !(mx < INFINITY) || !(mass > 0.f) || !(mass < INFINITY)) {
    // Nothing to weigh (all -inf or NaN, or an infinite logit): the greedy choice, first maximum.
    pick_key = order_key(mx);
    pick_rank = 0;
  } else {
    // Nucleus: the kept prefix ends where the mass reaches top_p * total (at least the top token).
    float kept = mass;
    uint32_t cut_key = 0;
    int cut_rank = 0x7fffffff;                       // tokens with key == cut_key kept: ranks 0..cut_rank
    const float p = top_p[r];
    if (p < 1.0f) {
      // The reference stops at the first token with cumulative >= top_p: the crossing of a target just
      // below top_p * mass in the "exceeds" sense.
      const float target = fmaxf(0.f, nextafterf(p * mass, 0.f));
      Crossing c = find_crossing(row, vocab, mx, inv_t, target, scratch);
      const float each = expf((__uint_as_float((c.key & 0x80000000u) ? (c.key & 0x7fffffffu) : ~c.key) - mx) * inv_t);
      int rank = (each > 0.f) ? (int)floorf((target - c.above) / each) : 0;
      rank = max(rank, 0);
      cut_key = c.key;
      cut_rank = rank;
      kept = c.above + (float)(rank + 1) * each;
    }
    const float target = uniform[r] * kept;
    Crossing c = find_crossing(row, vocab, mx, inv_t, target, scratch);
    const float each = expf((__uint_as_float((c.key & 0x80000000u) ? (c.key & 0x7fffffffu) : ~c.key) - mx) * inv_t);
    int rank = (each > 0.f) ? (int)floorf((target - c.above) / each) : 0;
    rank = max(rank, 0);
    pick_key = c.key;
    pick_rank = rank;
    if (pick_key < cut_key || (pick_key == cut_key && pick_rank > cut_rank)) {   // past the kept prefix: its last token
      pick_key = cut_key;
      pick_rank = cut_rank;
    }
  }
  // The pick_rank-th lowest index among the tokens whose key is pick_key (the last of them if there are fewer).
  const int chunk = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = threadIdx.x * chunk, end = min(vocab, begin + chunk);
  int mine = 0;
  for (int i = begin; i < end; ++i) mine += (order_key(row[i]) == pick_key) ? 1 : 0;
  count_s[threadIdx.x] = mine;
  if (threadIdx.x == 0) found_s = 0;
  __syncthreads();
  if (threadIdx.x == 0) {
    int seen = 0, all = 0;
    for (int t = 0; t < SAMPLE_THREADS; ++t) all += count_s[t];
    const int want = min(pick_rank, max(all - 1, 0));
    int owner = 0;
    for (int t = 0; t < SAMPLE_THREADS; ++t) {
      if (seen + count_s[t] > want) { owner = t; break; }
      seen += count_s[t];
    }
    count_s[0] = owner;           // thread that holds the token
    found_s = want - seen;        // its rank inside that thread's chunk
  }
  __syncthreads();
  const int owner = count_s[0];
  if (threadIdx.x == owner) {
    int left = found_s, answer = 0;
    for (int i = begin; i < end; ++i) {
      if (order_key(row[i]) == pick_key) {
        if (left == 0) { answer = i; break; }
        --left;
      }
    }
    out[r] = answer;
  }
}

extern "C" int ta_sample(const void* logits, const void* temperature, const void* top_p, const void* uniform,
                         void* out, int n_rows, int vocab, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab < 1) return -1;
  sample_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>((const float*)logits, (const float*)temperature,
                                                      (const float*)top_p, (const float*)uniform, (int*)out, vocab);
  return LAUNCH_STATUS();
}
