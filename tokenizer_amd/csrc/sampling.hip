// Greedy pick on the device: the first maximum wins, as a scan with `>` from -inf does.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

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
  // Eight loads at a time (one after the other, each would be a trip to memory of its own), compared in their order.
  for (int i0 = begin + threadIdx.x; i0 < end; i0 += 8 * ARGMAX_THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[min(i0 + j * ARGMAX_THREADS, end - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j * ARGMAX_THREADS;
      if (i < end && v[j] > best) { best = v[j]; at = i; }    // ascending i per thread: its first maximum stays
    }
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

// What the description of a decode step (one token per request, row i = request i) needs to describe the step
// after it, in which every request is one position further: the picked ids as the next tokens, positions and first
// positions one up, and for every cache group the slot of the new position from the request's row of the block
// table (an entry past the row's end is not looked up: the last one stands in, and the host fills the description
// in again before a step for which that matters; a page that is not there gives no slot).
#define NEXT_STEP_GROUPS 4
struct NextStep {
  int* token_ids; int* positions; int* first_position;
  int page_size, n_groups;
  int* slots[NEXT_STEP_GROUPS];
  const int* tables[NEXT_STEP_GROUPS];
  int widths[NEXT_STEP_GROUPS];
};

// Stage two of the greedy pick as above, which also turns the step's description into the next step's: a run
// of decode steps then needs nothing from the host between its steps.
__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_rows_next(const float* __restrict__ partial_v, const int* __restrict__ partial_i, int* __restrict__ out,
                 int chunks, NextStep next) {
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
  if (threadIdx.x == 0) {
    const int id = (at == 0x7fffffff) ? 0 : at;
    out[row] = id;
    next.token_ids[row] = id;
    const int p = next.positions[row] + 1;
    next.positions[row] = p;
    next.first_position[row] = p;
#pragma unroll
    for (int g = 0; g < NEXT_STEP_GROUPS; ++g) {
      if (g < next.n_groups) {
        const int width = next.widths[g];
        const int page = next.tables[g][(size_t)row * width + min(p / next.page_size, width - 1)];
        next.slots[g][row] = page < 0 ? -1 : page * next.page_size + p % next.page_size;
      }
    }
  }
}

// token_ids, positions, first_position int32 [n_rows]; for each of the n_groups (at most four) cache groups
// slots int32 [n_rows] and its block table int32 [n_rows, width].
extern "C" int ta_argmax_next_step(const void* logits, void* out, void* partial_v, void* partial_i, int n_rows,
                                   int vocab, int chunks, void* token_ids, void* positions, void* first_position,
                                   int page_size, int n_groups, void* slots0, const void* table0, int width0,
                                   void* slots1, const void* table1, int width1, void* slots2, const void* table2,
                                   int width2, void* slots3, const void* table3, int width3, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (chunks < 1 || vocab < 1 || page_size < 1 || n_groups < 0 || n_groups > NEXT_STEP_GROUPS) return -1;
  if (!logits || !out || !partial_v || !partial_i || !token_ids || !positions || !first_position) return -1;
  NextStep next = {};
  next.token_ids = (int*)token_ids; next.positions = (int*)positions; next.first_position = (int*)first_position;
  next.page_size = page_size; next.n_groups = n_groups;
  void* const slots[NEXT_STEP_GROUPS] = {slots0, slots1, slots2, slots3};
  const void* const tables[NEXT_STEP_GROUPS] = {table0, table1, table2, table3};
  const int widths[NEXT_STEP_GROUPS] = {width0, width1, width2, width3};
  for (int g = 0; g < n_groups; ++g) {
    if (!slots[g] || !tables[g] || widths[g] < 1) return -1;
    next.slots[g] = (int*)slots[g]; next.tables[g] = (const int*)tables[g]; next.widths[g] = widths[g];
  }
  dim3 grid(chunks, n_rows);
  argmax_pieces<<<grid, ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)partial_v, (int*)partial_i,
                                                    vocab, chunks);
  int status = LAUNCH_STATUS();
  if (status) return status;
  argmax_rows_next<<<n_rows, ARGMAX_THREADS, 0, stream>>>((const float*)partial_v, (const int*)partial_i, (int*)out,
                                                          chunks, next);
  return LAUNCH_STATUS();
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

// The same pick for callers that cannot allocate (see no_alloc.h): the pieces' maxima live in this array.  In
// host code its name is only a stand-in; the address kernels can use is looked up per device, once, below.
static __device__ __align__(256) unsigned char argmax_scratch[TA_ARGMAX_STATIC_PAIRS * (sizeof(float) + sizeof(int))];

#define TA_MAX_DEVICES 64
static void* g_argmax_scratch[TA_MAX_DEVICES];      // each GPU holds its own copy of the array at its own address
static std::mutex g_argmax_scratch_lock;

// The device address of `argmax_scratch` on the current device; 0 and a HIP error code in *status on failure.
static void* argmax_scratch_here(int* status) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) { *status = (int)err; return nullptr; }
  if (device < 0 || device >= TA_MAX_DEVICES) { *status = (int)hipErrorInvalidDevice; return nullptr; }
  std::lock_guard<std::mutex> hold(g_argmax_scratch_lock);
  if (!g_argmax_scratch[device]) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(argmax_scratch));
    if (err != hipSuccess || !found) { *status = err != hipSuccess ? (int)err : (int)hipErrorInvalidSymbol; return nullptr; }
    g_argmax_scratch[device] = found;
  }
  *status = 0;
  return g_argmax_scratch[device];
}

extern "C" int ta_argmax_static(const void* logits, void* out, int n_rows, int vocab, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab < 1) return -1;
  if (n_rows > TA_ARGMAX_STATIC_PAIRS) return TA_STATIC_TOO_LARGE;
  // Pieces per row as the allocating wrapper chooses them, within what the array holds.
  int chunks = vocab / 2048;
  if (chunks > 256) chunks = 256;
  if (chunks > TA_ARGMAX_STATIC_PAIRS / n_rows) chunks = TA_ARGMAX_STATIC_PAIRS / n_rows;
  if (chunks < 1) chunks = 1;
  int status = 0;
  unsigned char* scratch = (unsigned char*)argmax_scratch_here(&status);
  if (!scratch) return status;
  float* partial_v = (float*)scratch;
  int* partial_i = (int*)(scratch + TA_ARGMAX_STATIC_PAIRS * sizeof(float));
  return ta_argmax(logits, out, partial_v, partial_i, n_rows, vocab, chunks, stream);
}

// ------------------------------------------------------------------------------------------------
// Temperature / nucleus sampling without a sort.
//
// The reference orders the tokens by falling logit (lower index first among equals), keeps the shortest
// prefix whose probability reaches top_p, and walks that prefix with a uniform number until the mass is
// used up.  Both questions are "where does the running mass, in that order, cross a value": answered here
// by narrowing an order-preserving 32-bit key of the logit four bits at a time, each round summing the
// weights exp((l - max) / T) of the sixteen candidate ranges, and then counting indices among the tokens
// whose logit equals the crossing one.
//
// A row is cut into SAMPLE_PIECES slices with a workgroup each, and every round is a launch of its own: a
// round's workgroups first add up what the round before left for their row (in the fixed order of the slices,
// so the result does not change from run to run, and every workgroup of a row comes to the same decision),
// then sum their slice for the next round.  Some twenty small launches replace one workgroup walking a
// vocabulary of 150,000 twenty times on its own.
#define SAMPLE_THREADS 256
#define SAMPLE_PIECES 32

__device__ __forceinline__ uint32_t order_key(float v) {
  // Larger float -> larger key; NaN is treated as the smallest value.
  if (v != v) return 0u;
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// What a row keeps between launches (floats and ints of one array, SAMPLE_ROW_WORDS per row).
enum {
  SW_MAX = 0,                                   // [PIECES] maximum of each slice
  SW_MASS = SW_MAX + SAMPLE_PIECES,             // [PIECES] mass of each slice
  SW_PART = SW_MASS + SAMPLE_PIECES,            // [2][PIECES][16] masses of the sixteen ranges, by round parity
  SW_COUNT = SW_PART + 2 * SAMPLE_PIECES * 16,  // [PIECES] tokens with the picked key in each slice
  SW_STATE = SW_COUNT + SAMPLE_PIECES,          // [2][2] (prefix, above) by round parity
  SW_CUT = SW_STATE + 4,                        // cut_key, cut_rank, kept
  SW_PICK = SW_CUT + 4,                         // pick_key, pick_rank
  SAMPLE_ROW_WORDS = SW_PICK + 4
};

struct RowFacts {
  float max_logit, mass, inv_t;
  bool weighable;       // a finite maximum and a finite positive mass: else the greedy choice
};

// Block-wide sum in a fixed order; every thread gets it.  `scratch`: SAMPLE_THREADS / WAVE floats.
__device__ __forceinline__ float sample_block_sum(float v, float* scratch) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < SAMPLE_THREADS / WAVE; ++w) total += scratch[w];
  return total;
}

// What the launches before left for the row, fetched into LDS by the whole workgroup at once (one trip to
// memory instead of a chain of them): the slices' maxima and masses, and the range masses of one round
// (`parity`, or none for -1) added up over the slices in their order.
struct RowCopy {
  float max_of[SAMPLE_PIECES], mass_of[SAMPLE_PIECES];
  float part[SAMPLE_PIECES * 16];
  float total[16];
  float kept[SAMPLE_ROW_WORDS - SW_STATE];      // the settled state, the cut and the pick, as stored
};

__device__ __forceinline__ void fetch_row(const float* work, RowCopy& copy, int parity) {
  constexpr int PER_THREAD = SAMPLE_PIECES * 16 / SAMPLE_THREADS;
  static_assert(SAMPLE_PIECES * 16 % SAMPLE_THREADS == 0 && 2 * SAMPLE_PIECES <= SAMPLE_THREADS, "fetch_row's split");
  float held[PER_THREAD], summary = 0.f;
  if (threadIdx.x < 2 * SAMPLE_PIECES) summary = work[SW_MAX + threadIdx.x];          // maxima, then masses
  if (parity >= 0) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j)
      held[j] = work[SW_PART + parity * SAMPLE_PIECES * 16 + j * SAMPLE_THREADS + threadIdx.x];
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) copy.part[j * SAMPLE_THREADS + threadIdx.x] = held[j];
  }
  constexpr int KEPT = SAMPLE_ROW_WORDS - SW_STATE;
  static_assert(2 * SAMPLE_PIECES + KEPT <= SAMPLE_THREADS, "fetch_row's split");
  if (threadIdx.x >= 2 * SAMPLE_PIECES && threadIdx.x < 2 * SAMPLE_PIECES + KEPT)
    copy.kept[threadIdx.x - 2 * SAMPLE_PIECES] = work[SW_STATE + threadIdx.x - 2 * SAMPLE_PIECES];
  if (threadIdx.x < SAMPLE_PIECES) copy.max_of[threadIdx.x] = summary;
  else if (threadIdx.x < 2 * SAMPLE_PIECES) copy.mass_of[threadIdx.x - SAMPLE_PIECES] = summary;
  __syncthreads();
  if (parity >= 0) {
    if (threadIdx.x < 16) {
      float t = 0.f;
#pragma unroll
      for (int g = 0; g < SAMPLE_PIECES; ++g) t += copy.part[g * 16 + threadIdx.x];
      copy.total[threadIdx.x] = t;
    }
    __syncthreads();
  }
}

__device__ __forceinline__ RowFacts row_facts(const RowCopy& copy, float temperature, bool with_mass) {
  RowFacts f;
  f.inv_t = 1.0f / temperature;
  f.max_logit = -INFINITY;
  for (int g = 0; g < SAMPLE_PIECES; ++g) f.max_logit = fmaxf(f.max_logit, copy.max_of[g]);
  f.mass = 0.f;
  if (with_mass)
    for (int g = 0; g < SAMPLE_PIECES; ++g) f.mass += copy.mass_of[g];
  f.weighable = (f.max_logit > -INFINITY) && (f.max_logit < INFINITY) && (f.mass > 0.f) && (f.mass < INFINITY);
  return f;
}

__device__ __forceinline__ float weight_of(float v, const RowFacts& f) {
  return (v != v) ? 0.f : expf((v - f.max_logit) * f.inv_t);
}

// One round's decision: the masses of the sixteen ranges under `prefix` (`total`, summed over the slices in their
// order) are walked from the largest keys down until the running mass exceeds `target`.  If rounding leaves the
// target at or past the whole mass, the crossing is in the last range that holds anything.
__device__ __forceinline__ void walk_round(const float* total, float target, int shift, uint32_t& prefix, float& above) {
  float held[16];
#pragma unroll
  for (int n = 0; n < 16; ++n) held[n] = total[n];
  int pick = -1, last = 0;
  float run = above, run_at_last = above;
#pragma unroll
  for (int n = 15; n >= 0; --n) {
    if (pick < 0) {
      if (held[n] > 0.f) { last = n; run_at_last = run; }
      if (target < run + held[n]) pick = n;
      else run += held[n];
    }
  }
  if (pick < 0) { pick = last; run = run_at_last; }
  above = run;
  prefix |= (uint32_t)pick << shift;
}

// Where a crossing ended: the key, and how many tokens with that key (in index order) lie before the crossing one.
__device__ __forceinline__ int rank_at(uint32_t key, float above, float target, const RowFacts& f, float& each) {
  each = expf((key_value(key) - f.max_logit) * f.inv_t);
  const int rank = (each > 0.f) ? (int)floorf((target - above) / each) : 0;
  return max(rank, 0);
}

__device__ __forceinline__ void slice_of(int vocab, int& begin, int& end) {
  const int per = (vocab + SAMPLE_PIECES - 1) / SAMPLE_PIECES;
  begin = min(vocab, (int)blockIdx.x * per);
  end = min(vocab, begin + per);
}

// Calls use(value, index) for every token of the slice [begin, end), each thread taking every SAMPLE_THREADS-th
// one.  SAMPLE_BATCH loads are requested before the first is used: a slice is a few trips to memory, not one
// per token.
#define SAMPLE_BATCH 16
template <typename Use>
__device__ __forceinline__ void for_slice(const float* __restrict__ row, int begin, int end, Use use) {
  for (int base = begin + threadIdx.x; base < end; base += SAMPLE_BATCH * SAMPLE_THREADS) {
    float v[SAMPLE_BATCH];
#pragma unroll
    for (int j = 0; j < SAMPLE_BATCH; ++j) {
      const int i = base + j * SAMPLE_THREADS;
      v[j] = row[min(i, end - 1)];
    }
#pragma unroll
    for (int j = 0; j < SAMPLE_BATCH; ++j) {
      const int i = base + j * SAMPLE_THREADS;
      if (i < end) use(v[j], i);
    }
  }
}

// Launch 1: the maximum of every slice (fmaxf skips NaN).
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_max(const float* __restrict__ logits, float* __restrict__ workspace, int vocab) {
  __shared__ float scratch[SAMPLE_THREADS / WAVE];
  const float* row = logits + (size_t)blockIdx.y * vocab;
  float* work = workspace + (size_t)blockIdx.y * SAMPLE_ROW_WORDS;
  int begin, end;
  slice_of(vocab, begin, end);
  float mx = -INFINITY;
  for_slice(row, begin, end, [&](float v, int) { mx = fmaxf(mx, v); });
  mx = wave_max(mx);
  if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_THREADS / WAVE; ++w) mx = fmaxf(mx, scratch[w]);
    work[SW_MAX + blockIdx.x] = mx;
  }
}

// Launch 2: the mass of every slice under the row's maximum.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_mass(const float* __restrict__ logits, const float* __restrict__ temperature, float* __restrict__ workspace,
            int vocab) {
  __shared__ float scratch[SAMPLE_THREADS / WAVE];
  __shared__ RowCopy copy;
  const float* row = logits + (size_t)blockIdx.y * vocab;
  float* work = workspace + (size_t)blockIdx.y * SAMPLE_ROW_WORDS;
  fetch_row(work, copy, -1);
  const RowFacts f = row_facts(copy, temperature[blockIdx.y], false);
  int begin, end;
  slice_of(vocab, begin, end);
  float sum = 0.f;
  for_slice(row, begin, end, [&](float v, int) { sum += weight_of(v, f); });
  sum = sample_block_sum(sum, scratch);
  if (threadIdx.x == 0) work[SW_MASS + blockIdx.x] = sum;
}

// The crossing a round belongs to: the nucleus cut (the kept prefix ends where the mass reaches top_p * total;
// the reference stops at the first token with cumulative >= top_p, which is the crossing of a target just
// below top_p * mass in the "exceeds" sense) or the pick (the uniform number times the kept mass).
enum { CROSS_CUT = 0, CROSS_PICK = 1 };

// What the rounds before this one have settled for the row: every workgroup of the row works it out for itself
// (the same numbers in the same order give the same result); workgroup 0 stores it for the next launch.
// `round` 0..7 of crossing `cross`; a round's shift is 28 - 4 * round.  Returns the crossing's target.
__device__ float settle(float* work, const RowCopy& copy, const RowFacts& f, float top_p, float uniform, int cross,
                        int round, bool had_cut, uint32_t& prefix, float& above) {
  const bool writer = blockIdx.x == 0 && threadIdx.x == 0;
  float kept = f.mass;
  if (cross == CROSS_PICK && had_cut && top_p < 1.0f) {
    if (round == 0) {
      // The cut crossing's last round ended in the launch before: finish it.
      uint32_t cut_prefix = __float_as_uint(copy.kept[2 * 1 + 0]);     // state before round 7 (odd parity)
      float cut_above = copy.kept[2 * 1 + 1];
      const float cut_target = fmaxf(0.f, nextafterf(top_p * f.mass, 0.f));
      walk_round(copy.total, cut_target, 0, cut_prefix, cut_above);
      float each;
      const int rank = rank_at(cut_prefix, cut_above, cut_target, f, each);
      kept = cut_above + (float)(rank + 1) * each;
      if (writer) {
        work[SW_CUT + 0] = __uint_as_float(cut_prefix);
        work[SW_CUT + 1] = __int_as_float(rank);
        work[SW_CUT + 2] = kept;
      }
    } else {
      kept = copy.kept[SW_CUT - SW_STATE + 2];
    }
  }
  const float target = cross == CROSS_CUT ? fmaxf(0.f, nextafterf(top_p * f.mass, 0.f)) : uniform * kept;
  prefix = 0;
  above = 0.f;
  if (round > 0) {
    // State before round - 1 (stored under that round's parity), then that round's walk.
    const int before = (round - 1) & 1;
    if (round > 1) {
      prefix = __float_as_uint(copy.kept[2 * before + 0]);
      above = copy.kept[2 * before + 1];
    }
    walk_round(copy.total, target, 28 - 4 * (round - 1), prefix, above);
    if (writer) {
      work[SW_STATE + 2 * (round & 1) + 0] = __uint_as_float(prefix);
      work[SW_STATE + 2 * (round & 1) + 1] = above;
    }
  }
  return target;
}

// Launches 3..: one round of a crossing.  Sums the masses of the sixteen ranges under the settled prefix over
// this workgroup's slice.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_round(const float* __restrict__ logits, const float* __restrict__ temperature, const float* __restrict__ top_p,
             const float* __restrict__ uniform, float* __restrict__ workspace, int vocab, int cross, int round,
             int had_cut) {
  __shared__ float bins[16][SAMPLE_THREADS + 1];            // a row one longer: the reduction's reads spread over the banks
  __shared__ float segment[16][16];
  __shared__ RowCopy copy;
  const int r = blockIdx.y;
  const float* row = logits + (size_t)r * vocab;
  float* work = workspace + (size_t)r * SAMPLE_ROW_WORDS;
  // The round before this one left its range masses under its parity; the pick's first round finishes the cut.
  fetch_row(work, copy, round > 0 ? (round - 1) & 1 : (cross == CROSS_PICK && had_cut) ? 1 : -1);
  const RowFacts f = row_facts(copy, temperature[r], true);
  if (!f.weighable) return;                                 // the greedy choice, made at the end
  if (cross == CROSS_CUT && !(top_p[r] < 1.0f)) return;     // everything is kept
  uint32_t prefix;
  float above;
  settle(work, copy, f, top_p[r], uniform[r], cross, round, had_cut != 0, prefix, above);
  const int shift = 28 - 4 * round;
  const uint32_t mask = (round == 0) ? 0u : (0xffffffffu << (shift + 4));
#pragma unroll
  for (int n = 0; n < 16; ++n) bins[n][threadIdx.x] = 0.f;
  int begin, end;
  slice_of(vocab, begin, end);
  for_slice(row, begin, end, [&](float v, int) {
    const uint32_t key = order_key(v);
    if ((key & mask) == prefix) bins[(key >> shift) & 15u][threadIdx.x] += weight_of(v, f);   // a thread's own column
  });
  // Every range's sum over the workgroup, in a fixed order: thread (n, s) adds sixteen neighbouring threads' sums
  // of range n, then thread n adds the sixteen segments.
  __syncthreads();
  {
    static_assert(SAMPLE_THREADS == 256, "sixteen ranges times sixteen segments of sixteen threads");
    const int n = threadIdx.x & 15, seg = threadIdx.x >> 4;
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) t += bins[n][seg * 16 + k];
    segment[n][seg] = t;
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    float total = 0.f;
#pragma unroll
    for (int seg = 0; seg < 16; ++seg) total += segment[threadIdx.x][seg];
    work[SW_PART + (round & 1) * SAMPLE_PIECES * 16 + blockIdx.x * 16 + threadIdx.x] = total;
  }
}

// After the last round of the pick: the key and rank of the drawn token (held back to the end of the kept prefix),
// and how many tokens of each slice have that key.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_count(const float* __restrict__ logits, const float* __restrict__ temperature, const float* __restrict__ top_p,
             const float* __restrict__ uniform, float* __restrict__ workspace, int vocab, int had_cut) {
  __shared__ float scratch[SAMPLE_THREADS / WAVE];
  __shared__ RowCopy copy;
  const int r = blockIdx.y;
  const float* row = logits + (size_t)r * vocab;
  float* work = workspace + (size_t)r * SAMPLE_ROW_WORDS;
  fetch_row(work, copy, 1);                                 // the pick's last round
  const RowFacts f = row_facts(copy, temperature[r], true);
  uint32_t pick_key;
  int pick_rank = 0;
  if (!f.weighable) {
    pick_key = order_key(f.max_logit);        // nothing to weigh (all -inf or NaN, or an infinite logit): first maximum
  } else {
    const bool cut = had_cut && top_p[r] < 1.0f;
    const float kept = cut ? copy.kept[SW_CUT - SW_STATE + 2] : f.mass;
    const float target = uniform[r] * kept;
    uint32_t prefix = __float_as_uint(copy.kept[2 * 1 + 0]);     // state before round 7
    float above = copy.kept[2 * 1 + 1];
    walk_round(copy.total, target, 0, prefix, above);
    float each;
    pick_rank = rank_at(prefix, above, target, f, each);
    pick_key = prefix;
    if (cut) {
      const uint32_t cut_key = __float_as_uint(copy.kept[SW_CUT - SW_STATE + 0]);
      const int cut_rank = __float_as_int(copy.kept[SW_CUT - SW_STATE + 1]);
      if (pick_key < cut_key || (pick_key == cut_key && pick_rank > cut_rank)) {   // past the kept prefix: its last token
        pick_key = cut_key;
        pick_rank = cut_rank;
      }
    }
  }
  int begin, end;
  slice_of(vocab, begin, end);
  float mine = 0.f;                                          // counts stay exact in float (a slice is far below 2^24)
  for_slice(row, begin, end, [&](float v, int) { mine += (order_key(v) == pick_key) ? 1.f : 0.f; });
  mine = sample_block_sum(mine, scratch);
  if (threadIdx.x == 0) {
    work[SW_COUNT + blockIdx.x] = mine;
    if (blockIdx.x == 0) {
      work[SW_PICK + 0] = __uint_as_float(pick_key);
      work[SW_PICK + 1] = __int_as_float(pick_rank);
    }
  }
}

// Last launch: the pick_rank-th lowest index among the tokens whose key is pick_key (the last of them if there
// are fewer); the workgroup whose slice holds it writes it.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_locate(const float* __restrict__ logits, const float* __restrict__ workspace, int* __restrict__ out, int vocab) {
  __shared__ int wave_count[SAMPLE_THREADS / WAVE];
  const int r = blockIdx.y;
  const float* row = logits + (size_t)r * vocab;
  const float* work = workspace + (size_t)r * SAMPLE_ROW_WORDS;
  const uint32_t pick_key = __float_as_uint(work[SW_PICK + 0]);
  const int pick_rank = __float_as_int(work[SW_PICK + 1]);
  __shared__ int count_of[SAMPLE_PIECES];
  if (threadIdx.x < SAMPLE_PIECES) count_of[threadIdx.x] = (int)work[SW_COUNT + threadIdx.x];
  __syncthreads();
  int all = 0, before = 0;
  for (int g = 0; g < SAMPLE_PIECES; ++g) {
    if (g < (int)blockIdx.x) before += count_of[g];
    all += count_of[g];
  }
  const int here = count_of[blockIdx.x];
  if (all == 0) {                                           // no token has the key (cannot be, but never leave out[r] unset)
    if (blockIdx.x == 0 && threadIdx.x == 0) out[r] = 0;
    return;
  }
  const int want = min(pick_rank, all - 1);
  if (want < before || want >= before + here) return;      // another slice's
  int left = want - before;                                 // matches of this slice to pass over
  int begin, end;
  slice_of(vocab, begin, end);
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  for (int batch = begin; batch < end; batch += SAMPLE_BATCH * SAMPLE_THREADS) {
    float v[SAMPLE_BATCH];
#pragma unroll
    for (int j = 0; j < SAMPLE_BATCH; ++j) v[j] = row[min(batch + j * SAMPLE_THREADS + (int)threadIdx.x, end - 1)];
#pragma unroll 1
    for (int j = 0; j < SAMPLE_BATCH; ++j) {                 // 256 consecutive tokens at a time, in order
      const int base = batch + j * SAMPLE_THREADS;
      if (base >= end) return;
      const int i = base + threadIdx.x;
      float mine = v[0];
#pragma unroll
      for (int q = 1; q < SAMPLE_BATCH; ++q) mine = (q == j) ? v[q] : mine;     // registers have no index
      const bool match = i < end && order_key(mine) == pick_key;
      const unsigned long long votes = __ballot(match);
      __syncthreads();
      if (lane == 0) wave_count[wave] = __popcll(votes);
      __syncthreads();
      int in_block = 0, before_wave = 0;
      for (int w = 0; w < SAMPLE_THREADS / WAVE; ++w) {
        if (w < wave) before_wave += wave_count[w];
        in_block += wave_count[w];
      }
      if (left < in_block) {
        const int my_place = before_wave + __popcll(votes & ((1ull << lane) - 1ull));
        if (match && my_place == left) out[r] = i;
        return;
      }
      left -= in_block;
    }
  }
}

// Floats of workspace a row needs.
extern "C" int ta_sample_workspace_words() { return SAMPLE_ROW_WORDS; }

// workspace: n_rows * ta_sample_workspace_words() floats.  any_cut: 0 if no row has top_p < 1 (the rounds of the
// nucleus cut are then left out).
extern "C" int ta_sample(const void* logits, const void* temperature, const void* top_p, const void* uniform,
                         void* out, void* workspace, int n_rows, int vocab, int any_cut, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab < 1 || !workspace) return -1;
  const dim3 grid(SAMPLE_PIECES, n_rows);
  const float* lg = (const float*)logits;
  const float *t = (const float*)temperature, *p = (const float*)top_p, *u = (const float*)uniform;
  float* work = (float*)workspace;
  sample_max<<<grid, SAMPLE_THREADS, 0, stream>>>(lg, work, vocab);
  sample_mass<<<grid, SAMPLE_THREADS, 0, stream>>>(lg, t, work, vocab);
  for (int cross = any_cut ? CROSS_CUT : CROSS_PICK; cross <= CROSS_PICK; ++cross)
    for (int round = 0; round < 8; ++round)
      sample_round<<<grid, SAMPLE_THREADS, 0, stream>>>(lg, t, p, u, work, vocab, cross, round, any_cut);
  sample_count<<<grid, SAMPLE_THREADS, 0, stream>>>(lg, t, p, u, work, vocab, any_cut);
  sample_locate<<<grid, SAMPLE_THREADS, 0, stream>>>(lg, work, (int*)out, vocab);
  return LAUNCH_STATUS();
}
