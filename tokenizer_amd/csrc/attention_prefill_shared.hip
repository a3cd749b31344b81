// Prompt attention whose waves share their keys: the workgroup of a tile of 16 tokens and one kv head holds four
// waves, each with HG (1 or 2) of the query heads that share the kv head, and all of them walk the same blocks of
// 64 keys.  A block's keys and values come from the pages once for the whole workgroup, by loads that write
// straight into LDS (no register on the way), two buffers deep: the next block is on its way while the matrix
// cores work on the current one, and every wave takes its fragments from LDS.  With KG = 2 a second group of
// four waves with the same heads takes every other block, and the groups merge their softmax states at the end.
// Against the kernel in attention_prefill.hip (each wave fetches its own blocks for its own two heads) a key is
// read from the cache half or a quarter as often, and no wave waits for memory with nothing else to do; which
// of the two kernels, and which shape of this one, a launch gets is `ta_prefill_attention_shared_plan`'s
// choice.  Same fragment layouts and key order as there: S^T = K Q^T and O^T = V^T P^T with 16x16x32 MFMAs,
// token index in `lane % 16`, softmax online in float, probabilities rounded to bfloat16 for the second product
// (whose row block of ones also yields their sums).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define SHARED_WAVES 4       // waves of a workgroup: each brings one of a block's four runs of sixteen keys

// A block in LDS.  A load that writes into LDS puts lane i's sixteen bytes at its base + 16 i, so what one
// instruction brings is one KB on end, and where a piece lands is decided by which lane asks for it.
// Keys: 64 rows of D / 8 pieces, no padding; the piece that holds elements 8 p .. 8 p + 7 of key k stands at
// place p ^ swizzle(k), so that the eight rows which neighbouring lanes read at once lie in different banks.
// Values: run by run, D rows of the run's sixteen keys (32 bytes), which neighbouring lanes read 32 bytes apart.
// attention_decode.hip: the parts of a tile's keys, merged into the output rows of the tile's tokens.
extern "C" int ta_attention_merge_tiles(const void* part_o, const void* part_ml, const void* tiles, int n_tiles,
                                        const void* cu_q, void* out, int n_q, int d, int splits, hipStream_t stream);

template <int D>
struct Staged {
  static_assert(D == 64 || D == 128, "a key row must be a power of two of pieces for the swizzle");
  static constexpr int PIECES = D / 8;                      // 16-byte pieces of a key row
  static constexpr int K_ROW = 2 * D;
  static constexpr int K_BYTES = 64 * K_ROW;
  static constexpr int V_RUN = 32 * D;
  static constexpr int BYTES = K_BYTES + 4 * V_RUN;
  static constexpr int KEYS_A_LOAD = 64 / PIECES;           // key rows that one instruction of a wave brings
  static constexpr int K_LOADS = 16 / KEYS_A_LOAD;          // instructions for a run's keys
  static constexpr int V_LOADS = D / 32;                    // and for its values (32 rows of D each)
  // Keys k, k + 1, k + 2, k + 3 and k + 8 .. k + 11 (k a multiple of 4) are read at once.
  __device__ static constexpr int swizzle(int key) { return (key & 3) | ((key >> 1) & 4); }
};

__device__ __forceinline__ float max2(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float max16(const float (&v)[16]) {
  const float a = max2(max2(v[0], v[1]), v[2]), b = max2(max2(v[3], v[4]), v[5]), c = max2(max2(v[6], v[7]), v[8]);
  const float d = max2(max2(v[9], v[10]), v[11]), e = max2(max2(v[12], v[13]), v[14]);
  return max2(max2(max2(a, b), c), max2(max2(d, e), v[15]));
}

__device__ __forceinline__ bf16x8 sh_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

struct SharedTile {
  const bf16_t* k_pages;
  const bf16_t* vt_pages;
  const int* table;
  int kvh, n_kv, page_size;
  int lo, hi;                 // first and last key that any token of the tile sees
  int lo_page, hi_page;       // their places in the block table
};

// What a wave brings of every block: one of its four runs of sixteen keys (a run lies inside one page), so
// that per block a wave looks up one page number and every load is a scalar base plus an offset that the lane
// worked out once.
template <int D>
struct Carrier {
  typedef Staged<D> S;
  int run;                                                  // which of a block's runs
  uint32_t k_from[S::K_LOADS];                              // byte offsets of the lane's pieces inside the run's part of its page
  uint32_t v_from;
  int at_page, at_slot;                                     // where the run of the next block to look up lies: index into the block table, slot in the page
  int step_pages, step_slots;                               // from one of the wave's blocks to the next
  int page, slot;                                           // of the run of the block to fetch next
  int page_size;
  uint32_t page_elements, first_element;                    // elements of a page (all kv heads); where this kv head's begin

  // run: which of a block's runs; first_key: the first key of the wave's first block; stride: keys from one of
  // its blocks to the next (a multiple of 64).
  __device__ __forceinline__ void plan(int which_run, int lane, const SharedTile& tile, int first_key, int stride) {
    run = which_run;
    page_size = tile.page_size;
    page_elements = (uint32_t)tile.n_kv * page_size * D;
    first_element = (uint32_t)tile.kvh * page_size * D;
    at_page = (first_key + 16 * run) / page_size;
    at_slot = (first_key + 16 * run) % page_size;
    step_pages = stride / page_size;
    step_slots = stride % page_size;
#pragma unroll
    for (int j = 0; j < S::K_LOADS; ++j) {
      const int key = S::KEYS_A_LOAD * j + lane / S::PIECES;             // within the run; the run starts at a multiple of 16
      const int part = (lane % S::PIECES) ^ S::swizzle(key);            // the piece that belongs at this lane's place
      k_from[j] = (uint32_t)(key * D + part * 8) * 2;
    }
    v_from = (uint32_t)((lane >> 1) * page_size + (lane & 1) * 8) * 2;
  }

  // Where the wave's run of block `kb` lies, looked up a turn before the block is fetched, so that no wave waits
  // for a page number.  Blocks are looked up in order.  `full`: every key of the block exists and is seen by
  // every token.  Otherwise a run without a key of lo..hi (before `lo`: its page may have been given back; after
  // `hi`: it may not exist yet) borrows the page of `lo` or `hi`, a valid address; what lies there never counts
  // (scores outside a token's range are masked by selection, values outside lo..hi are set to zero when read).
  __device__ __forceinline__ void look_up(const SharedTile& tile, int kb, bool full) {
    int index = at_page;
    if (!full) {
      const int key = kb + 16 * run;
      if (key + 15 < tile.lo) index = tile.lo_page;
      if (key > tile.hi) index = tile.hi_page;
    }
    page = scalar_int(tile.table + index);
    slot = at_slot;
    at_page += step_pages;
    at_slot += step_slots;
    if (at_slot >= page_size) {
      at_slot -= page_size;
      ++at_page;
    }
  }

  // The run that was looked up last, from its page straight into `buf`.  The loads are under way when this
  // returns; `landed` waits for them.
  __device__ __forceinline__ void fetch(const SharedTile& tile, char* buf) const {
    typedef const void __attribute__((address_space(1)))* from_t;
    typedef void __attribute__((address_space(3)))* to_t;
    const uint32_t head = (uint32_t)page * page_elements + first_element;
    const char* k_run = reinterpret_cast<const char*>(tile.k_pages + (head + (uint32_t)slot * D));
    const char* v_run = reinterpret_cast<const char*>(tile.vt_pages + (head + (uint32_t)slot));
    char* k_to = buf + run * 16 * S::K_ROW;
    char* v_to = buf + S::K_BYTES + run * S::V_RUN;
#pragma unroll
    for (int j = 0; j < S::K_LOADS; ++j)
      __builtin_amdgcn_global_load_lds((from_t)(k_run + k_from[j]), (to_t)(k_to + j * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < S::V_LOADS; ++j)
      __builtin_amdgcn_global_load_lds((from_t)(v_run + v_from + (uint32_t)j * 64 * page_size), (to_t)(v_to + j * 1024), 16, 0, 0);
  }

  // All that this wave fetched has arrived in LDS (vmcnt 0; the other counters stay as they are).
  __device__ __forceinline__ static void landed() { __builtin_amdgcn_s_waitcnt(0x0F70); }
};

// O^T += V^T P^T for one head over the block in `buf`, and the probabilities' sum by the same means: one more
// row block of V^T that holds ones gives every lane its token's sum over all 64 keys (of the rounded
// probabilities, the very weights of the product), where sixteen additions a head and two exchanges between
// lanes at the end stood.
template <int D, bool FULL>
__device__ __forceinline__ void second_product(const char* buf, int kb, int col, int g, int lo, int hi,
                                               const bf16x8 (&pf)[2], floatx4 (&acc)[D / 16], floatx4& l) {
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    l = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[u], l, 0, 0, 0);
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      bf16x8 vf = *reinterpret_cast<const bf16x8*>(buf + Staged<D>::K_BYTES + (2 * u + (g >> 1)) * Staged<D>::V_RUN +
                                                   (db * 16 + col) * 32 + (g & 1) * 16);
      if (!FULL) {
        // A probability of zero times whatever lies in a slot that was never written, or in a borrowed page,
        // must stay zero.
        const int first = kb + 32 * u + 8 * g;             // the lane's keys: first .. first + 7
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (first + i > hi || first + i < lo) vf[i] = (__bf16)0.0f;
      }
      acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], acc[db], 0, 0, 0);
    }
  }
}

// One step of the online softmax of a wave's HG heads over the block of 64 keys in `buf`.  Row r of the first
// product's instruction t of a half of 32 keys is key 8 (r / 4) + 4 t + r % 4 of the half, whose score then lies
// in the lane group that holds that key in the second product (lane group g: keys 8g .. 8g+7).
// lo, hi: the first and last key that any token of the tile sees (unless FULL, values outside them may be anything).
template <int D, int HG, bool FULL>
__device__ __forceinline__ void shared_block(const char* buf, int kb, int col, int g, int my_pos, int my_lo, int lo, int hi,
                                             float c, const bf16x8 (&qf)[HG][D / 32], floatx4 (&acc)[HG][D / 16],
                                             float (&m)[HG], floatx4 (&l)[HG]) {
  constexpr int KS = D / 32;
  constexpr int DB = D / 16;
  float s[HG][16];
  const int turned = (col & 3) | ((col >> 2) & 1) << 2;    // swizzle of the lane's keys: the same in every instruction
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int key = 32 * (t >> 1) + 8 * (col >> 2) + 4 * (t & 1) + (col & 3);
    bf16x8 kf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      kf[ks] = *reinterpret_cast<const bf16x8*>(buf + key * Staged<D>::K_ROW + ((ks * 4 + g) ^ turned) * 16);
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      floatx4 st = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[h][ks], st, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (FULL) {
          s[h][t * 4 + r] = st[r];
        } else {
          const int at = kb + 32 * (t >> 1) + 8 * g + 4 * (t & 1) + r;
          s[h][t * 4 + r] = (at <= my_pos && at >= my_lo) ? st[r] : -INFINITY;
        }
      }
    }
  }
  bf16x8 pf[HG][2];
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    const float (&sh)[16] = s[h];
    // The IEEE maximum (a NaN would spread, but masked scores are -inf and the others products of stored numbers)
    // rather than fmaxf: the compiler joins it into v_maximum3_f32, eight instructions for sixteen scores, where
    // fmaxf first rewrites every score that might be a signalling NaN.  (Not inline assembly: the scores come
    // straight from matrix instructions, whose results a vector instruction may only read after wait states that
    // the compiler counts for the instructions it knows; a v_max3_f32 written in assembly read them too early.)
    float mx = max16(sh);
    mx = max2(mx, __shfl_xor(mx, 16, WAVE));
    mx = max2(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = max2(m[h], mx);
    // A token that has seen no key yet keeps m = -inf; exp2 of (-inf) - (-inf) would be NaN.
    const float mc = (m_new == -INFINITY) ? 0.f : m_new * c;
    if (__any(m_new > m[h])) {                          // rescale only when some token's maximum moved
      const float corr = __builtin_amdgcn_exp2f(m[h] * c - mc);   // m = -inf gives 0
#pragma unroll
      for (int r = 0; r < 4; ++r) l[h][r] *= corr;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][db][r] *= corr;
      m[h] = m_new;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
      pf[h][i >> 3][i & 7] = (__bf16)__builtin_amdgcn_exp2f(fmaf(sh[i], c, -mc));   // masked keys: exp2(-inf) = 0
    // The head's second product follows at once, so that the matrix cores work on it while the vector unit
    // works on the next head's probabilities (the values are read from LDS once per head for that).
    second_product<D, FULL>(buf, kb, col, g, lo, hi, pf[h], acc[h], l[h]);
  }
}

// Arguments as in prefill_attention_kernel.  Dynamic LDS: two blocks for each of the KG groups of four waves
// (2 * KG * Staged<D>::BYTES).
// KG = 2: two groups of four waves, each with the same heads, take the blocks in turn (group i the blocks i,
// i + 2, ...) and merge their softmax states through LDS at the end: half as many turns for a long walk, for
// launches that cannot fill the device with workgroups.
template <int D, int HG, int KG>
__global__ void __launch_bounds__(SHARED_WAVES * KG * WAVE, 1)
prefill_attention_shared_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                                const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages,
                                const int* __restrict__ tiles, int n_tiles, const int* __restrict__ cu_q,
                                const int* __restrict__ first_position, const int* __restrict__ block_table,
                                int table_stride, int n_q, int n_kv, int page_size, int window, float scale_log2,
                                int key_splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int KS = D / 32;
  constexpr int DB = D / 16;
  constexpr int NW = SHARED_WAVES;
  constexpr int STRIDE = 64 * KG;                          // keys a turn of the whole workgroup covers
  HELD(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, first_position, block_table, table_stride, n_q, n_kv,
       page_size, window, scale_log2, key_splits, part_o, part_ml);
  extern __shared__ __attribute__((aligned(16))) char staged[];
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int head_wave = wave % NW, key_group = wave / NW;
  const int col = lane & 15, g = lane >> 4;
  const int group = n_q / n_kv;
  const int head_blocks = (group + HG * NW - 1) / (HG * NW);
  // Late tiles first, as in the other prompt kernel: they see the most keys.
  const int per_tile = n_kv * head_blocks;
  const int split = blockIdx.x % key_splits;               // which part of the tile's keys (of key_splits)
  const int block = blockIdx.x / key_splits;
  const int which = block % per_tile;
  const int kvh = which / head_blocks, hb = which % head_blocks;
  const int first_head = hb * HG * NW + head_wave * HG;       // among the heads of the kv head
  const int heads_here = max(0, min(HG, group - first_head));  // a wave past the last head only brings blocks
  const int head0 = kvh * group + first_head;
  const int tile_index = n_tiles - 1 - block / per_tile;
  // (Through the scalar unit, the three that hang on the entry asked for together: see scalar_int.)
  const int entry = scalar_int(tiles + 2 * tile_index);
  const int offset = scalar_int(tiles + 2 * tile_index + 1);
  const int entry_row = scalar_int(cu_q + entry), next_row = scalar_int(cu_q + entry + 1);
  const int entry_position = scalar_int(first_position + entry);
  HELD(entry_row, next_row, entry_position);
  const int row0 = entry_row + offset;
  const int n_valid = min(16, next_row - row0);
  if (n_valid <= 0) return;                                // a tile that only fills the list up (its entry has no rows)
  const int p0 = entry_position + offset;                  // position of the tile's first token
  const int my_pos = p0 + min(col, n_valid - 1);          // padded columns repeat the last token
  const int my_row = row0 + min(col, n_valid - 1);
  const int hi = p0 + n_valid - 1;                         // last key any token of the tile sees
  const int lo = (window >= 0 && p0 > window) ? p0 - window : 0;      // first key any token sees
  const int lo_all = (window >= 0 && hi > window) ? hi - window : 0;  // first key every token sees
  const int my_lo = (window >= 0 && my_pos > window) ? my_pos - window : 0;
  SharedTile tile;
  tile.k_pages = k_pages;
  tile.vt_pages = vt_pages;
  tile.table = block_table + (size_t)entry * table_stride;
  tile.kvh = kvh;
  tile.n_kv = n_kv;
  tile.page_size = page_size;
  tile.lo = lo;
  tile.hi = hi;
  tile.lo_page = lo / page_size;
  tile.hi_page = hi / page_size;

  bf16x8 qf[HG][KS];
#pragma unroll
  for (int h = 0; h < HG; ++h)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[h][ks] = sh_zero8();
      if (h < heads_here)
        qf[h][ks] = *reinterpret_cast<const bf16x8*>(q + (size_t)my_row * q_stride + (size_t)(head0 + h) * D + ks * 32 + 8 * g);
    }
  floatx4 acc[HG][DB], l[HG];                              // l: the sum of a token's probabilities, four times over
  float m[HG];
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    m[h] = -INFINITY;
    l[h] = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[h][db] = (floatx4){0.f, 0.f, 0.f, 0.f};
  }

  // A turn of the workgroup covers KG blocks, one for each group of waves.  Turns come in three runs (the
  // window's edge, those whose blocks every token sees whole, the diagonal), each a loop of its own over one
  // variant of the block, so that the accumulators stay in the same registers within a loop.  In a turn a wave
  // asks for its group's next block into the buffer that the turn before read, works on the current one, waits
  // for what it asked for, and meets the other waves: after the barrier every wave's part of the next blocks has
  // landed, and nobody reads the current ones any more.  A group whose block of a turn lies past the last key
  // leaves it out.
  // With the keys cut over workgroups (key_splits > 1: few tiles behind a long context), this one takes a run of
  // whole turns of the tile's walk, `kb` .. `end`; a workgroup past the last turn walks nothing and hands on an
  // empty state.
  const int first_turn = (lo / 64) * 64;
  const int turns_each = ((hi - first_turn) / STRIDE + key_splits) / key_splits;
  int kb = first_turn + split * turns_each * STRIDE;       // the turn's first key
  const int end = min(hi, kb + turns_each * STRIDE - 1);   // the last key of this workgroup's turns
  int cur = 0;
  char* buffers = staged + key_group * 2 * Staged<D>::BYTES;
  const int ahead = 64 * key_group;                        // the group's block within a turn
  Carrier<D> carrier;
  carrier.plan(head_wave, lane, tile, kb + ahead, STRIDE);
  const auto whole = [&](int turn) { return turn >= lo_all && turn + STRIDE - 1 <= p0; };
  carrier.look_up(tile, kb + ahead, whole(kb));
  if (kb + ahead <= end) carrier.fetch(tile, buffers);
  if (kb + STRIDE + ahead <= end) carrier.look_up(tile, kb + STRIDE + ahead, whole(kb + STRIDE));
  carrier.landed();
  __syncthreads();
#define TURN(FULL)                                                                                            \
  {                                                                                                           \
    const int next = kb + STRIDE;                                                                             \
    if (next + ahead <= end) carrier.fetch(tile, buffers + (cur ^ 1) * Staged<D>::BYTES);                     \
    if (next + STRIDE + ahead <= end) carrier.look_up(tile, next + STRIDE + ahead, whole(next + STRIDE));     \
    if (heads_here > 0 && (FULL || kb + ahead <= end))                                                        \
      shared_block<D, HG, FULL>(buffers + cur * Staged<D>::BYTES, kb + ahead, col, g, my_pos, my_lo, lo, hi,  \
                                scale_log2, qf, acc, m, l);                                                   \
    carrier.landed();                                                                                         \
    __syncthreads();                                                                                          \
    cur ^= 1;                                                                                                 \
  }
  for (; kb <= end && kb < lo_all; kb += STRIDE) TURN(false)
  for (; kb <= end && kb + STRIDE - 1 <= p0; kb += STRIDE) TURN(true)
  for (; kb <= end; kb += STRIDE) TURN(false)
#undef TURN

  if (KG > 1) {
    // The later groups hand their state to the first (the last turn ended with a barrier: the buffers are free):
    // maximum, sum and the output accumulators of each head.
    float* handed = reinterpret_cast<float*>(staged);      // [KG - 1][NW][HG][DB * 4 + 2][WAVE]
    const auto at = [&](int from_group, int h, int item) {
      return handed + ((((from_group - 1) * NW + head_wave) * HG + h) * (DB * 4 + 2) + item) * WAVE + lane;
    };
    if (key_group > 0) {
#pragma unroll
      for (int h = 0; h < HG; ++h) {
        *at(key_group, h, DB * 4) = m[h];
        *at(key_group, h, DB * 4 + 1) = l[h][0];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) *at(key_group, h, db * 4 + r) = acc[h][db][r];
      }
    }
    __syncthreads();
    if (key_group > 0) return;
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      float m_all = m[h];
#pragma unroll
      for (int k = 1; k < KG; ++k) m_all = fmaxf(m_all, *at(k, h, DB * 4));
      const float mc = (m_all == -INFINITY) ? 0.f : m_all * scale_log2;
      const float f0 = __builtin_amdgcn_exp2f(m[h] * scale_log2 - mc);       // a group without keys: exp2(-inf) = 0
      l[h][0] *= f0;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][db][r] *= f0;
#pragma unroll
      for (int k = 1; k < KG; ++k) {
        const float f = __builtin_amdgcn_exp2f(*at(k, h, DB * 4) * scale_log2 - mc);
        l[h][0] += f * *at(k, h, DB * 4 + 1);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[h][db][r] += f * *at(k, h, db * 4 + r);
      }
      m[h] = m_all;                                        // what the sums now stand under (a part hands it on)
    }
  }
  if (key_splits > 1) {
    // This workgroup's part of the keys: the state goes out as it is, item (tile, token) x head x part, for the
    // kernel that merges the parts (maximum in natural units of the scaled scores, sum, unnormalised output).
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      if (h >= heads_here) break;
      if (col >= n_valid) continue;
      const size_t at = (((size_t)tile_index * 16 + col) * n_q + head0 + h) * key_splits + split;
      if (g == 0) {
        part_ml[2 * at] = (m[h] == -INFINITY) ? -INFINITY : m[h] * scale_log2 * 0.6931471805599453f;
        part_ml[2 * at + 1] = l[h][0];
      }
#pragma unroll
      for (int db = 0; db < DB; ++db)
        *reinterpret_cast<float4*>(part_o + at * D + db * 16 + 4 * g) =
            make_float4(acc[h][db][0], acc[h][db][1], acc[h][db][2], acc[h][db][3]);
    }
    return;
  }
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    if (h >= heads_here) break;
    if (col >= n_valid) continue;
    const float inv = 1.0f / l[h][0];
    bf16_t* dst = out + (size_t)my_row * n_q * D + (size_t)(head0 + h) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      union { bf16x4 v; uint2 bits; } packed;
#pragma unroll
      for (int r = 0; r < 4; ++r) packed.v[r] = (__bf16)(acc[h][db][r] * inv);
      *reinterpret_cast<uint2*>(dst + db * 16 + 4 * g) = packed.bits;
    }
  }
}

template <int D, int HG, int KG>
static int launch_shared(const void* q, int q_stride, void* out, const void* k_pages, const void* vt_pages,
                         const void* tiles, int n_tiles, const void* cu_q, const void* first_position,
                         const void* block_table, int table_stride, int n_q, int n_kv, int page_size, int window,
                         float scale, int key_splits, void* part_o, void* part_ml, hipStream_t stream) {
  const int group = n_q / n_kv;
  const long workgroups = (long)n_tiles * n_kv * ((group + HG * SHARED_WAVES - 1) / (HG * SHARED_WAVES)) * key_splits;
  if (workgroups > 0x7fffffffL) return -1;
  constexpr int lds = 2 * KG * Staged<D>::BYTES;
  static_assert(lds <= 160 * 1024, "the blocks must fit a compute unit's LDS");
  static_assert((KG - 1) * SHARED_WAVES * HG * (D / 4 + 2) * WAVE * 4 <= lds, "the groups' states are handed over in the blocks' place");
  if (lds > 48 * 1024) {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attention_shared_kernel<D, HG, KG>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (err != hipSuccess) return (int)err;
  }
  prefill_attention_shared_kernel<D, HG, KG><<<(unsigned)workgroups, SHARED_WAVES * KG * WAVE, lds, stream>>>(
      (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)vt_pages, (const int*)tiles,
      n_tiles, (const int*)cu_q, (const int*)first_position, (const int*)block_table, table_stride, n_q, n_kv, page_size,
      window, scale * 1.4426950408889634f, key_splits, (float*)part_o, (float*)part_ml);
  int status = LAUNCH_STATUS();
  if (status == 0 && key_splits > 1)
    status = ta_attention_merge_tiles(part_o, part_ml, tiles, n_tiles, cu_q, out, n_q, D, key_splits, stream);
  return status;
}

// Into how many parts the keys of a tile are cut over workgroups when the kernel runs in `shape`: one, unless the
// launch has fewer workgroups than the device has compute units and the tokens look back over sixteen turns or
// more.  Then a workgroup walks its keys while most of the device idles, and parts of at least eight turns each,
// up to sixteen of them, fill it (28 / 4 heads of 128 behind 8,192 cached tokens, uncut | cut: 256 tokens 117 | 78
// us, 128 tokens 110 | 45, 16 tokens 109 | 25; 12 / 2 heads: 512 tokens 122 | 79, 128 tokens 114 | 29).
extern "C" int ta_prefill_attention_shared_key_splits(int n_tiles, int n_q, int n_kv, int reach, int shape) {
  if (shape <= 0 || n_kv <= 0) return 1;
  const int heads = shape % 10, key_groups = shape / 10 + 1;
  const int group = n_q / n_kv;
  const long workgroups = (long)n_tiles * n_kv * ((group + heads * SHARED_WAVES - 1) / (heads * SHARED_WAVES));
  const long units = compute_units();
  if (workgroups >= units || workgroups <= 0) return 1;
  const int turns = reach / (64 * key_groups);
  long parts = (units + workgroups - 1) / workgroups;
  if (parts > turns / 8) parts = turns / 8;
  if (parts > 16) parts = 16;
  return parts < 1 ? 1 : (int)parts;
}

// Whether the workgroup-shared kernel is the faster one, and in which shape: 0 = no, else heads a wave (1 or 2)
// + 10 if two key groups share a workgroup.  Five to eight query heads per kv head (or more) fill its four waves
// at two heads a wave, three or four at one.  A workgroup walks all its keys alone, so the launch must fill the device some other way:
// with 1,024 workgroups and more, two heads a wave; below that two key groups halve the walk, and one head a
// wave doubles the workgroups (each reading its blocks for half the heads); below 128 workgroups the per-wave
// kernel, whose waves split the keys of a tile, is the faster one.
// reach: how far back the farthest-seeing token looks, as the launcher plans it.
// (Measured on 256 compute units against the per-wave kernel, times in us as per-wave | 1 head | 2 heads |
// 1 head, 2 groups | 2 heads, 2 groups.  14 / 2 heads of 64: 1,024 tokens 14.3 | 17.4 | 23.6 | 13.6 | 18.6;
// 2,048 tokens 31.5 | 31.1 | 42.1 | 24.9 | 31.6; 4,096 tokens 87 | 63 | 80 | 62 | 63; 8,192 tokens 298 | 201 |
// 179 | 206 | 215; 2,048 tokens after 8,192 cached ones 174 | 138 | 178 | 121 | 126; 512 after 8,192: 59 | 100 | 151
// | 69 | 105.  28 / 4 heads of 128: 512 tokens 18.5 | 16.4 | 20.0 | 14.0 | 18.3; 2,048 tokens 103 | 66 | 66 | 79 |
// 58; 8,192 tokens 1,199 | 750 | 561 | 899 | 643; 2,048 after 8,192: 656 | 418 | 321 | 481 | 339.  12 / 2 heads of
// 128: 2,048 tokens 44.4 | 48.3 | 56.0 | 40.5 | 44.1; 2,048 after 8,192: 316 | 221 | 250 | 256 | 184.)
extern "C" int ta_prefill_attention_shared_plan(int n_tiles, int n_q, int n_kv, int d, int reach) {
  if (d != 64 && d != 128) return 0;
  const int group = n_q / n_kv;
  if (group < 3) return 0;
  // A short portion behind a cached context at head size 128: however few the workgroups, the per-wave kernel's
  // waves (two a tile there) each walk their keys with nothing to hide a block's trip to memory, and one head a
  // wave with two key groups is ahead (12 / 2 heads: 512 tokens behind 8,192: 147 | 121 us, behind 30,000: 504 |
  // 395; 128 behind 8,192: 151 | 114; 64 behind 2,000: 36 | 32; behind 1,000: 22 | 21.  28 / 4 heads: 256 behind
  // 8,192: 130 | 116), the more so as its tiles' keys can be cut over workgroups (below).  At head size 64 the
  // per-wave kernel (which gives such tiles eight waves) stays ahead up to some 3,000 keys (14 / 2 heads, 64 tokens
  // behind 2,000: 19 | 20 us) and falls behind the cut tiles beyond (16 behind 3,500: 27 | 20; 256 behind 8,192: 50 |
  // 30; 512 behind 30,000: 162 | 136).
  const bool far = reach >= (d == 128 ? 1024 : 3072);
  if (group < 5) {
    // Three or four heads per kv head fill the four waves at one head each (32 / 8 heads of 128, per-wave | 1 head
    // | 1 head, 2 groups: 1,024 tokens 37 | 30 | 28; 2,048 tokens 106 | 69 | 81; 8,192 tokens 1,217 | 790 | 913;
    // 16 / 4 heads of 64: 2,048 tokens 30.0 | 30.1 | 24.4; 8,192 tokens 307 | 213 | 221).
    const long one = (long)n_tiles * n_kv;
    if (one < 256) return far ? 11 : 0;
    return one < (d == 64 ? 2048 : 1024) ? 11 : 1;
  }
  const long two = (long)n_tiles * n_kv * ((group + 7) / 8);      // workgroups at two heads a wave
  // Behind 6,144 keys and more, with the keys cut over workgroups where those are few, what a launch pulls through
  // the fabric counts: two heads a wave read every block half as often (28 / 4 heads of 128, one | two heads a wave,
  // 256 tokens behind 8,192: 78 | 62 us, 512 tokens: 120 | 102, 256 behind 16,000: 121 | 93; 12 / 2 heads: 512 behind
  // 8,192: 73 | 58, 1,024: 128 | 101; 14 / 2 heads of 64: 512 behind 8,192: 47 | 41), but for the shortest portions
  // one head a wave stays ahead (64 tokens of 28 / 4 heads: 29 | 34; 128 of 12 / 2: 27 | 33).
  const bool very_far = far && reach >= 6144;
  if (two < 128) return !far ? 0 : (very_far && two >= 32) ? 12 : 11;
  if (two >= 1024) return 2;
  if (d == 64) return (very_far && two < 256) ? 12 : 11;
  if (two >= 512) return 12;
  if (two >= 256) return reach >= 4096 ? 12 : 11;
  return very_far ? 12 : 11;
}

// Returns -2 for a head size without an instance (the caller then uses the other kernel).
// shape: heads a wave (1 or 2), + 10 for two key groups in a workgroup.  key_splits: parts of a tile's keys, each
// a workgroup's; more than one needs part_o float [n_tiles * 16, n_q, key_splits, d] and part_ml float [.., 2].
extern "C" int ta_prefill_attention_shared_bf16(const void* q, int q_stride, void* out, const void* k_pages,
                                                const void* vt_pages, const void* tiles, int n_tiles,
                                                const void* cu_q, const void* first_position,
                                                const void* block_table, int table_stride, int n_q, int n_kv, int d,
                                                int page_size, int window, float scale, int shape,
                                                int key_splits, void* part_o, void* part_ml, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  const int heads_per_wave = shape % 10, key_groups = shape / 10 + 1;
  if (n_kv <= 0 || n_q % n_kv || page_size % 16 || heads_per_wave < 1 || heads_per_wave > 2 || key_groups > 2) return -1;
  if (key_splits < 1 || key_splits > 64 || (key_splits > 1 && (!part_o || !part_ml))) return -1;
#define GO(DD, HG, KG) return launch_shared<DD, HG, KG>(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, \
    first_position, block_table, table_stride, n_q, n_kv, page_size, window, scale, key_splits, part_o, part_ml, stream);
#define SIZE(DD) case DD: if (key_groups == 2) { if (heads_per_wave == 1) GO(DD, 1, 2) GO(DD, 2, 2) } \
    if (heads_per_wave == 1) GO(DD, 1, 1) GO(DD, 2, 1)
  switch (d) {
    SIZE(64) SIZE(128)
    default: return -2;
  }
#undef SIZE
#undef GO
}
