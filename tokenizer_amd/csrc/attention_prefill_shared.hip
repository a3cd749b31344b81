// Prompt attention for many query heads per kv head and long reaches: the workgroup of a tile of 16 tokens and one
// kv head holds NW waves, each with HG of the query heads that share the kv head, and all of them walk the
// same blocks of 64 keys.  A block's keys and values come from the pages once for the whole workgroup, through
// registers into LDS, two buffers deep: the next block is on its way while the matrix cores work on the
// current one, and every wave takes its fragments from LDS.  Against the kernel in attention_prefill.hip
// (each wave fetches its own blocks for its own two heads) a key is read from the cache 1/NW as often and
// no wave waits for memory with nothing else to do; it pays where the pages' traffic or its latency bound
// that kernel: large heads, long prompts.  Same fragment layouts and key order as there: S^T = K Q^T and
// O^T = V^T P^T with 16x16x32 MFMAs, token index in `lane % 16`, softmax online in float, probabilities
// rounded to bfloat16 for the second product.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t piece_t __attribute__((ext_vector_type(4)));   // sixteen bytes on their way from a page to LDS

// A block in LDS: 64 rows of keys, then D rows of 64 values each (V^T).  Rows are 16 bytes longer than their
// contents, so that the rows which eight neighbouring lanes read at once start four banks apart.
template <int D>
struct Staged {
  static constexpr int K_ROW = 2 * D + 16;
  static constexpr int V_ROW = 2 * 64 + 16;
  static constexpr int K_BYTES = 64 * K_ROW;
  static constexpr int BYTES = K_BYTES + D * V_ROW;
};

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

// What a thread carries of every block: the same pieces of each of the block's four runs of sixteen keys (a run
// lies inside one page), so that per block only four page numbers change, which are the same for the whole
// workgroup, and a load is a scalar base plus an offset that the lane worked out once.
template <int D, int THREADS>
struct Carrier {
  static constexpr int RUN_PIECES = 2 * D;                  // 16 keys of D / 8 pieces; as many of the values
  static constexpr int ROUNDS = (RUN_PIECES + THREADS - 1) / THREADS;
  uint32_t k_from[ROUNDS], v_from[ROUNDS];                  // element offsets inside a run's part of its page
  uint32_t k_to[ROUNDS], v_to[ROUNDS];                      // byte offsets inside a block in LDS (run 0)
  bool mine[ROUNDS];
  int v_first[ROUNDS];                                      // first key of the value piece, within its run
  piece_t k[4][ROUNDS], v[4][ROUNDS];
  int at_page, at_slot;                                     // where the next run to look up lies: index into the block table, slot in the page
  int page[4], slot[4];                                     // of the runs of the block to fetch next (the same for all threads)
  bool there[4];                                            // whether the run holds a key of lo..hi
  int page_size;
  uint32_t page_elements, first_element;                    // elements of a page (all kv heads); where this kv head's begin

  // first_key: the first key of the first block.
  __device__ __forceinline__ void plan(int tid, const SharedTile& tile, int first_key) {
    page_size = tile.page_size;
    page_elements = (uint32_t)tile.n_kv * page_size * D;
    first_element = (uint32_t)tile.kvh * page_size * D;
    at_page = first_key / page_size;
    at_slot = first_key % page_size;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int piece = r * THREADS + tid;
      mine[r] = RUN_PIECES % THREADS == 0 || piece < RUN_PIECES;
      const int key = piece / (D / 8), part = piece % (D / 8);
      k_from[r] = (uint32_t)(key * D + part * 8);
      k_to[r] = (uint32_t)(key * Staged<D>::K_ROW + part * 16);
      const int d = piece >> 1, half = piece & 1;
      v_from[r] = (uint32_t)(d * page_size + half * 8);
      v_to[r] = (uint32_t)(Staged<D>::K_BYTES + d * Staged<D>::V_ROW + half * 16);
      v_first[r] = 8 * half;
    }
  }

  // Where the four runs of block `kb` lie: their pages and slots, looked up a turn before the block is fetched,
  // so that no wave waits for a page number.  Blocks are looked up in order.  `full`: every key of the block
  // exists and is seen by every token.  Otherwise a run without a key of lo..hi (before `lo`: its page may have
  // been given back; after `hi`: it may not exist yet) borrows the page of `lo` or `hi`, a valid address.
  __device__ __forceinline__ void look_up(const SharedTile& tile, int kb, bool full) {
    if (full) {                                            // the usual block: nothing to decide per run
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        page[q] = tile.table[at_page];
        slot[q] = at_slot;
        there[q] = true;
        step();
      }
      return;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int key = kb + 16 * q;
      int index = at_page;
      there[q] = key + 15 >= tile.lo && key <= tile.hi;
      if (key + 15 < tile.lo) index = tile.lo_page;
      if (key > tile.hi) index = tile.hi_page;
      page[q] = tile.table[index];
      slot[q] = at_slot;
      step();
    }
  }

  // On to the next run: pages hold whole runs.
  __device__ __forceinline__ void step() {
    at_slot += 16;
    if (at_slot >= page_size) {
      at_slot = 0;
      ++at_page;
    }
  }

  // The block that was looked up last, from the pages into registers.  Unless the block is `full`, the values
  // of a borrowed run become zero, as do values past `hi` (slots never written): a probability of zero times
  // whatever lies there must stay zero.  Keys need no such care, their scores are masked by selection.
  __device__ __forceinline__ void fetch(const SharedTile& tile, int kb, bool full) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t head = (uint32_t)page[q] * page_elements + first_element;
      const bf16_t* k_run = tile.k_pages + (head + (uint32_t)slot[q] * D);
      const bf16_t* v_run = tile.vt_pages + (head + (uint32_t)slot[q]);
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) {
        if (!mine[r]) continue;
        k[q][r] = *reinterpret_cast<const piece_t*>(k_run + k_from[r]);
        v[q][r] = *reinterpret_cast<const piece_t*>(v_run + v_from[r]);
      }
    }
    if (full) return;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) {
        if (!mine[r]) continue;
        const int left = there[q] ? tile.hi - (kb + 16 * q + v_first[r]) : -1;     // keys of this piece that exist: 0..left
        if (left < 7) {
          piece_t x = v[q][r];
          if (left < 0) x.x = 0; else if (left < 1) x.x &= 0xffffu;
          if (left < 2) x.y = 0; else if (left < 3) x.y &= 0xffffu;
          if (left < 4) x.z = 0; else if (left < 5) x.z &= 0xffffu;
          if (left < 6) x.w = 0; else x.w &= 0xffffu;
          v[q][r] = x;
        }
      }
  }

  __device__ __forceinline__ void put(char* buf) const {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) {
        if (!mine[r]) continue;
        *reinterpret_cast<piece_t*>(buf + k_to[r] + q * 16 * Staged<D>::K_ROW) = k[q][r];
        *reinterpret_cast<piece_t*>(buf + v_to[r] + q * 32) = v[q][r];
      }
  }
};

// One step of the online softmax of a wave's HG heads over the block of 64 keys in `buf`.  Row r of the first
// product's instruction t of a half of 32 keys is key 8 (r / 4) + 4 t + r % 4 of the half, whose score then lies
// in the lane group that holds that key in the second product (lane group g: keys 8g .. 8g+7).
template <int D, int HG, bool FULL>
__device__ __forceinline__ void shared_block(const char* buf, int kb, int col, int g, int my_pos, int my_lo, float c,
                                             const bf16x8 (&qf)[HG][(D + 31) / 32], floatx4 (&acc)[HG][D / 16],
                                             float (&m)[HG], float (&l)[HG]) {
  constexpr int KS = (D + 31) / 32;
  constexpr int DB = D / 16;
  float s[HG][16];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int key = 32 * (t >> 1) + 8 * (col >> 2) + 4 * (t & 1) + (col & 3);
    bf16x8 kf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = sh_zero8();
      if (ks * 32 + 8 * g < D)
        kf[ks] = *reinterpret_cast<const bf16x8*>(buf + key * Staged<D>::K_ROW + (ks * 32 + 8 * g) * 2);
    }
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
    float mx = fmaxf(fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3])), fmaxf(fmaxf(sh[4], sh[5]), fmaxf(sh[6], sh[7])));
    mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(sh[8], sh[9]), fmaxf(sh[10], sh[11])), fmaxf(fmaxf(sh[12], sh[13]), fmaxf(sh[14], sh[15]))));
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m[h], mx);
    // A token that has seen no key yet keeps m = -inf; exp2 of (-inf) - (-inf) would be NaN.
    const float mc = (m_new == -INFINITY) ? 0.f : m_new * c;
    if (__any(m_new > m[h])) {                          // rescale only when some token's maximum moved
      const float corr = __builtin_amdgcn_exp2f(m[h] * c - mc);   // m = -inf gives 0
      l[h] *= corr;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][db][r] *= corr;
      m[h] = m_new;
    }
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = __builtin_amdgcn_exp2f(fmaf(sh[i], c, -mc));   // masked keys: exp2(-inf) = 0
      psum += p;
      pf[h][i >> 3][i & 7] = (__bf16)p;
    }
    l[h] += psum;
  }
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(buf + Staged<D>::K_BYTES + (db * 16 + col) * Staged<D>::V_ROW +
                                                         (32 * u + 8 * g) * 2);
#pragma unroll
      for (int h = 0; h < HG; ++h) acc[h][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[h][u], acc[h][db], 0, 0, 0);
    }
}

// Arguments as in prefill_attention_kernel.  Dynamic LDS: two blocks (2 * Staged<D>::BYTES).
template <int D, int HG, int NW>
__global__ void __launch_bounds__(NW * WAVE, 1)
prefill_attention_shared_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                                const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages,
                                const int* __restrict__ tiles, int n_tiles, const int* __restrict__ cu_q,
                                const int* __restrict__ first_position, const int* __restrict__ block_table,
                                int table_stride, int n_q, int n_kv, int page_size, int window, float scale_log2) {
  constexpr int KS = (D + 31) / 32;
  constexpr int DB = D / 16;
  constexpr int THREADS = NW * WAVE;
  extern __shared__ __attribute__((aligned(16))) char staged[];
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int col = lane & 15, g = lane >> 4;
  const int group = n_q / n_kv;
  const int head_blocks = (group + HG * NW - 1) / (HG * NW);
  // Late tiles first, as in the other prompt kernel: they see the most keys.
  const int per_tile = n_kv * head_blocks;
  const int which = blockIdx.x % per_tile;
  const int kvh = which / head_blocks, hb = which % head_blocks;
  const int first_head = hb * HG * NW + wave * HG;            // among the heads of the kv head
  const int heads_here = max(0, min(HG, group - first_head));  // a wave past the last head only carries blocks
  const int head0 = kvh * group + first_head;
  const int tile_index = n_tiles - 1 - blockIdx.x / per_tile;
  const int entry = __builtin_amdgcn_readfirstlane(tiles[2 * tile_index]);
  const int offset = __builtin_amdgcn_readfirstlane(tiles[2 * tile_index + 1]);
  const int row0 = __builtin_amdgcn_readfirstlane(cu_q[entry]) + offset;
  const int n_valid = min(16, __builtin_amdgcn_readfirstlane(cu_q[entry + 1]) - row0);
  const int p0 = __builtin_amdgcn_readfirstlane(first_position[entry]) + offset;   // position of the tile's first token
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
      const int d0 = ks * 32 + 8 * g;
      qf[h][ks] = sh_zero8();
      if (h < heads_here && d0 < D)
        qf[h][ks] = *reinterpret_cast<const bf16x8*>(q + (size_t)my_row * q_stride + (size_t)(head0 + h) * D + d0);
    }
  floatx4 acc[HG][DB];
  float m[HG], l[HG];
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[h][db] = (floatx4){0.f, 0.f, 0.f, 0.f};
  }

  // Blocks come in three runs (the window's edge, those every token sees whole, the diagonal), each a loop of
  // its own over one variant of the block, so that the accumulators stay in the same registers within a loop.
  // Every thread goes through every turn: the barrier at its end hands the buffer that was just filled to the
  // next turn, and the buffer that was just read to the turn after it.
  int kb = (lo / 64) * 64;
  int cur = 0;
  Carrier<D, THREADS> carrier;
  carrier.plan(tid, tile, kb);
  const auto whole = [&](int block) { return block >= lo_all && block + 63 <= p0; };
  carrier.look_up(tile, kb, whole(kb));
  carrier.fetch(tile, kb, whole(kb));
  if (kb + 64 <= hi) carrier.look_up(tile, kb + 64, whole(kb + 64));
  carrier.put(staged);
  __syncthreads();
#define TURN(FULL)                                                                                            \
  {                                                                                                           \
    const int next = kb + 64;                                                                                 \
    const bool more = next <= hi;                                                                             \
    if (more) carrier.fetch(tile, next, whole(next));                                                         \
    if (next + 64 <= hi) carrier.look_up(tile, next + 64, whole(next + 64));                                  \
    if (heads_here > 0)                                                                                       \
      shared_block<D, HG, FULL>(staged + cur * Staged<D>::BYTES, kb, col, g, my_pos, my_lo, scale_log2, qf, acc, m, l); \
    if (more) carrier.put(staged + (cur ^ 1) * Staged<D>::BYTES);                                             \
    __syncthreads();                                                                                          \
    cur ^= 1;                                                                                                 \
  }
  for (; kb <= hi && kb < lo_all; kb += 64) TURN(false)
  for (; kb + 63 <= p0; kb += 64) TURN(true)
  for (; kb <= hi; kb += 64) TURN(false)
#undef TURN

#pragma unroll
  for (int h = 0; h < HG; ++h) {
    if (h >= heads_here) break;
    float total = l[h];
    total += __shfl_xor(total, 16, WAVE);
    total += __shfl_xor(total, 32, WAVE);
    if (col >= n_valid) continue;
    const float inv = 1.0f / total;
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

template <int D, int HG, int NW>
static int launch_shared(const void* q, int q_stride, void* out, const void* k_pages, const void* vt_pages,
                         const void* tiles, int n_tiles, const void* cu_q, const void* first_position,
                         const void* block_table, int table_stride, int n_q, int n_kv, int page_size, int window,
                         float scale, hipStream_t stream) {
  const int group = n_q / n_kv;
  const long workgroups = (long)n_tiles * n_kv * ((group + HG * NW - 1) / (HG * NW));
  if (workgroups > 0x7fffffffL) return -1;
  constexpr int lds = 2 * Staged<D>::BYTES;
  static_assert(lds <= 160 * 1024, "two blocks must fit a compute unit's LDS");
  if (lds > 48 * 1024) {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attention_shared_kernel<D, HG, NW>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (err != hipSuccess) return (int)err;
  }
  prefill_attention_shared_kernel<D, HG, NW><<<(unsigned)workgroups, NW * WAVE, lds, stream>>>(
      (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)vt_pages, (const int*)tiles,
      n_tiles, (const int*)cu_q, (const int*)first_position, (const int*)block_table, table_stride, n_q, n_kv, page_size,
      window, scale * 1.4426950408889634f);
  return LAUNCH_STATUS();
}

// Where the workgroup-shared kernel is the faster one: five to eight query heads per kv head (or a multiple of
// that many) fill its four waves, and the launch must have two workgroups or so for every compute unit, because a
// workgroup walks all its keys alone (measured at head size 128 on 256 compute units: 0.5-0.95x with 64 to 256
// workgroups, 1.4-1.9x from 512 on, for 5, 6, 7 and 8 heads per kv head; at head size 64 the two kernels are
// level even at 32,768 tokens, so it has no instance there).
extern "C" int ta_prefill_attention_shared_pays(int n_tiles, int n_q, int n_kv, int d) {
  if (d != 96 && d != 128) return 0;
  const int group = n_q / n_kv;
  if (group < 5) return 0;
  return (long)n_tiles * n_kv * ((group + 7) / 8) >= 512;
}

// Returns -2 for a head size without an instance (the caller then uses the other kernel).
extern "C" int ta_prefill_attention_shared_bf16(const void* q, int q_stride, void* out, const void* k_pages,
                                                const void* vt_pages, const void* tiles, int n_tiles,
                                                const void* cu_q, const void* first_position,
                                                const void* block_table, int table_stride, int n_q, int n_kv, int d,
                                                int page_size, int window, float scale, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (n_kv <= 0 || n_q % n_kv || page_size % 16) return -1;
#define SIZE(DD) case DD: return launch_shared<DD, 2, 4>(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, \
    first_position, block_table, table_stride, n_q, n_kv, page_size, window, scale, stream);
  switch (d) {
    SIZE(96) SIZE(128)
    default: return -2;
  }
#undef SIZE
}
