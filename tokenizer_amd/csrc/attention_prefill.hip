// Causal (optionally windowed) attention of prompt portions over paged bfloat16 keys and values on the
// matrix cores.  A workgroup owns a tile of 16 consecutive tokens of one request, one kv head and a block of
// HG of the query heads that share it; its NWV waves take the blocks of 64 keys in turn and merge their
// partial softmax states through LDS at the end, so that a tile late in a long prompt is not one long
// serial walk and a SIMD holds several waves whose matrix and vector work overlap.  As in the decode kernel both products are computed transposed
// (S^T = K Q^T, O^T = V^T P^T) with 16x16x32 MFMAs: the token index sits in `lane % 16` for scores and
// outputs, keys and values are read 16 bytes per lane straight from the pages, each key tile once for all
// HG heads.  Softmax runs online in float; probabilities are rounded to bfloat16 for the second product.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 pf_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// One step of the online softmax over 64 keys (sixteen consecutive keys lie inside one page) for the HG heads of
// the wave.  FULL: every key of the block is visible to every token of the tile, so nothing is masked.
// Scores stay unscaled; `c` = scale * log2(e) enters in exp2(s*c - m*c).
template <int D, int HG, bool FULL>
__device__ __forceinline__ void prefill_block(
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages, const int* __restrict__ table,
    int kb, int kvh, int n_kv, int page_size, int col, int g, int heads_here, int my_pos, int my_lo, int lo, int hi,
    float c, const bf16x8 (&qf)[HG][(D + 31) / 32], floatx4 (&acc)[HG][D / 16], float (&m)[HG], float (&l)[HG]) {
  constexpr int KS = (D + 31) / 32;
  constexpr int DB = D / 16;
  // The block is two halves of 32 keys.  Key base + k of a half is index k of the second product's contraction
  // (lane group g holds k = 8g .. 8g+7), so a lane's eight values of a row of V^T are sixteen contiguous bytes
  // of one page: one load.  For that the first product's instructions take a half's keys in an order of their
  // own: row r of instruction t is key base + 8 (r / 4) + 4 t + r % 4, whose score then lands in the lane group
  // that holds that key in the second product.  Sixteen consecutive keys lie in one page.
  bf16x8 kf[4][KS];                                    // [2 u + t]: instruction t of half u
  union VFrag { uint4 bits; bf16x8 v; } vf[2][DB];
  int left[2] = {7, 7};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int base_key = kb + 32 * u;
    const bool active = FULL || ((base_key <= hi) && (base_key + 31 >= lo));      // the same for the whole wave
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[2 * u + t][ks] = pf_zero8();
#pragma unroll
    for (int db = 0; db < DB; ++db) vf[u][db].bits = make_uint4(0, 0, 0, 0);
    if (active) {
      // A half's two runs of sixteen keys: one that holds no key of the range (before `lo`: its page may have been
      // given back; after `hi`: it may not exist yet) borrows the other's page, a valid address; what is read
      // there never counts (scores outside the range are masked, such values are set to zero).
      const bool there0 = FULL || base_key + 15 >= lo, there1 = FULL || base_key + 16 <= hi;
      const int page0 = scalar_int(table + (there0 ? base_key : base_key + 16) / page_size);
      const int page1 = scalar_int(table + (there1 ? base_key + 16 : base_key) / page_size);
      const uint32_t page_elems = (uint32_t)page_size * D;
      {
        const int half = col >> 3;
        const uint32_t at = ((uint32_t)(half ? page1 : page0) * n_kv + kvh) * page_elems +
                            (uint32_t)(((base_key + 16 * half) % page_size) + 8 * ((col >> 2) & 1) + (col & 3)) * D + 8 * g;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            if (ks * 32 + 8 * g < D)
              kf[2 * u + t][ks] = *reinterpret_cast<const bf16x8*>(k_pages + at + t * 4 * D + ks * 32);
      }
      {
        const int half = g >> 1;
        const uint32_t at = ((uint32_t)(half ? page1 : page0) * n_kv + kvh) * page_elems + (uint32_t)col * page_size +
                            ((base_key + 16 * half) % page_size) + 8 * (g & 1);
        // (Nothing that was loaded is touched before all of the block is asked for: a value that is used makes the
        // wave wait for everything it asked for before.)
        if (!FULL) left[u] = (half ? there1 : there0) ? hi - (base_key + 8 * g) : -1;    // keys of this lane that exist: 0..left
#pragma unroll
        for (int db = 0; db < DB; ++db)
          vf[u][db].bits = *reinterpret_cast<const uint4*>(vt_pages + at + db * 16 * page_size);
      }
    }
  }
  if (!FULL) {                                             // slots past the last key may never have been written
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (left[u] >= 7) continue;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        uint4 v = vf[u][db].bits;
        if (left[u] < 0) v.x = 0; else if (left[u] < 1) v.x &= 0xffffu;
        if (left[u] < 2) v.y = 0; else if (left[u] < 3) v.y &= 0xffffu;
        if (left[u] < 4) v.z = 0; else if (left[u] < 5) v.z &= 0xffffu;
        if (left[u] < 6) v.w = 0; else v.w &= 0xffffu;
        vf[u][db].bits = v;
      }
    }
  }
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    if (h >= heads_here) break;
    float s[16];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      floatx4 st = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks], qf[h][ks], st, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (FULL) {
          s[t * 4 + r] = st[r];
        } else {
          const int key = kb + 32 * (t >> 1) + 8 * g + 4 * (t & 1) + r;     // (keys outside lo..hi lie outside my_lo..my_pos)
          s[t * 4 + r] = (key <= my_pos && key >= my_lo) ? st[r] : -INFINITY;
        }
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])), fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
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
    bf16x8 pf[2];
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[i], c, -mc));   // masked keys: exp2(-inf) = 0
      psum += p;
      pf[i >> 3][i & 7] = (__bf16)p;
    }
    l[h] += psum;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      acc[h][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[0][db].v, pf[0], acc[h][db], 0, 0, 0);
      acc[h][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[1][db].v, pf[1], acc[h][db], 0, 0, 0);
    }
  }
}

// tiles: [n_tiles, 2] = (entry, offset of the tile's first token inside the entry's tokens).
// cu_q[e]: first row of entry e; first_position[e]: position of that row.
// K pages [n_pages, n_kv, page_size, D]; V^T pages [n_pages, n_kv, D, page_size]; page_size % 16 == 0.
template <int D, int HG, int NWV>
__global__ void __launch_bounds__(NWV * WAVE, (D <= 64 && HG <= 2) ? 3 : 1)
prefill_attention_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                         const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages,
                         const int* __restrict__ tiles, int n_tiles, const int* __restrict__ cu_q,
                         const int* __restrict__ first_position, const int* __restrict__ block_table,
                         int table_stride, int n_q, int n_kv, int page_size, int window, float scale_log2) {
  constexpr int KS = (D + 31) / 32;
  constexpr int DB = D / 16;
  HELD(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, first_position, block_table, table_stride, n_q, n_kv,
       page_size, window, scale_log2);
  __shared__ float merge[NWV > 1 ? NWV - 1 : 1][HG][DB * 4 + 2][WAVE];
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int col = lane & 15, g = lane >> 4;
  const int group = n_q / n_kv;
  const int head_blocks = (group + HG - 1) / HG;
  // The launch is one line of workgroups, all head blocks of the last tile first, then those of the tile before
  // it and so on: late tiles see the most keys, and every one of them should be under way before the short
  // ones fill the device (ordered by head block instead, half of the long tiles would start only when the
  // first half of the launch had drained, and the kernel would end with them alone on the device).
  const int per_tile = n_kv * head_blocks;
  const int which = blockIdx.x % per_tile;
  const int kvh = which / head_blocks, hb = which % head_blocks;
  const int heads_here = min(HG, group - hb * HG);
  const int head0 = kvh * group + hb * HG;
  const int tile_index = n_tiles - 1 - blockIdx.x / per_tile;
  // What describes the tile is the same for every lane; taken through the scalar unit so that all that is derived
  // from it (which keys are visible, which blocks need no mask) lives in scalar registers and branches on it
  // are scalar branches.
  const int entry = scalar_int(tiles + 2 * tile_index);
  const int offset = scalar_int(tiles + 2 * tile_index + 1);
  const int entry_row = scalar_int(cu_q + entry), next_row = scalar_int(cu_q + entry + 1);
  const int entry_position = scalar_int(first_position + entry);
  HELD(entry_row, next_row, entry_position);               // (the three that hang on the entry: one trip)
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
  const int* table = block_table + (size_t)entry * table_stride;

  bf16x8 qf[HG][KS];
#pragma unroll
  for (int h = 0; h < HG; ++h)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + 8 * g;
      qf[h][ks] = pf_zero8();
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

  // A wave's blocks come in three runs: those at the window's edge (some keys masked), those that every token
  // of the tile sees whole, and those on the diagonal.  Each run is a loop of its own over one variant of the
  // block: in one loop over both, the accumulators would be copied between the variants' registers every turn.
  int kb = (lo / 64) * 64 + 64 * wave;
  for (; kb <= hi && kb < lo_all; kb += 64 * NWV)
    prefill_block<D, HG, false>(k_pages, vt_pages, table, kb, kvh, n_kv, page_size, col, g, heads_here, my_pos,
                                my_lo, lo, hi, scale_log2, qf, acc, m, l);
  for (; kb + 63 <= p0; kb += 64 * NWV)
    prefill_block<D, HG, true>(k_pages, vt_pages, table, kb, kvh, n_kv, page_size, col, g, heads_here, my_pos,
                               my_lo, lo, hi, scale_log2, qf, acc, m, l);
  for (; kb <= hi; kb += 64 * NWV)
    prefill_block<D, HG, false>(k_pages, vt_pages, table, kb, kvh, n_kv, page_size, col, g, heads_here, my_pos,
                                my_lo, lo, hi, scale_log2, qf, acc, m, l);
  if (NWV > 1) {
    // Waves 1.. hand their state to wave 0: maximum, sum and the output accumulators of each head.
    if (wave > 0) {
#pragma unroll
      for (int h = 0; h < HG; ++h) {
        merge[wave - 1][h][DB * 4][lane] = m[h];
        merge[wave - 1][h][DB * 4 + 1][lane] = l[h];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) merge[wave - 1][h][db * 4 + r][lane] = acc[h][db][r];
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      float m_all = m[h];
#pragma unroll
      for (int w = 0; w < NWV - 1; ++w) m_all = fmaxf(m_all, merge[w][h][DB * 4][lane]);
      const float mc = (m_all == -INFINITY) ? 0.f : m_all * scale_log2;
      const float f0 = __builtin_amdgcn_exp2f(m[h] * scale_log2 - mc);       // a wave without keys: exp2(-inf) = 0
      l[h] *= f0;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][db][r] *= f0;
#pragma unroll
      for (int w = 0; w < NWV - 1; ++w) {
        const float f = __builtin_amdgcn_exp2f(merge[w][h][DB * 4][lane] * scale_log2 - mc);
        l[h] += f * merge[w][h][DB * 4 + 1][lane];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[h][db][r] += f * merge[w][h][db * 4 + r][lane];
      }
    }
  }
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

template <int D, int HG, int NWV>
static int launch_prefill_waves(const void* q, int q_stride, void* out, const void* k_pages, const void* vt_pages,
                                const void* tiles, int n_tiles, const void* cu_q, const void* first_position,
                                const void* block_table, int table_stride, int n_q, int n_kv, int page_size,
                                int window, float scale, hipStream_t stream) {
  const int group = n_q / n_kv;
  const long workgroups = (long)n_tiles * n_kv * ((group + HG - 1) / HG);
  if (workgroups > 0x7fffffffL) return -1;
  prefill_attention_kernel<D, HG, NWV><<<(unsigned)workgroups, NWV * WAVE, 0, stream>>>(
      (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)vt_pages, (const int*)tiles,
      n_tiles, (const int*)cu_q, (const int*)first_position, (const int*)block_table, table_stride, n_q, n_kv, page_size,
      window, scale * 1.4426950408889634f);
  return LAUNCH_STATUS();
}

// How far back the farthest-seeing token of the batch looks, by the context rounded up to a multiple of 512 keys,
// so that a launch planned for a range of contexts (one recorded in a graph) and a launch for the exact context
// make the same choices.
static int planned_reach(int max_keys, int window) {
  const int planned = (max_keys + 511) / 512 * 512;
  return (window >= 0 && window + 16 < planned) ? window + 16 : planned;
}

// waves: waves per tile (1, 2, 4, or 8 at head sizes 48 and 64); 0 = by the longest reach of a token: one wave per
// 256 keys or so, eight for few tiles with a long reach.
template <int D, int HG>
static int launch_prefill(const void* q, int q_stride, void* out, const void* k_pages, const void* vt_pages,
                          const void* tiles, int n_tiles, const void* cu_q, const void* first_position,
                          const void* block_table, int table_stride, int n_q, int n_kv, int page_size, int window,
                          float scale, int max_keys, int waves, hipStream_t stream) {
  if (waves == 0) {
    const int reach = planned_reach(max_keys, window);
    waves = reach > 768 ? 4 : reach > 256 ? 2 : 1;
    // A short portion behind a long cached context: a handful of tiles, each with thousands of keys to walk and a
    // SIMD to itself, so that nothing hides a block's trip to memory.  Eight waves halve each wave's walk (512
    // tokens of 14 / 2 heads of 64 behind 8,192: 64 -> 56 us; behind 30,000: 240 -> 161 us; 256 behind 8,192:
    // 58 -> 49 us); from 1,024 tokens on, where the waves crowd the compute units, they are slower (89 -> 109 us).
    const long workgroups = (long)n_tiles * n_kv * ((n_q / n_kv + HG - 1) / HG);
    if ((D == 48 || D == 64) && reach >= 4096 && workgroups <= 256) waves = 8;
    // Head sizes above 64 need so many registers that a SIMD holds one wave: two workgroups of two waves fill a
    // compute unit better than one of four (measured at head sizes 96, 128 and 256, 512 to 8,192 tokens).
    if (D > 64 && waves > 2) waves = 2;
  }
#define GO(NWV) launch_prefill_waves<D, HG, NWV>(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, \
    first_position, block_table, table_stride, n_q, n_kv, page_size, window, scale, stream)
  if constexpr (D == 48 || D == 64) {          // (the eight waves' states fit the static LDS at these sizes)
    if (waves >= 8) return GO(8);
  }
  if (waves >= 4) return GO(4);
  if (waves >= 2) return GO(2);
  return GO(1);
#undef GO
}

// The kernel whose waves share a block of keys through LDS (attention_prefill_shared.hip).
extern "C" int ta_prefill_attention_shared_plan(int n_tiles, int n_q, int n_kv, int d, int reach);
extern "C" int ta_prefill_attention_shared_key_splits(int n_tiles, int n_q, int n_kv, int reach, int shape);
extern "C" int ta_prefill_attention_shared_bf16(const void* q, int q_stride, void* out, const void* k_pages,
                                                const void* vt_pages, const void* tiles, int n_tiles,
                                                const void* cu_q, const void* first_position,
                                                const void* block_table, int table_stride, int n_q, int n_kv, int d,
                                                int page_size, int window, float scale, int shape,
                                                int key_splits, void* part_o, void* part_ml, hipStream_t stream);

// The shape in which the workgroup-shared kernel takes a launch (0: the per-wave kernel takes it), by what the
// caller asked for and the launch's own plan.
static int shared_shape_for(int n_tiles, int n_q, int n_kv, int d, int window, int shared_shape, int max_keys,
                            int waves, int shared) {
  if (shared < 0 || waves != 0 || (d != 64 && d != 128)) return 0;
  int shape = ta_prefill_attention_shared_plan(n_tiles, n_q, n_kv, d, planned_reach(max_keys, window));
  if (shared > 0) shape = shared_shape > 0 ? shared_shape : shape ? shape : 2;
  return shape;
}

// Into how many parts the launch below cuts the keys of a tile over workgroups (1: it does not).  More than one
// needs the buffers `part_o` float [n_tiles * 16, n_q, parts, d] and `part_ml` float [n_tiles * 16, n_q, parts, 2].
extern "C" int ta_prefill_attention_key_splits(int n_tiles, int n_q, int n_kv, int d, int window, int shared_shape,
                                               int max_keys, int waves, int shared) {
  if (n_tiles <= 0 || n_kv <= 0 || n_q % n_kv) return 1;
  const int shape = shared_shape_for(n_tiles, n_q, n_kv, d, window, shared_shape, max_keys, waves, shared);
  return ta_prefill_attention_shared_key_splits(n_tiles, n_q, n_kv, planned_reach(max_keys, window), shape);
}

// Returns -2 for a head size without an instance (the caller then uses another kernel).
// max_keys: the highest position of the batch + 1 (a hint for the number of waves per tile).
// shared: 1 = the workgroup-shared kernel wherever it has an instance (in the shape `shared_shape` names: 1 or 2
// heads a wave, + 10 for two key groups; 0 = its own choice), -1 = never, 0 = where it is the faster one (by the shape of the launch and the planned
// reach, so that a launch recorded for a range of contexts and a launch for the exact context make the same
// choice).  waves: waves that share a tile's keys in the per-wave kernel (1, 2, 4, 8; 0 = by the reach); asking
// for a number asks for that kernel.  part_o, part_ml: buffers for `ta_prefill_attention_key_splits(...)` parts of
// a tile's keys (null: the keys are not cut).
extern "C" int ta_prefill_attention_bf16(const void* q, int q_stride, void* out, const void* k_pages,
                                         const void* vt_pages, const void* tiles, int n_tiles, const void* cu_q,
                                         const void* first_position, const void* block_table, int table_stride,
                                         int n_q, int n_kv, int d, int page_size, int window, float scale,
                                         int shared_shape, int max_keys, int waves, int shared,
                                         void* part_o, void* part_ml, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (n_kv <= 0 || n_q % n_kv || page_size % 16) return -1;
  const int shape = shared_shape_for(n_tiles, n_q, n_kv, d, window, shared_shape, max_keys, waves, shared);
  if (shape) {
    const int parts = (part_o && part_ml)
        ? ta_prefill_attention_shared_key_splits(n_tiles, n_q, n_kv, planned_reach(max_keys, window), shape) : 1;
    const int status = ta_prefill_attention_shared_bf16(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q,
                                                        first_position, block_table, table_stride, n_q, n_kv, d,
                                                        page_size, window, scale, shape, parts, part_o, part_ml, stream);
    if (status != -2) return status;
  }
#define CASE(DD, HG) case DD: return launch_prefill<DD, HG>(q, q_stride, out, k_pages, vt_pages, tiles, n_tiles, cu_q, \
    first_position, block_table, table_stride, n_q, n_kv, page_size, window, scale, max_keys, waves, stream);
  switch (d) {
    CASE(16, 4) CASE(32, 4) CASE(48, 2) CASE(64, 2) CASE(80, 2) CASE(96, 2) CASE(112, 2) CASE(128, 2)
    CASE(160, 1) CASE(192, 1) CASE(224, 1) CASE(256, 1)
    default: return -2;
  }
#undef CASE
}
