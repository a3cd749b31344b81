// Attention of single query tokens over paged bfloat16 keys and values on the matrix cores, with the
// key range of every token split over several workgroups (partial results are merged by a second kernel).
//
// One workgroup handles one (token, kv head, block of up to 16 query heads, split).  The query heads that
// share a kv head form the N dimension of the 16x16x32 MFMA, so keys and values are read once for all of
// them.  Both products are computed transposed, S^T = K Q^T and O^T = V^T P^T, which keeps the head index
// in `lane % 16` for scores and outputs alike: the online-softmax rescaling needs no cross-lane traffic.
// Values are stored transposed inside a page ([page, kv head, d, slot]), so that the eight keys a lane
// contracts over are contiguous in memory.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));


__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// D: head size (multiple of 16).  Pages: K [n_pages, n_kv, page_size, D], V^T [n_pages, n_kv, D, page_size],
// page_size a multiple of 16.  rows: the token rows to serve (null: row i = item i; a negative row is passed over).
// Token at position p sees keys max(0, p - window)..p (window < 0: from 0).
// Partials: part_o [n_items, n_q, splits, D] (unnormalised), part_ml [n_items, n_q, splits, 2] (max, sum);
// with splits == 1 the result goes straight to `out` [n_tokens, n_q * D].
// AHEAD: a wave asks for its next block of keys while it works on the current one (see below).
template <int D, int DEC_WAVES, bool AHEAD>
__global__ void __launch_bounds__(DEC_WAVES * WAVE)
decode_attention_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                        const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages,
                        const int* __restrict__ rows, const int* __restrict__ positions,
                        const int* __restrict__ entry_of_token, const int* __restrict__ block_table,
                        int table_stride, float* __restrict__ part_o, float* __restrict__ part_ml,
                        int n_q, int n_kv, int page_size, int window, float scale, int split_keys, int splits) {
  constexpr int KS = (D + 31) / 32;   // 32-wide steps over the head size for Q K^T
  constexpr int DB = D / 16;          // 16-row blocks of O^T
  HELD(q, q_stride, out, k_pages, vt_pages, rows, positions, entry_of_token, block_table, table_stride, part_o, part_ml,
       n_q, n_kv, page_size, window, scale, split_keys, splits);
  __shared__ float acc_s[DEC_WAVES][D][17];
  __shared__ float m_s[DEC_WAVES][16], l_s[DEC_WAVES][16];

  const int split = blockIdx.x;
  const int group = n_q / n_kv;
  const int head_blocks = (group + 15) / 16;
  const int kvh = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int item = blockIdx.z;
  const int t = rows ? scalar_int(rows + item) : item;      // the same for every lane
  if (t < 0) return;                                       // a row that only fills the list up: nothing to do
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int col = lane & 15, g = lane >> 4;
  const int heads_here = min(16, group - hb * 16);
  const int head = kvh * group + hb * 16 + col;          // valid when col < heads_here
  // entry_of_token null: every request has one token in the batch, request e is row e (one dependent load fewer).
  const int* table = block_table + (size_t)(entry_of_token ? scalar_int(entry_of_token + t) : t) * table_stride;
  // Without a window the split's first key does not hang on the position, so the pages of the wave's first block
  // are looked up beside the position rather than after it (one trip fewer before the first keys are asked for).
  // An entry past the request's pages may hold anything; it is only used for keys that exist (see load_block).
  const int early_kb = split * split_keys + wave * 32;
  int early_page0 = 0, early_page1 = 0;
  if (window < 0) {
    early_page0 = scalar_int(table + min(early_kb / page_size, table_stride - 1));
    early_page1 = scalar_int(table + min((early_kb + 16) / page_size, table_stride - 1));
  }
  const int pos = scalar_int(positions + t);
  const int lo = (window >= 0 && pos > window) ? pos - window : 0;
  const int first = (lo / 32) * 32 + split * split_keys;  // first key of this split (a multiple of 32)
  const int last = min(pos, first + split_keys - 1);

  // Q^T fragments: lane holds head `col`, head-size elements ks*32 + 8g .. +7.
  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + 8 * g;
    qf[ks] = zero8();
    if (col < heads_here && d0 < D)
      qf[ks] = *reinterpret_cast<const bf16x8*>(q + (size_t)t * q_stride + (size_t)head * D + d0);
  }
  floatx4 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = (floatx4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // A block of 32 keys as the matrix instructions want it.  Key kb + k is index k of the second product's
  // contraction (lane group g holds k = 8g .. 8g+7), so a lane's eight values of a row of V^T are sixteen
  // contiguous bytes of one page: one load.  For that the first product's two instructions take the keys in an
  // order of their own: row r of instruction t is key kb + 8 (r / 4) + 4 t + r % 4, whose score then lands in
  // the lane group that holds that key in the second product.  Keys kb .. kb+15 lie in one page, kb+16 .. kb+31
  // in one (page sizes are multiples of 16).
  struct KeyBlock {
    bf16x8 kf[2][KS];
    union VFrag { uint4 bits; bf16x8 v; } vf[DB];
    bool active;
    int left;                                              // this lane's eight keys of the block that exist: 0 .. left
  };
  // All loads of a block are issued together: keys, and values (whose addresses do not wait for the scores).
  // Nothing that was loaded is touched here (values of slots nobody wrote are set to zero when the block is used):
  // a value that is used makes the wave wait for all it asked for before, one trip to memory for every such use.
  auto load_block = [&](KeyBlock& blk, int kb) {
    blk.active = (kb <= last) && (kb + 31 >= lo);
    blk.left = 7;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) blk.kf[t][ks] = zero8();
#pragma unroll
    for (int db = 0; db < DB; ++db) blk.vf[db].bits = make_uint4(0, 0, 0, 0);
    if (blk.active) {
      // The two halves of sixteen keys: a half that holds no key of the range (before `lo`: its page may have been
      // given back; after `last`: it may not exist yet) borrows the other half's page, which is a valid address;
      // what is read there never counts (scores outside lo..last are masked, such values are set to zero).  So
      // the branch is the same for the whole wave, and the addresses are a page number a lane away from scalars.
      const bool there0 = kb + 15 >= lo, there1 = kb + 16 <= last;
      int page0, page1;
      if (window < 0 && kb == early_kb) {                    // (without a window the first half always holds keys)
        page0 = early_page0;
        page1 = there1 ? early_page1 : early_page0;
      } else {
        page0 = scalar_int(table + (there0 ? kb : kb + 16) / page_size);
        page1 = scalar_int(table + (there1 ? kb + 16 : kb) / page_size);
      }
      const uint32_t page_elems = (uint32_t)page_size * D;                  // same element count for K and V^T pages
      {
        const int half = col >> 3;
        const uint32_t at = ((uint32_t)(half ? page1 : page0) * n_kv + kvh) * page_elems +
                            (uint32_t)(((kb + 16 * half) % page_size) + 8 * ((col >> 2) & 1) + (col & 3)) * D + 8 * g;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            if (ks * 32 + 8 * g < D) blk.kf[t][ks] = *reinterpret_cast<const bf16x8*>(k_pages + at + t * 4 * D + ks * 32);
      }
      {
        const int half = g >> 1;
        const uint32_t at = ((uint32_t)(half ? page1 : page0) * n_kv + kvh) * page_elems + (uint32_t)col * page_size +
                            ((kb + 16 * half) % page_size) + 8 * (g & 1);
        blk.left = (half ? there1 : there0) ? last - (kb + 8 * g) : -1;
#pragma unroll
        for (int db = 0; db < DB; ++db)
          blk.vf[db].bits = *reinterpret_cast<const uint4*>(vt_pages + at + db * 16 * page_size);
      }
    }
  };
  // One step of the online softmax over a block that has been brought in.
  auto attend = [&](KeyBlock& blk, int kb) {
    if (blk.left < 7) {                                      // slots nobody wrote may hold anything: 0 * NaN would poison the sum
      const int left = blk.left;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        uint4 v = blk.vf[db].bits;
        if (left < 0) v.x = 0; else if (left < 1) v.x &= 0xffffu;
        if (left < 2) v.y = 0; else if (left < 3) v.y &= 0xffffu;
        if (left < 4) v.z = 0; else if (left < 5) v.z &= 0xffffu;
        if (left < 6) v.w = 0; else v.w &= 0xffffu;
        blk.vf[db].bits = v;
      }
    }
    float s[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      floatx4 st = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kf[t][ks], qf[ks], st, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = kb + 8 * g + 4 * t + r;
        s[t][r] = (blk.active && key >= lo && key <= last) ? st[r] * scale : -INFINITY;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                     fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m, mx);
    if (__all(m_new == -INFINITY)) return;                 // nothing visible yet: the same for every head, a scalar branch
    const float corr = (m_new == -INFINITY) ? 1.f : __expf(m - m_new);
    bf16x8 pf;
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __expf(s[t][r] - m_new);           // exp(-inf) = 0 for masked keys
        psum += p;
        pf[t * 4 + r] = (__bf16)p;
      }
    l = l * corr + psum;
    m = m_new;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[db][r] *= corr;
      acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.vf[db].v, pf, acc[db], 0, 0, 0);
    }
  };
  constexpr int STRIDE = DEC_WAVES * 32;
  int kb = first + wave * 32;
  if constexpr (AHEAD) {
    // Two blocks in turn: while one is worked on, the next one's keys and values are on their way (a wave that
    // asked for them only when it got there would wait a trip to memory in every block).  That pays while a wave
    // has a few blocks; over dozens of blocks the second set of registers costs more in waves a SIMD holds
    // (measured at batch 64, head size 64: 1.03x at a context of 2,048, level at 8,192, 0.89x at 30,000).
    if (kb <= last) {
      KeyBlock one, two;
      load_block(one, kb);
      while (true) {
        const bool more = kb + STRIDE <= last;
        if (more) load_block(two, kb + STRIDE);
        attend(one, kb);
        kb += STRIDE;
        if (!more) break;
        const bool further = kb + STRIDE <= last;
        if (further) load_block(one, kb + STRIDE);
        attend(two, kb);
        kb += STRIDE;
        if (!further) break;
      }
    }
  } else {
    for (; kb <= last; kb += STRIDE) {
      KeyBlock one;
      load_block(one, kb);
      attend(one, kb);
    }
  }
  // Sum of the lane groups' partial denominators (the maximum is already common to them).
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc_s[wave][db * 16 + 4 * g + r][col] = acc[db][r];
  if (g == 0) { m_s[wave][col] = m; l_s[wave][col] = l; }
  __syncthreads();
  // Merge the waves: thread (head h, element block) walks over D.
  for (int idx = threadIdx.x; idx < 16 * D; idx += DEC_WAVES * WAVE) {
    const int h = idx / D, d = idx % D;
    if (h >= heads_here) continue;
    float big = -INFINITY;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) big = fmaxf(big, m_s[w][h]);
    float o = 0.f, denom = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) {
      const float wgt = (m_s[w][h] == -INFINITY) ? 0.f : __expf(m_s[w][h] - big);
      o += acc_s[w][d][h] * wgt;
      denom += l_s[w][h] * wgt;
    }
    const int hg = kvh * group + hb * 16 + h;
    if (splits == 1) {
      st(out + (size_t)t * n_q * D + (size_t)hg * D + d, o / denom);
    } else {
      const size_t p = ((size_t)item * n_q + hg) * splits + split;
      part_o[p * D + d] = o;
      if (d == 0) { part_ml[p * 2] = big; part_ml[p * 2 + 1] = denom; }
    }
  }
}

// out[t, head, :] = sum_s part_o[s] * exp(m_s - M) / sum_s l_s * exp(m_s - M).  One wave per (item, head).
// Sixteen lanes share a split's 64 elements (a float4 each), the four groups of sixteen take every fourth
// split, and all of a lane's loads are requested before the first is used: the kernel is one trip to memory.
// A separate kernel on purpose: a last-arrival merge inside the first kernel needs device-wide fences,
// which flush the L2 of every XCD and cost more than this launch.
__global__ void __launch_bounds__(WAVE)
decode_attention_merge(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                       const int* __restrict__ rows, bf16_t* __restrict__ out, int n_q, int d, int splits,
                       const int* __restrict__ tiles, const int* __restrict__ cu_q) {
  HELD(part_o, part_ml, rows, out, n_q, d, splits, tiles);   // (the words that are there when a wave starts)
  const int item = blockIdx.x / n_q, head = blockIdx.x % n_q;
  int t = rows ? scalar_int(rows + item) : item;
  if (t < 0) return;
  if (tiles) {
    // Items are (tile, token of the tile): the output row is the tile's first row + the token; a tile's padding
    // has no row.
    const int tile = item >> 4, token = item & 15;
    const int entry = scalar_int(tiles + 2 * tile), row0 = scalar_int(cu_q + entry) + scalar_int(tiles + 2 * tile + 1);
    if (token >= scalar_int(cu_q + entry + 1) - row0) return;
    t = row0 + token;
  }
  const size_t base = ((size_t)item * n_q + head) * splits;
  const int lane = threadIdx.x, part = lane & 15, grp = lane >> 4;
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + base;
  constexpr int HELD = 8;                                    // splits a lane holds at once: 32 per round
  for (int e0 = 0; e0 < d; e0 += 64) {
    const int e = e0 + 4 * part;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    float big = -INFINITY, denom = 0.f;
    for (int s0 = 0; s0 < splits; s0 += 4 * HELD) {
      float4 v[HELD];
      float2 stat[HELD];
#pragma unroll
      for (int j = 0; j < HELD; ++j) {
        const int s = s0 + 4 * j + grp;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        stat[j] = make_float2(-INFINITY, 0.f);
        if (s < splits) {
          stat[j] = ml[s];
          if (e < d) v[j] = *reinterpret_cast<const float4*>(part_o + (base + s) * d + e);
        }
      }
      float round_big = big;
#pragma unroll
      for (int j = 0; j < HELD; ++j) round_big = fmaxf(round_big, stat[j].x);
      const float keep = (big == -INFINITY) ? 0.f : __expf(big - round_big);   // this lane's sums so far, rescaled
      o.x *= keep; o.y *= keep; o.z *= keep; o.w *= keep;
      denom *= keep;
      big = round_big;
#pragma unroll
      for (int j = 0; j < HELD; ++j) {
        const float w = (stat[j].x == -INFINITY) ? 0.f : __expf(stat[j].x - big);
        o.x += v[j].x * w; o.y += v[j].y * w; o.z += v[j].z * w; o.w += v[j].w * w;
        denom += stat[j].y * w;
      }
    }
    // The four lane groups hold sums over different splits under different maxima: bring them together.
    float all_big = fmaxf(big, __shfl_xor(big, 16, WAVE));
    all_big = fmaxf(all_big, __shfl_xor(all_big, 32, WAVE));
    const float w = (big == -INFINITY) ? 0.f : __expf(big - all_big);
    o.x *= w; o.y *= w; o.z *= w; o.w *= w;
    denom *= w;
#pragma unroll
    for (int shift = 16; shift <= 32; shift *= 2) {
      o.x += __shfl_xor(o.x, shift, WAVE); o.y += __shfl_xor(o.y, shift, WAVE);
      o.z += __shfl_xor(o.z, shift, WAVE); o.w += __shfl_xor(o.w, shift, WAVE);
      denom += __shfl_xor(denom, shift, WAVE);
    }
    if (grp == 0 && e < d) {
      const float inv = 1.0f / denom;
      bf16_t* dst = out + (size_t)t * n_q * d + (size_t)head * d + e;
      union { bf16x4 v; uint2 bits; } packed;
      packed.v[0] = (__bf16)(o.x * inv); packed.v[1] = (__bf16)(o.y * inv);
      packed.v[2] = (__bf16)(o.z * inv); packed.v[3] = (__bf16)(o.w * inv);
      *reinterpret_cast<uint2*>(dst) = packed.bits;
    }
  }
}

template <int D>
static int launch_decode(const void* q, int q_stride, void* out, const void* k_pages, const void* vt_pages,
                         const void* rows, const void* positions, const void* entry_of_token,
                         const void* block_table, int table_stride, void* part_o, void* part_ml, int n_items,
                         int n_q, int n_kv, int page_size, int window, float scale, int split_keys, int splits,
                         hipStream_t stream) {
  const int group = n_q / n_kv;
  dim3 grid(splits, n_kv * ((group + 15) / 16), n_items);
  constexpr int NW = D > 128 ? 2 : 4;   // keeps the merge buffer within 64 KB of LDS
#define GO(AHEAD) decode_attention_kernel<D, NW, AHEAD><<<grid, NW * WAVE, 0, stream>>>( \
      (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)vt_pages, (const int*)rows, \
      (const int*)positions, (const int*)entry_of_token, (const int*)block_table, table_stride, (float*)part_o, \
      (float*)part_ml, n_q, n_kv, page_size, window, scale, split_keys, splits)
  if (split_keys <= 32 * NW * 8) GO(true); else GO(false);      // up to eight blocks a wave
#undef GO
  int status = LAUNCH_STATUS();
  if (status == 0 && splits > 1) {
    decode_attention_merge<<<n_items * n_q, 64, 0, stream>>>((const float*)part_o, (const float*)part_ml,
                                                             (const int*)rows, (bf16_t*)out, n_q, D, splits,
                                                             nullptr, nullptr);
    status = LAUNCH_STATUS();
  }
  return status;
}

// The same merge for the prompt kernel whose tiles' keys were cut over workgroups: items are (tile, token of the
// tile), part_o float [n_tiles * 16, n_q, splits, d], part_ml float [n_tiles * 16, n_q, splits, 2].
extern "C" int ta_attention_merge_tiles(const void* part_o, const void* part_ml, const void* tiles, int n_tiles,
                                        const void* cu_q, void* out, int n_q, int d, int splits, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if ((long)n_tiles * 16 * n_q > 0x7fffffffL || d % 4 || splits < 1) return -1;
  decode_attention_merge<<<n_tiles * 16 * n_q, 64, 0, stream>>>((const float*)part_o, (const float*)part_ml, nullptr,
                                                                (bf16_t*)out, n_q, d, splits, (const int*)tiles,
                                                                (const int*)cu_q);
  return LAUNCH_STATUS();
}

// Returns -2 for a head size this kernel has no instance for (the caller then uses the generic kernel).
extern "C" int ta_decode_attention_bf16(const void* q, int q_stride, void* out, const void* k_pages,
                                        const void* vt_pages, const void* rows, const void* positions,
                                        const void* entry_of_token, const void* block_table, int table_stride,
                                        void* part_o, void* part_ml, int n_items, int n_q, int n_kv, int d,
                                        int page_size, int window, float scale, int split_keys, int splits,
                                        hipStream_t stream) {
  if (n_items <= 0) return 0;
  if (n_kv <= 0 || n_q % n_kv || page_size % 16 || split_keys % 32 || splits < 1) return -1;
#define CASE(DD) case DD: return launch_decode<DD>(q, q_stride, out, k_pages, vt_pages, rows, positions, entry_of_token, \
    block_table, table_stride, part_o, part_ml, n_items, n_q, n_kv, page_size, window, scale, split_keys, splits, stream);
  switch (d) {
    CASE(16) CASE(32) CASE(48) CASE(64) CASE(80) CASE(96) CASE(112) CASE(128) CASE(160) CASE(192) CASE(224) CASE(256)
    default: return -2;
  }
#undef CASE
}
