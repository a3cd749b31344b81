// C[M,N] = A[M,K] * W[N,K]^T (+ bias) for few rows (M <= 64): the decode-time product, bound by the
// one pass over the weights.  Computed transposed on the matrix cores, C^T = W A^T: sixteen weight rows are
// the M side of a 16x16x32 MFMA, up to four blocks of sixteen activation rows the N side, so every weight
// element is loaded once, 16 bytes per lane.  The waves of a workgroup split K between them and add up
// through LDS.  With GATED the kernel computes silu(A Wg^T) * (A Wu^T) for W = [Wg; Wu] in one pass.
#include "common.h"
#include "splitk_reduce.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 load8(const bf16_t* p, bool ok) {
  bf16x8 z;
  if (ok) return *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ void store4(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float* v) {
  uint2 packed;
  packed.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
  packed.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = packed;
}
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// grid.x: tiles of 16 output columns (of N, or of N/2 with GATED).  NW waves per workgroup.
// grid.y: parts of K of `k_chunk` elements (a multiple of 32) each: with more than one, a workgroup writes the
// float sums of its part into its slab of `partial` [parts, M, N] and `splitk_reduce` finishes the product.  That is
// for few output tiles and a long K (the down projection of a decode batch): every compute unit gets a share.
//
// ROPE (with GATED's two sets of weight rows): the product is the joined q/k/v projection.  A tile is sixteen
// elements of the first half of a head and the sixteen half a head further on, which the half-split rotation
// pairs; the epilogue adds the bias, rotates query and key heads by the row's position and writes queries to
// C [M, n_q * d], keys and values into their pages (values transposed inside a page).
struct RopeStore {
  const int* positions; const float* cos_sin; const int* slots;
  bf16_t* k_pages; bf16_t* v_pages;
  int n_q, n_kv, d, page_size;
};

// NB: blocks of sixteen output columns per workgroup.  Every workgroup reads all the rows of A for its part of K;
// with two blocks the rows are read half as often, which is what a product of many rows is bound by once the
// rows outweigh a tile's weights (what comes over the fabric from the caches counts like what comes from memory).
// LINES: the weights are read line by line (`lines_to_rows` in common.h), K walked in steps of 64; for products that
// are one long stream over a big matrix.
template <int MB, int NW, bool GATED, typename OutT, bool ROPE = false, int NB = 1, bool LINES = false>
__global__ void __launch_bounds__(NW * WAVE)
skinny_gemm_kernel(const bf16_t* __restrict__ A, int lda, int k_chunk, const bf16_t* __restrict__ W,
                   OutT* __restrict__ C, int ldc, int M, int N, int K_all, float* __restrict__ partial,
                   const float* __restrict__ bias, const RopeStore rope = RopeStore()) {
  // (What the walk over K needs stands in the first fourteen words of the arguments, which are in scalar registers
  // when a wave starts; the bias and the rotation's arguments, which the epilogue needs, lie behind.)
  HELD(A, lda, k_chunk, W, C, ldc, M, N, K_all, partial);
  static_assert(!ROPE || GATED, "the rotation uses the two sets of weight rows");
  static_assert(!ROPE || NB == 1, "the rotation pairs rows within one block");
  constexpr int HALVES = GATED ? 2 : 1;                     // gate and up rows (or the two halves of a head)
  constexpr int SETS = HALVES * NB;                         // set h * NB + b: half h, column block b
  __shared__ float red[NW][HALVES * MB * 4][WAVE];
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int col = lane & 15, g = lane >> 4;
  const int n_out = ROPE ? N : GATED ? N / 2 : N;
  // ROPE: tile t is block t % (d/32) of sixteen elements in the first half of head t / (d/32).
  const int rope_half = ROPE ? rope.d / 2 : 0;
  const int rope_head = ROPE ? blockIdx.x / (rope_half / 16) : 0;
  const int rope_first = ROPE ? (blockIdx.x % (rope_half / 16)) * 16 : 0;      // first element of the tile in its head
  const int n_first = ROPE ? rope_head * rope.d + rope_first : blockIdx.x * 16 * NB;
  const int k_lo = blockIdx.y * k_chunk;
  const int K = min(K_all, k_lo + k_chunk) - k_lo;                // this workgroup's part of K
  // grid.z: the rows in shares of MB blocks of sixteen (one share unless the launcher cut them: a small matrix
  // whose tiles would not fill the device otherwise; the weights are then read once per share).
  const int m_base = blockIdx.z * (MB * 16);
  // Rows past the end are clamped, not masked: they only feed outputs that are never stored.
  // The second half: the `up` rows when GATED, the rows half a head further on with ROPE.
  const bf16_t* wp[SETS];
#pragma unroll
  for (int h = 0; h < HALVES; ++h)
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int wrow = min(n_first + 16 * b + col, n_out - 1) + h * (ROPE ? rope_half : n_out);
      wp[h * NB + b] = W + (size_t)wrow * K_all + k_lo + 8 * g;
    }
  // Lanes of activation rows past M load nothing and hold zeros: a load costs the memory pipeline by its
  // active lanes, and with few rows most of a block's lanes are such.
  const bf16_t* a_row[MB];
  bool a_ok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    a_ok[mb] = m_base + mb * 16 + col < M;
    a_row[mb] = A + (size_t)min(m_base + mb * 16 + col, M - 1) * lda + k_lo + 8 * g;
  }

  floatx4 acc[SETS][MB];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[s][mb] = (floatx4){0.f, 0.f, 0.f, 0.f};

  constexpr int UN = (SETS * MB > 4) ? 2 : 4;
  if constexpr (LINES) {
    const int sub = col & 7, piece = 2 * g + (col >> 3);
    const bool low_lane = col < 8;
    const bf16_t* wl[SETS][2];
#pragma unroll
    for (int h = 0; h < HALVES; ++h)
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          const int wrow = min(n_first + 16 * b + 8 * hh + sub, n_out - 1) + h * (ROPE ? rope_half : n_out);
          wl[h * NB + b][hh] = W + (size_t)wrow * K_all + k_lo + 8 * piece;
        }
    const int pairs = (K + 63) / 64;                        // lines of a row; the last may be short
    constexpr int UP = UN / 2;
    for (int first = wave; first < pairs; first += UP * NW) {
      word4 wf[UP][SETS][2];
      bf16x8 af[UP][MB][2];
#pragma unroll
      for (int q = 0; q < UP; ++q) {
        const int pair = first + q * NW;
        const bool valid = pair < pairs;
        const int at = min(pair, pairs - 1) * 64;
        const bool mine = valid && at + 8 * piece < K;        // this lane's sixteen bytes lie inside K
#pragma unroll
        for (int s = 0; s < SETS; ++s)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) {
            wf[q][s][hh] = (word4){0u, 0u, 0u, 0u};
            if (mine) wf[q][s][hh] = *reinterpret_cast<const word4*>(wl[s][hh] + at);
          }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {          // the rows' sixteen bytes 2 g and 2 g + 1 of the line: what the weights' are after the exchange
          af[q][mb][0] = load8(a_row[mb] + at + 8 * g, valid && a_ok[mb] && at + 16 * g < K);
          af[q][mb][1] = load8(a_row[mb] + at + 8 * g + 8, valid && a_ok[mb] && at + 16 * g + 8 < K);
        }
      }
#pragma unroll
      for (int q = 0; q < UP; ++q) {
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
          bf16x8 b0, b1;
          lines_to_rows(wf[q][s][0], wf[q][s][1], low_lane, b0, b1);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            acc[s][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b0, af[q][mb][0], acc[s][mb], 0, 0, 0);
            acc[s][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b1, af[q][mb][1], acc[s][mb], 0, 0, 0);
          }
        }
      }
    }
  } else {
  const int full_steps = K / 32;
  // UN steps at a time, all loads first, so that many are in flight per lane.  A wave's last batch may reach
  // past the end of K: such steps load nothing and multiply zeros (no matrix instruction sits behind a
  // condition), so that a wave's share of K is as few trips to memory as can be, never one trip per step.
  for (int ks = wave; ks < full_steps; ks += UN * NW) {
    bf16x8 wf[UN][SETS], af[UN][MB];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int step = ks + u * NW;
      const bool valid = step < full_steps;
      const int k = min(step, full_steps - 1) * 32;
#pragma unroll
      for (int s = 0; s < SETS; ++s) wf[u][s] = load8(wp[s] + k, valid);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) af[u][mb] = load8(a_row[mb] + k, valid && a_ok[mb]);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int s = 0; s < SETS; ++s)
          acc[s][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][s], af[u][mb], acc[s][mb], 0, 0, 0);
  }
  if (K & 31) {
    // The tail of K (a multiple of 8), zero-filled, is one wave's; the others multiply zeros, so that no matrix
    // instruction sits behind a condition on the wave (it would run whatever a lane mask says).
    const int k = full_steps * 32;
    const bool k_ok = wave == full_steps % NW && k + 8 * g < K;
    bf16x8 wt[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) wt[s] = load8(wp[s] + k, k_ok);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const bf16x8 af = load8(a_row[mb] + k, k_ok && a_ok[mb]);
#pragma unroll
      for (int s = 0; s < SETS; ++s) acc[s][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wt[s], af, acc[s][mb], 0, 0, 0);
    }
  }
  }
  // One column block at a time through LDS (both halves of it), so that more blocks need no more LDS.
#pragma unroll
  for (int b = 0; b < NB; ++b) {
  const int n0 = n_first + 16 * b;
  if (b > 0) __syncthreads();                                   // the block before has been read
#pragma unroll
  for (int h = 0; h < HALVES; ++h)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][(h * MB + mb) * 4 + r][lane] = acc[h * NB + b][mb][r];
  __syncthreads();
  // Lane (col, g) of block mb holds C^T rows n0 + 4g + r (r = 0..3), column m = mb*16 + col.
  for (int item = threadIdx.x; item < MB * WAVE; item += NW * WAVE) {
    const int mb = item / WAVE, ln = item % WAVE;
    const int m = m_base + mb * 16 + (ln & 15);
    const int n = n0 + 4 * (ln >> 4);
    if (m >= M || n >= n_out) continue;
    float v[4], v2[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        sum0 += red[w][mb * 4 + r][ln];
        if (GATED) sum1 += red[w][(MB + mb) * 4 + r][ln];
      }
      if (ROPE) {
        v[r] = sum0 + (bias ? bias[n + r] : 0.f);
        v2[r] = sum1 + (bias ? bias[n + rope_half + r] : 0.f);
        continue;
      }
      if (bias && !partial && n + r < n_out) sum0 += bias[n + r];
      v[r] = GATED ? sum0 / (1.0f + __expf(-sum0)) * sum1 : sum0;
    }
    if constexpr (ROPE) {
      const int d = rope.d, i = rope_first + 4 * (ln >> 4);          // elements i..i+3 of the head, and i + half
      if (rope_head < rope.n_q + rope.n_kv && rope.cos_sin) {
        const float* cs = rope.cos_sin + (size_t)rope.positions[m] * d;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float c = cs[i + r], sn = cs[rope_half + i + r], x1 = v[r], x2 = v2[r];
          v[r] = x1 * c - x2 * sn;
          v2[r] = x2 * c + x1 * sn;
        }
      }
      if (rope_head < rope.n_q) {
        bf16_t* dst = reinterpret_cast<bf16_t*>(C) + (size_t)m * ldc + (size_t)rope_head * d + i;
        store4(dst, v);
        store4(dst + rope_half, v2);
        continue;
      }
      const int slot = rope.slots ? rope.slots[m] : -1;
      if (slot < 0) continue;                                     // this row's keys and values are not stored
      const int page = slot / rope.page_size, off = slot % rope.page_size;
      if (rope_head < rope.n_q + rope.n_kv) {
        bf16_t* dst = rope.k_pages + (((size_t)page * rope.n_kv + (rope_head - rope.n_q)) * rope.page_size + off) * d + i;
        store4(dst, v);
        store4(dst + rope_half, v2);
      } else {
        bf16_t* dst = rope.v_pages + (((size_t)page * rope.n_kv + (rope_head - rope.n_q - rope.n_kv)) * d + i) * rope.page_size + off;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          store1(dst + (size_t)r * rope.page_size, v[r]);
          store1(dst + (size_t)(rope_half + r) * rope.page_size, v2[r]);
        }
      }
      continue;
    }
    if (partial) {                                              // (never GATED; N is a multiple of 4)
      store4(partial + ((size_t)blockIdx.y * M + m) * n_out + n, v);
      continue;
    }
    OutT* dst = C + (size_t)m * ldc + n;
    if (n + 3 < n_out && (ldc & 3) == 0) {
      store4(dst, v);
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < n_out) store1(dst + r, v[r]);
    }
  }
  }
}

// Column blocks per workgroup, by the launcher's choice (`asked` 0) or the caller's (1 or 2): two once there are
// more than 32 rows and the workgroups still fill the device.
static int column_blocks(int asked, int M, int n_out, int splits) {
  if (asked == 1 || asked == 2) return asked;
  return (M > 32 && (long)((n_out + 31) / 32) * splits >= 128) ? 2 : 1;
}

static int g_lines = 1;        // whether the long streams read their weights line by line (tests and measurements switch it)
extern "C" void ta_skinny_lines(int on) { g_lines = on; }

template <int MB, int NW, bool GATED, int NB = 1, bool LINES = false>
static int launch_skinny(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int M, int N,
                         int K, int out_dtype, hipStream_t stream, int splits = 1, void* partial = nullptr) {
  const int n_out = GATED ? N / 2 : N;
  const int k_chunk = splits > 1 ? ((K + splits - 1) / splits + 31) / 32 * 32 : K;
  if (splits > 1) splits = (K + k_chunk - 1) / k_chunk;          // no part without a step of its own
  const dim3 grid((n_out + 16 * NB - 1) / (16 * NB), splits);
  float* slabs = splits > 1 ? (float*)partial : nullptr;
  if (out_dtype == DT_F32)
    skinny_gemm_kernel<MB, NW, GATED, float, false, NB, LINES><<<grid, NW * WAVE, 0, stream>>>(
        (const bf16_t*)A, lda, k_chunk, (const bf16_t*)W, (float*)C, ldc, M, N, K, slabs, (const float*)bias);
  else
    skinny_gemm_kernel<MB, NW, GATED, bf16_t, false, NB, LINES><<<grid, NW * WAVE, 0, stream>>>(
        (const bf16_t*)A, lda, k_chunk, (const bf16_t*)W, (bf16_t*)C, ldc, M, N, K, slabs, (const float*)bias);
  int status = LAUNCH_STATUS();
  if (status == 0 && splits > 1 && C) status = launch_splitk_reduce(slabs, bias, C, M, N, ldc, splits, out_dtype, stream);
  return status;
}

template <int MB, bool GATED>
static int pick_waves(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int M, int N,
                      int K, int out_dtype, hipStream_t stream, int col_blocks = 0) {
  if constexpr (MB >= 3) {
    if (column_blocks(col_blocks, M, GATED ? N / 2 : N, 1) == 2)
      return launch_skinny<MB, 8, GATED, 2>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
  }
  if constexpr (MB == 1 && !GATED) {
    // Up to sixteen rows against tens of thousands of output columns (the vocabulary projection of a decode
    // step): four column blocks per workgroup, or a quarter of the workgroups would each read all the rows again.
    if ((col_blocks == 0 || col_blocks == 4) && (N + 15) / 16 >= 4096 && K <= 8192) {
      // The one long stream of a decode step: its weights are read line by line (0.5B sizes, 8 rows: 61.7 -> 55.7 us;
      // 7B sizes: 229 -> 201 us, 16 rows 248 -> 211 us).
      if (g_lines) return launch_skinny<1, 4, false, 4, true>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
      return launch_skinny<1, 4, false, 4>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
    }
  }
  // Few output tiles and a long K: more waves per tile, so that enough loads are in flight.
  const int tiles = ((GATED ? N / 2 : N) + 15) / 16;
  const int k_steps = (K + 31) / 32;
  if (tiles >= 1024 || k_steps <= 8)
    return launch_skinny<MB, 4, GATED>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
  if (tiles >= 256 || k_steps <= 32 || MB * (GATED ? 2 : 1) > 2)
    return launch_skinny<MB, 8, GATED>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
  return launch_skinny<MB, 16, GATED>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream);
}

// M <= 64; K, lda multiples of 8; pointers 16-byte aligned; with `gated` N is even and C is [M, N/2].
// col_blocks: blocks of sixteen output columns per workgroup, 0 = the launcher's choice (see column_blocks).
extern "C" int ta_gemm_skinny_bf16(const void* A, int lda, const void* W, const void* bias, void* C, int ldc,
                                   int M, int N, int K, int out_dtype, int gated, int col_blocks, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || (K & 7) || (lda & 7) || (gated && (N & 1))) return -1;
  const int mb = (M + 15) / 16;
#define GO(MBV) (gated ? pick_waves<MBV, true>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream, col_blocks) \
                       : pick_waves<MBV, false>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream, col_blocks))
  switch (mb) {
    case 1: return GO(1);
    case 2: return GO(2);
    case 3: return GO(3);
    default: return GO(4);
  }
#undef GO
}

// The same product (not gated) with K cut into `splits` parts (at most; parts are multiples of 32) over the
// workgroups, the parts' float sums added afterwards in a fixed order.  partial: room for splits * M * N floats;
// N % 4 == 0; M <= 64.  With C null (and more than one part after the rounding of the parts' length) the sums are
// left in `partial` for a later kernel to add.
extern "C" int ta_gemm_skinny_bf16_splitk(const void* A, int lda, const void* W, const void* bias, void* C, int ldc,
                                          void* partial, int M, int N, int K, int out_dtype, int splits,
                                          int col_blocks, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || (K & 7) || (lda & 7) || (N & 3) || splits < 1 || (splits > 1 && !partial)) return -1;
  if (!C && parts_of_k(K, splits, 32) < 2) return -1;
#define GO(MBV, NBV) launch_skinny<MBV, 8, false, NBV>(A, lda, W, bias, C, ldc, M, N, K, out_dtype, stream, splits, partial)
  const bool two = column_blocks(col_blocks, M, N, parts_of_k(K, splits, 32)) == 2;
  switch ((M + 15) / 16) {
    case 1: return GO(1, 1);
    case 2: return GO(2, 1);
    case 3: return two ? GO(3, 2) : GO(3, 1);
    default: return two ? GO(4, 2) : GO(4, 1);
  }
#undef GO
}

// The joined q/k/v projection of 17 to 64 rows with bias, rotation and the cache write in its epilogue (see
// RopeStore): x bfloat16 [M, K] (row stride lda), W [(n_q + 2 n_kv) d, K], bias float32 or null; queries go to
// q_out [M, n_q d]; cos_sin float32 [positions, d] or null (no rotation); slots int32 [M] or null (nothing is
// stored; a negative slot skips its row).  d a multiple of 32.
extern "C" int ta_gemm_skinny_qkv_rope(const void* x, int lda, const void* W, const void* bias, void* q_out,
                                       const void* positions, const void* cos_sin, const void* slots, void* k_pages,
                                       void* v_pages, int M, int K, int n_q, int n_kv, int d, int page_size,
                                       hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 64 || (K & 7) || (lda & 7) || (d & 31) || n_q <= 0 || n_kv <= 0 || page_size <= 0 || !positions) return -1;
  if (slots && (!k_pages || !v_pages)) return -1;
  RopeStore rope;
  rope.positions = (const int*)positions; rope.cos_sin = (const float*)cos_sin; rope.slots = (const int*)slots;
  rope.k_pages = (bf16_t*)k_pages; rope.v_pages = (bf16_t*)v_pages;
  rope.n_q = n_q; rope.n_kv = n_kv; rope.d = d; rope.page_size = page_size;
  const int N = (n_q + 2 * n_kv) * d;
  const int tiles = (n_q + 2 * n_kv) * (d / 32);
  const int blocks = (M + 15) / 16;
  // Few tiles (a small model's joined matrix is a few dozen): the blocks of sixteen rows are dealt to workgroups
  // of their own, as many shares as it takes to fill the device; every share reads the matrix again.
  const int shares = min(blocks, (compute_units() + tiles - 1) / tiles);
  const int per_share = (blocks + shares - 1) / shares;
  const dim3 grid(tiles, 1, (blocks + per_share - 1) / per_share);
#define GO(MBV) skinny_gemm_kernel<MBV, 8, true, bf16_t, true><<<grid, 8 * WAVE, 0, stream>>>( \
    (const bf16_t*)x, lda, K, (const bf16_t*)W, (bf16_t*)q_out, n_q * d, M, N, K, nullptr, (const float*)bias, rope)
  switch (per_share) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    default: GO(4); break;
  }
#undef GO
  return LAUNCH_STATUS();
}
