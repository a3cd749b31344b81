// Fused products for decode batches of up to 16 rows.  Each keeps the layout of the weight-streaming kernel
// (C^T = W A^T on 16x16x32 MFMAs, the waves of a workgroup split K and add up through LDS) and folds the
// neighbouring small kernels into its prologue or epilogue:
//   NORM prologue   the rows are read from the float residual stream and RMS-normalised on the fly into LDS
//                   (or, normalised already, copied there once: what a workgroup pulls in over the fabric from
//                   the caches counts like what it pulls from memory, and rows asked for again in every batch
//                   of weights would be half as many bytes again as the weights)
//   ROPE_STORE      q/k/v projection: bias, half-split rotation, keys and values written into their pages
//   GATED           silu(gate) * up
//   RESIDUAL        the product is added into the float residual stream in place
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

enum { EPI_ROPE_STORE = 0, EPI_GATED = 1, EPI_RESIDUAL = 2 };

struct FusedArgs {
  // input rows: bfloat16 activations, or (with the NORM prologue) the float residual with norm weight and eps
  const bf16_t* a; int lda;
  const float* residual_in; const float* norm_weight; float eps;
  const bf16_t* w; const float* bias;
  int m, n, k;
  int rows;                                                // weight rows per workgroup
  // EPI_GATED / plain output (bfloat16 [m, ldc])
  bf16_t* out; int ldc;
  // EPI_RESIDUAL
  float* residual_out;
  // EPI_ROPE_STORE
  const int* positions; const float* cos_sin; const int* slots;
  bf16_t* k_pages; bf16_t* v_pages; int n_q, n_kv, d, page_size;
};

__device__ __forceinline__ bf16x8 fz8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}
// Registers with whatever they hold, for lanes whose load is left out and whose products are never stored (a row
// of the weights only feeds its own row of the result).  Zeros would do as well, but the compiler keeps one zero
// for many purposes, copies a loaded value over it, and waits for the load to do so, in the middle of a batch of
// loads: the batch then takes two trips to memory instead of one.
__device__ __forceinline__ bf16x8 any8() {
  bf16x8 v;
  asm volatile("" : "=v"(v));
  return v;
}

// A workgroup owns `p.rows` weight rows (output columns), in PASSES blocks of up to sixteen: the M side of the
// MFMA.  Lanes whose weight row or input row only feeds results that are never stored load nothing: a
// load costs the memory pipeline by its active lanes.  So a small matrix is spread thinly over many
// workgroups (4 rows each), and a large one is cut so that every compute unit streams the same share.
//
// UN: steps of 32 along K that a wave requests at once.  ONE: the host has checked that a wave's whole share
// of K is one such batch, so there is no loop, the batches of all passes are requested at the start, and a
// small matrix is over after one trip to memory instead of several.
//
// The arguments are all asked for at the kernel's start (`HELD`): left to itself the compiler fetches each piece
// of the argument block where it is first used, and a small kernel then begins with several trips to memory one
// after the other.  What the epilogue needs from memory is asked for before the weights where a second load hangs
// on a first one (the angle table's row on the position), and otherwise right after them and left alone until the
// epilogue: a value that is used early makes the wave wait for everything it asked for before, the weights included.
//
// The kernel takes its arguments one by one, those that every instance needs before its first load in the first
// sixteen words of the argument block: the library is compiled so that these are in scalar registers when a wave
// starts (`-amdgpu-kernarg-preload-count`; fourteen words in fact), and the products with the gated and the residual
// epilogue then begin without any fetch of arguments (the bias, which only the epilogue needs, lies behind).  One pointer serves for the rows (bfloat16, or the float residual for the norm
// prologue) and one for the result (bfloat16 rows, or the float residual that is added to), which never occur
// together.  The rotation's own arguments lie behind; only wave 0, which writes the results, waits for them.
template <int NW, int EPI, bool NORM, int UN, bool ONE, int PASSES>
__global__ void __launch_bounds__(NW * WAVE)
fused_decode_kernel(const bf16_t* w, const void* rows_in, void* result, const float* norm_weight,
                    int m, int n, int k, int rows, int lda, float eps, const float* bias,
                    const int* positions, const float* cos_sin, const int* slots, bf16_t* k_pages, bf16_t* v_pages,
                    int n_q, int n_kv, int d, int page_size) {
  HELD(w, rows_in, result, norm_weight, m, n, k, rows, lda, eps);          // (the fourteen words that are there)
  if constexpr (EPI == EPI_ROPE_STORE) HELD(n_q, n_kv, d, page_size);      // (where a tile's rows lie)
  FusedArgs p;
  // (Rows with a norm weight are the float residual; without one they are bfloat16, normalised already or plain.)
  p.a = norm_weight ? nullptr : (const bf16_t*)rows_in; p.lda = lda;
  p.residual_in = norm_weight ? (const float*)rows_in : nullptr; p.norm_weight = norm_weight; p.eps = eps;
  p.w = w; p.bias = bias; p.m = m; p.n = n; p.k = k; p.rows = rows;
  p.out = (bf16_t*)result; p.ldc = EPI == EPI_GATED ? n / 2 : n_q * d;
  p.residual_out = (float*)result;
  p.positions = positions; p.cos_sin = cos_sin; p.slots = slots; p.k_pages = k_pages; p.v_pages = v_pages;
  p.n_q = n_q; p.n_kv = n_kv; p.d = d; p.page_size = page_size;
  constexpr int SETS = (EPI == EPI_RESIDUAL) ? 1 : 2;
  constexpr int HELD = ONE ? PASSES : 1;                     // batches of weights held at once
  static_assert(EPI != EPI_ROPE_STORE || PASSES == 1, "the rotation pairs rows within one block");
  __shared__ float red[NW][SETS * 4][WAVE];
  extern __shared__ __attribute__((aligned(16))) uint16_t a_s[];   // NORM: the m normalised rows of K + 8 bfloat16
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int col = lane & 15, g = lane >> 4;
  const int M = p.m, K = p.k, R = p.rows;
  const int tile = blockIdx.x;

  // Which weight rows this workgroup owns: `row0` onwards (+ `row1` onwards for the second set).
  int row0, row1 = 0;
  bool paired = true;
  if (EPI == EPI_ROPE_STORE) {
    const int half = p.d / 2, per_half = half / R;
    const int n_pair_tiles = (p.n_q + p.n_kv) * per_half;
    if (tile < n_pair_tiles) {
      const int hd = tile / per_half, j = tile % per_half;
      row0 = hd * p.d + j * R;
      row1 = row0 + half;
    } else {
      paired = false;
      row0 = (p.n_q + p.n_kv) * p.d + (tile - n_pair_tiles) * R;
      row1 = row0;
    }
  } else if (EPI == EPI_GATED) {
    row0 = tile * R;
    row1 = row0 + p.n / 2;
  } else {
    row0 = tile * R;
  }
  const int n_limit = (EPI == EPI_GATED) ? p.n / 2 : p.n;
  const bf16_t* w0[PASSES];
  const bf16_t* w1[PASSES];
  bool w_lane[PASSES];
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps) {
    const int r = 16 * ps + col;
    w_lane[ps] = r < R && row0 + r < n_limit;
    w0[ps] = p.w + (size_t)min(row0 + r, n_limit - 1) * K + 8 * g;
    w1[ps] = p.w + (size_t)min(row1 + r, p.n - 1) * K + 8 * g;
  }
  const bool a_lane = col < M;
  const int a_m = min(col, M - 1);
  const int full_steps = K / 32;
  const int lds_stride = K + 8;

  // The rotation's angles hang on the row's position: that chain starts before anything else is asked for (wave 0
  // writes the results; lane (col, g) owns column m = col and rows 4g .. 4g+3 of each block).
  float pre_cos[4] = {1.f, 1.f, 1.f, 1.f}, pre_sin[4] = {0.f, 0.f, 0.f, 0.f};
  int pre_slot = -1;
  if (EPI == EPI_ROPE_STORE && wave == 0) HELD(bias, positions, cos_sin, slots, k_pages, v_pages);
  if (EPI == EPI_ROPE_STORE && wave == 0 && col < M && 4 * g < R) {
    pre_slot = p.slots ? p.slots[col] : -1;
    if (paired && p.cos_sin) {
      const float* cs = p.cos_sin + (size_t)p.positions[col] * p.d + row0 % p.d + 4 * g;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pre_cos[r] = cs[r];
        pre_sin[r] = cs[p.d / 2 + r];
      }
    }
  }

  // Weight fragments come from HBM and take longest; the first batch is requested before the prologue.
  // Step j of a wave's batch: steps come in pairs (128 contiguous bytes of a weight row, one cache line),
  // pair q of the batch starting at pair `base` is pair base + q * NW.
  auto step_of = [&](int base_pair, int u) { return (base_pair + (u >> 1) * NW) * 2 + (u & 1); };
  bf16x8 wf[HELD][UN][SETS];
  auto load_w = [&](int held, int ps, int base_pair) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int step = min(step_of(base_pair, u), max(full_steps - 1, 0));   // clamped loads are not used
      // (in the loop of the long walks the zeros stay: there the statement that leaves a register as it is would
      // stand between the loop's loads and products, which the compiler then no longer moves past each other)
      wf[held][u][0] = ONE ? any8() : fz8();
      if (SETS == 2) wf[held][u][SETS - 1] = ONE ? any8() : fz8();
      if (w_lane[ps]) {
        wf[held][u][0] = *reinterpret_cast<const bf16x8*>(w0[ps] + step * 32);
        if (SETS == 2) wf[held][u][SETS - 1] = *reinterpret_cast<const bf16x8*>(w1[ps] + step * 32);
      }
    }
  };
  load_w(0, 0, wave);
  if (ONE) {
#pragma unroll
    for (int ps = 1; ps < PASSES; ++ps) load_w(HELD - PASSES + ps, ps, wave);
  }
  const bf16_t* ar = NORM ? nullptr : p.a + (size_t)a_m * p.lda + 8 * g;
  bf16x8 af_one[ONE ? UN : 1];
  if (ONE && !NORM) {                                      // the rows' fragments as well
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      // (every lane: a row past the end repeats the last one and only feeds columns that are never stored)
      af_one[u] = *reinterpret_cast<const bf16x8*>(ar + min(step_of(wave, u), max(full_steps - 1, 0)) * 32);
    }
  }

  // What else the epilogue needs besides the sums is requested now as well, and not touched before the epilogue.
  float pre_a[PASSES][4], pre_b[PASSES][4];                  // the old residual and the bias; or the two halves' bias
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
    for (int r = 0; r < 4; ++r) pre_a[ps][r] = pre_b[ps][r] = 0.f;
  if (EPI == EPI_RESIDUAL && wave == 0) HELD(bias);
  if (wave == 0 && col < M) {
    if (EPI == EPI_RESIDUAL) {
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int local = 16 * ps + 4 * g + r, n = row0 + local;
          if (local < R && n < p.n) {
            pre_a[ps][r] = p.residual_out[(size_t)col * p.n + n];
            if (p.bias) pre_b[ps][r] = p.bias[n];
          }
        }
    } else if (EPI == EPI_ROPE_STORE && 4 * g < R && p.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r) { pre_a[0][r] = p.bias[row0 + 4 * g + r]; pre_b[0][r] = p.bias[row1 + 4 * g + r]; }
    }
  }

  if (NORM && !p.residual_in) {
    // Rows that are normalised already: copied into LDS once.
    for (int m = wave; m < M; m += NW) {
      const bf16_t* x = p.a + (size_t)m * p.lda;
      uint16_t* dst = a_s + (size_t)m * lds_stride;
      for (int k = lane * 8; k < K; k += WAVE * 8)
        *reinterpret_cast<uint4*>(dst + k) = *reinterpret_cast<const uint4*>(x + k);
    }
    __syncthreads();
  } else if (NORM) {
    // Each row once: 1 / sqrt(mean(x^2) + eps), then x * that * weight rounded to bfloat16 into LDS.
    for (int m = wave; m < M; m += NW) {
      const float* x = p.residual_in + (size_t)m * K;
      uint16_t* dst = a_s + (size_t)m * lds_stride;
      if (K <= 4 * WAVE * 4) {
        // The row fits in four float4 per lane: read it (and the norm weight) once and keep it in registers.
        float4 v[4], gw[4];
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int k = (i * WAVE + lane) * 4;
          v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
          gw[i] = v[i];
          if (k < K) {
            v[i] = *reinterpret_cast<const float4*>(x + k);          // K is a multiple of 8
            gw[i] = *reinterpret_cast<const float4*>(p.norm_weight + k);
          }
          sq += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
        }
        sq = wave_sum(sq);
        const float inv = 1.0f / sqrtf(sq / (float)K + p.eps);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int k = (i * WAVE + lane) * 4;
          if (k >= K) continue;
          union { bf16x4 v; uint2 bits; } packed;
          packed.v[0] = (__bf16)(v[i].x * inv * gw[i].x); packed.v[1] = (__bf16)(v[i].y * inv * gw[i].y);
          packed.v[2] = (__bf16)(v[i].z * inv * gw[i].z); packed.v[3] = (__bf16)(v[i].w * inv * gw[i].w);
          *reinterpret_cast<uint2*>(dst + k) = packed.bits;
        }
        continue;
      }
      float sq = 0.f;
      for (int k = lane * 4; k < K; k += WAVE * 4) {
        const float4 v = *reinterpret_cast<const float4*>(x + k);
        sq += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
      sq = wave_sum(sq);
      const float inv = 1.0f / sqrtf(sq / (float)K + p.eps);
      for (int k = lane * 4; k < K; k += WAVE * 4) {
        const float4 v = *reinterpret_cast<const float4*>(x + k);
        const float4 gw = *reinterpret_cast<const float4*>(p.norm_weight + k);
        union { bf16x4 v; uint2 bits; } packed;
        packed.v[0] = (__bf16)(v.x * inv * gw.x); packed.v[1] = (__bf16)(v.y * inv * gw.y);
        packed.v[2] = (__bf16)(v.z * inv * gw.z); packed.v[3] = (__bf16)(v.w * inv * gw.w);
        *reinterpret_cast<uint2*>(dst + k) = packed.bits;
      }
    }
    __syncthreads();
  }
  const uint16_t* as_row = a_s + (size_t)a_m * lds_stride + 8 * g;
  auto load_a = [&](int k) -> bf16x8 {
    if (NORM) return *reinterpret_cast<const bf16x8*>(as_row + k);
    return a_lane ? *reinterpret_cast<const bf16x8*>(ar + k) : fz8();
  };

#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps) {
    floatx4 acc[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) acc[s] = (floatx4){0.f, 0.f, 0.f, 0.f};
    if constexpr (ONE) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        // A step past the end of K is multiplied all the same, with zeros for the rows: no matrix instruction
        // sits behind a condition (it would run whatever a lane mask says, and whether the compiler masks
        // or branches here is its choice).  The weights of such a step were read from a clamped, valid place.
        const int step = step_of(wave, u);
        bf16x8 af = NORM ? load_a(min(step, max(full_steps - 1, 0)) * 32) : af_one[u];
        if (step >= full_steps) af = fz8();
#pragma unroll
        for (int s = 0; s < SETS; ++s)
          acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[HELD - PASSES + ps][u][s], af, acc[s], 0, 0, 0);
      }
    } else {
      // Batches of UN steps; the next batch's weights are requested before the current one is multiplied.
      for (int pair = wave; pair * 2 < full_steps; pair += (UN / 2) * NW) {
        bf16x8 wc[UN][SETS], af[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          wc[u][0] = wf[0][u][0];
          if (SETS == 2) wc[u][SETS - 1] = wf[0][u][SETS - 1];
          af[u] = load_a(min(step_of(pair, u), full_steps - 1) * 32);
          if (step_of(pair, u) >= full_steps) af[u] = fz8();      // past the end of K: zeros, see above
        }
        if ((pair + (UN / 2) * NW) * 2 < full_steps) load_w(0, ps, pair + (UN / 2) * NW);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
#pragma unroll
          for (int s = 0; s < SETS; ++s)
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[u][s], af[u], acc[s], 0, 0, 0);
        }
      }
      if (ps + 1 < PASSES) load_w(0, ps + 1, wave);          // the next block's first batch, before this one's sums
    }
    if (K & 31) {                                            // tail of K (a multiple of 8): zero-filled; wave 0's
      const int k = full_steps * 32;
      const bool ok = wave == 0 && k + 8 * g < K;
      const bf16x8 af = ok ? load_a(k) : fz8();
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ok ? *reinterpret_cast<const bf16x8*>(w0[ps] + k) : fz8(), af, acc[0], 0, 0, 0);
      if (SETS == 2)
        acc[SETS - 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ok ? *reinterpret_cast<const bf16x8*>(w1[ps] + k) : fz8(), af, acc[SETS - 1], 0, 0, 0);
    }
    if (ps > 0) __syncthreads();                             // wave 0 has read the block before
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][s * 4 + r][lane] = acc[s][r];
    __syncthreads();
    // Lane (col, g) of wave 0: output column m = col, rows 4g .. 4g+3 of the block.
    const int m = col;
    if (wave == 0 && m < M && 16 * ps + 4 * g < R) {
      float v0[4], v1[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
          s0 += red[w][r][lane];
          if (SETS == 2) s1 += red[w][4 + r][lane];
        }
        v0[r] = s0;
        v1[r] = s1;
      }
      const int local = 16 * ps + 4 * g;                      // first of this lane's rows within the workgroup's
      if (EPI == EPI_RESIDUAL) {
        const int n = row0 + local;
        float* dst = p.residual_out + (size_t)m * p.n + n;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (local + r < R && n + r < p.n) dst[r] = (pre_a[ps][r] + pre_b[ps][r]) + v0[r];   // old residual (+ bias) from the start
      } else if (EPI == EPI_GATED) {
        const int n = row0 + local;
        bf16_t* dst = p.out + (size_t)m * p.ldc + n;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (local + r < R && n + r < n_limit) st(dst + r, v0[r] / (1.0f + __expf(-v0[r])) * v1[r]);
      } else {
        const int d = p.d, half = d / 2;
        const int slot = pre_slot;
        const int page = slot >= 0 ? slot / p.page_size : 0, off = slot >= 0 ? slot % p.page_size : 0;
        if (paired) {
          const int hd = row0 / d, i = row0 % d + 4 * g;            // element i (< half) of head hd, and i + half
          float r1[4], r2[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x1 = v0[r] + pre_a[0][r], x2 = v1[r] + pre_b[0][r];
            r1[r] = x1 * pre_cos[r] - x2 * pre_sin[r];              // cos 1, sin 0 without a rotation
            r2[r] = x2 * pre_cos[r] + x1 * pre_sin[r];
          }
          bf16_t* dst = nullptr;
          if (hd < p.n_q) dst = p.out + (size_t)m * p.ldc + (size_t)hd * d + i;
          else if (slot >= 0) dst = p.k_pages + (((size_t)page * p.n_kv + (hd - p.n_q)) * p.page_size + off) * d + i;
          if (dst) {
#pragma unroll
            for (int r = 0; r < 4; ++r) { st(dst + r, r1[r]); st(dst + half + r, r2[r]); }
          }
        } else if (slot >= 0) {
          const int e = row0 - (p.n_q + p.n_kv) * d + 4 * g;        // element of the joined value heads
          const int kvh = e / d, dd = e % d;
          bf16_t* dst = p.v_pages + (((size_t)page * p.n_kv + kvh) * d + dd) * p.page_size + off;
#pragma unroll
          for (int r = 0; r < 4; ++r) st(dst + (size_t)r * p.page_size, v0[r] + pre_a[0][r]);
        }
      }
    }
  }
}

template <int NW, int EPI, bool NORM, int UN, bool ONE, int PASSES>
static int launch_kernel(const FusedArgs& args, int tiles, hipStream_t stream) {
  size_t lds = NORM ? (size_t)args.m * (args.k + 8) * sizeof(uint16_t) : 0;
  if (lds > 48 * 1024) {
    // More dynamic LDS than the default limit: ask for it (the device has 160 KB per compute unit).
    if (lds > 140 * 1024) return -1;
    hipError_t err = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&fused_decode_kernel<NW, EPI, NORM, UN, ONE, PASSES>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return (int)err;
  }
  // The kernel tells the float residual from bfloat16 rows by whether there is a norm weight.
  const bool from_residual = args.residual_in != nullptr;
  if (from_residual != (args.norm_weight != nullptr) || (!from_residual && !args.a) || !args.w) return -1;
  if (EPI == EPI_RESIDUAL ? !args.residual_out : !args.out) return -1;
  fused_decode_kernel<NW, EPI, NORM, UN, ONE, PASSES><<<tiles, NW * WAVE, lds, stream>>>(
      args.w, from_residual ? (const void*)args.residual_in : (const void*)args.a,
      EPI == EPI_RESIDUAL ? (void*)args.residual_out : (void*)args.out, args.norm_weight, args.m, args.n,
      args.k, args.rows, args.lda, args.eps, args.bias, args.positions, args.cos_sin, args.slots, args.k_pages, args.v_pages,
      args.n_q, args.n_kv, args.d, args.page_size);
  return LAUNCH_STATUS();
}

template <int NW, int EPI, bool NORM, int PASSES>
static int launch_one(const FusedArgs& args, int tiles, hipStream_t stream) {
  // Steps of a wave: pairs of steps are dealt round-robin to the waves.
  const int pairs = (args.k / 32 + 1) / 2;
  const int steps_per_wave = 2 * ((pairs + NW - 1) / NW);
  if (steps_per_wave <= 4) return launch_kernel<NW, EPI, NORM, 4, true, PASSES>(args, tiles, stream);
  if constexpr (NORM && (EPI == EPI_ROPE_STORE || PASSES == 1)) {
    // Rows in LDS: only the weights take registers, and a wave's whole share of up to eight steps is one trip
    // (rows of 1,025 to 2,048 elements at eight waves: two trips in the loop below; q/k/v at 1,536: 8.4 -> 7.5 us).
    // The gated product's matrix is several workgroups for every compute unit: it takes a whole share at once only
    // while two workgroups' registers fit a unit together, which is one block of rows and six steps (with two blocks
    // of rows 19.9 -> 22.3 us at 8,960 x 1,536, with eight steps 25.4 -> 31.3 us at 11,008 x 2,048).
    if (steps_per_wave <= 6) return launch_kernel<NW, EPI, NORM, 6, true, PASSES>(args, tiles, stream);
    if constexpr (EPI == EPI_ROPE_STORE)
      if (steps_per_wave <= 8) return launch_kernel<NW, EPI, NORM, 8, true, PASSES>(args, tiles, stream);
  }
  if constexpr (!NORM && PASSES == 1) {
    // Rows from memory: one trip for a wave's whole share if it fits the registers (128 a lane at 16 waves).
    if (steps_per_wave <= 8) return launch_kernel<NW, EPI, NORM, 8, true, 1>(args, tiles, stream);
    if (steps_per_wave <= 10) return launch_kernel<NW, EPI, NORM, 10, true, 1>(args, tiles, stream);
  }
  return launch_kernel<NW, EPI, NORM, 4, false, PASSES>(args, tiles, stream);
}

// waves 0: the launcher's choice of how many waves share a workgroup's K.
template <int EPI, bool NORM>
static int launch_rows(const FusedArgs& args, int tiles, int waves, hipStream_t stream) {
  const int k_steps = (args.k + 31) / 32;
  const bool two = args.rows > 16;
  if (waves == 0) waves = (tiles >= 1024 || k_steps <= 8) ? 4 : (tiles >= 256 || k_steps <= 64 || NORM || two) ? 8 : 16;
  if (EPI != EPI_RESIDUAL && waves > 8) waves = 8;           // two sets of weight registers: no room at 16 waves
  if constexpr (EPI != EPI_ROPE_STORE) {
    if (two) {
      if (waves == 4) return launch_one<4, EPI, NORM, 2>(args, tiles, stream);
      return launch_one<8, EPI, NORM, 2>(args, tiles, stream);
    }
  }
  if (waves == 4) return launch_one<4, EPI, NORM, 1>(args, tiles, stream);
  if (waves == 8 || NORM) return launch_one<8, EPI, NORM, 1>(args, tiles, stream);
  if constexpr (EPI == EPI_RESIDUAL) return launch_one<16, EPI, false, 1>(args, tiles, stream);
  return -1;
}

// Weight rows per workgroup for the rotation epilogue, where a block pairs rows half a head apart: 16, 8 or 4.
// Every workgroup reads and normalises all m input rows before its share of the weights, so the choice weighs
// the bytes the busiest compute unit has to ask for: rounds of workgroups x (prologue + its weight rows + what a
// unit could have streamed during the trips to memory that every workgroup begins with; without that last term one
// row of 3,584 took three rounds of four weight rows, 17.7 us, where one round of sixteen takes 14.0).
static int rows_per_tile(int n_q, int n_kv, int d, int m, int k, bool norm, int rows_override) {
  if (rows_override == 16 || rows_override == 8 || rows_override == 4) return rows_override;
  const long units = compute_units();
  const long prologue = (long)m * k * (norm ? 8 : 2);       // float rows and the norm weight per row, or bfloat16 rows
  int best = 16;
  long best_cost = -1;
  for (int r = 16; r >= 4; r /= 2) {
    const long tiles = (long)(n_q + n_kv) * (d / 2 / r) + (long)n_kv * d / r;
    const long cost = ((tiles + units - 1) / units) * (prologue + 2L * r * k * 2 + 64 * 1024);
    if (best_cost < 0 || cost < best_cost) { best = r; best_cost = cost; }
  }
  return best;
}

// Weight rows per workgroup elsewhere: the matrix is cut into a multiple of the compute units' number of
// equal shares of at most 32 rows, so that every unit streams the same number of bytes; never fewer than 4.
static int rows_per_workgroup(int n_rows, int rows_override) {
  if (rows_override >= 1 && rows_override <= 32) return rows_override;
  const int units = compute_units();
  const int rounds = (n_rows + units * 32 - 1) / (units * 32);
  int rows = (n_rows + units * rounds - 1) / (units * rounds);
  // One round of 17 to 31 rows would be a block of sixteen and a nearly empty second one, one after the other:
  // two workgroups of half the rows on every compute unit, one block each, are over sooner (measured at 4,864
  // rows of 896: 19 rows 8.6 us, 10 rows 8.2 us; with two rounds, 8,960 rows of 1,536, the halves are slower).
  if (rounds == 1 && rows > 16 && rows < 32) rows = (n_rows + 2 * units - 1) / (2 * units);
  return rows < 4 ? 4 : rows;
}

// The gated product from rows in LDS: where the even shares would be two blocks of rows a workgroup (17 to 32) and
// a wave's share of K at eight waves is at most six steps, workgroups of one block whose weights are asked for at
// once are over sooner: as many rounds of workgroups as blocks of sixteen need, in equal shares (8,960 rows of 1,536:
// 18 rows in two blocks 19.9 us, 12 rows 19.3 us at eight input rows; 18.3 and 17.3 us at one).  Up to eight input
// rows: every workgroup brings all of them in first, and half as many workgroups again weigh more than they save
// at sixteen (22.9 and 24.8 us).
static int rows_per_gated_workgroup(int n_rows, int m, int k, int rows_override) {
  int rows = rows_per_workgroup(n_rows, rows_override);
  if (rows_override >= 1 && rows_override <= 32) return rows;
  const int pairs = (k / 32 + 1) / 2;
  if (rows > 16 && m <= 8 && 2 * ((pairs + 7) / 8) <= 6) {
    const int units = compute_units();
    const int rounds = (n_rows + units * 16 - 1) / (units * 16);
    rows = (n_rows + units * rounds - 1) / (units * rounds);
  }
  return rows;
}

// Rows that are normalised already go through LDS (the NORM instances, which then copy instead of normalising)
// while a workgroup's copy fits a compute unit beside its other LDS (measured at a width of 3,584: 1.06x for 8
// rows, where two workgroups' copies fit, level for 12, 1.02x for 16).
static bool stage_rows(int m, int k) { return (size_t)m * (k + 8) * sizeof(uint16_t) <= 120 * 1024; }

static int fused_qkv_rope(const FusedArgs& base, bool norm, const void* w, const void* bias, void* q_out,
                          const void* positions, const void* cos_sin, const void* slots, void* k_pages, void* v_pages,
                          int m, int k, int n_q, int n_kv, int d, int page_size, int rows, int waves, hipStream_t stream) {
  if (m <= 0) return 0;
  if (m > 16 || (k & 7) || (d & 31)) return -1;
  FusedArgs a = base;
  a.w = (const bf16_t*)w; a.bias = (const float*)bias; a.m = m; a.n = (n_q + 2 * n_kv) * d; a.k = k;
  a.out = (bf16_t*)q_out; a.ldc = n_q * d;
  a.positions = (const int*)positions; a.cos_sin = (const float*)cos_sin; a.slots = (const int*)slots;
  a.k_pages = (bf16_t*)k_pages; a.v_pages = (bf16_t*)v_pages; a.n_q = n_q; a.n_kv = n_kv; a.d = d; a.page_size = page_size;
  a.rows = rows_per_tile(n_q, n_kv, d, m, k, norm, rows);
  const int tiles = (n_q + n_kv) * (d / 2 / a.rows) + n_kv * d / a.rows;
  if (norm || stage_rows(m, k)) return launch_rows<EPI_ROPE_STORE, true>(a, tiles, waves, stream);
  return launch_rows<EPI_ROPE_STORE, false>(a, tiles, waves, stream);
}

// q/k/v projection of up to 16 rows read from the float residual (normalised on the fly): bias, rotation,
// q into `q_out` [m, n_q * d], keys and values into their pages (slots null or negative: not stored).
// rows / waves: 0 = the launcher's choice of weight rows per workgroup and waves sharing a workgroup's K.
extern "C" int ta_fused_norm_qkv_rope(const void* residual, const void* norm_weight, float eps, const void* w,
                                      const void* bias, void* q_out, const void* positions, const void* cos_sin,
                                      const void* slots, void* k_pages, void* v_pages, int m, int k, int n_q,
                                      int n_kv, int d, int page_size, int rows, int waves, hipStream_t stream) {
  FusedArgs a = {};
  a.residual_in = (const float*)residual; a.norm_weight = (const float*)norm_weight; a.eps = eps;
  return fused_qkv_rope(a, true, w, bias, q_out, positions, cos_sin, slots, k_pages, v_pages, m, k, n_q, n_kv, d,
                        page_size, rows, waves, stream);
}

// The same from rows that are normalised already: x bfloat16 [m, k] with row stride lda.  For wide models, where
// normalising all rows again in every workgroup costs more than one small kernel before this one.
extern "C" int ta_fused_qkv_rope(const void* x, int lda, const void* w, const void* bias, void* q_out,
                                 const void* positions, const void* cos_sin, const void* slots, void* k_pages,
                                 void* v_pages, int m, int k, int n_q, int n_kv, int d, int page_size, int rows,
                                 int waves, hipStream_t stream) {
  if (lda & 7) return -1;
  FusedArgs a = {};
  a.a = (const bf16_t*)x; a.lda = lda;
  return fused_qkv_rope(a, false, w, bias, q_out, positions, cos_sin, slots, k_pages, v_pages, m, k, n_q, n_kv, d,
                        page_size, rows, waves, stream);
}

// out [m, n/2] = silu(x Wg^T) * (x Wu^T), x = the normalised residual rows, W = [Wg; Wu] of shape [n, k].
extern "C" int ta_fused_norm_gated(const void* residual, const void* norm_weight, float eps, const void* w,
                                   void* out, int m, int n, int k, int rows, int waves, hipStream_t stream) {
  if (m <= 0) return 0;
  if (m > 16 || (k & 7) || (n & 1)) return -1;
  FusedArgs a = {};
  a.residual_in = (const float*)residual; a.norm_weight = (const float*)norm_weight; a.eps = eps;
  a.w = (const bf16_t*)w; a.m = m; a.n = n; a.k = k; a.out = (bf16_t*)out; a.ldc = n / 2;
  a.rows = rows_per_gated_workgroup(n / 2, m, k, rows);
  return launch_rows<EPI_GATED, true>(a, (n / 2 + a.rows - 1) / a.rows, waves, stream);
}

// The same from rows that are normalised already: x bfloat16 [m, k] with row stride lda.
extern "C" int ta_fused_gated(const void* x, int lda, const void* w, void* out, int m, int n, int k, int rows,
                              int waves, hipStream_t stream) {
  if (m <= 0) return 0;
  if (m > 16 || (k & 7) || (lda & 7) || (n & 1)) return -1;
  FusedArgs a = {};
  a.a = (const bf16_t*)x; a.lda = lda;
  a.w = (const bf16_t*)w; a.m = m; a.n = n; a.k = k; a.out = (bf16_t*)out; a.ldc = n / 2;
  a.rows = stage_rows(m, k) ? rows_per_gated_workgroup(n / 2, m, k, rows) : rows_per_workgroup(n / 2, rows);
  if (stage_rows(m, k)) return launch_rows<EPI_GATED, true>(a, (n / 2 + a.rows - 1) / a.rows, waves, stream);
  return launch_rows<EPI_GATED, false>(a, (n / 2 + a.rows - 1) / a.rows, waves, stream);
}

// residual [m, n] += x W^T (+ bias), x bfloat16 [m, k] with row stride lda.
extern "C" int ta_fused_linear_residual(const void* x, int lda, const void* w, const void* bias, void* residual,
                                        int m, int n, int k, int rows, int waves, hipStream_t stream) {
  if (m <= 0) return 0;
  if (m > 16 || (k & 7) || (lda & 7)) return -1;
  FusedArgs a = {};
  a.a = (const bf16_t*)x; a.lda = lda; a.w = (const bf16_t*)w; a.bias = (const float*)bias;
  a.m = m; a.n = n; a.k = k; a.residual_out = (float*)residual;
  a.rows = rows_per_workgroup(n, rows);
  return launch_rows<EPI_RESIDUAL, false>(a, (n + a.rows - 1) / a.rows, waves, stream);
}
