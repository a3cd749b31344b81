// C[M,N] = A[M,K] * W[N,K]^T (+ bias): bfloat16 operands, float accumulation on the matrix cores
// (v_mfma_f32_32x32x16_bf16), output bfloat16 or float.  Tiles are staged through LDS; one block of
// four waves owns a BM x BN tile of C, each wave a quarter of it.
#include "common.h"
#include "splitk_reduce.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));



// BK: elements of K per step; rows in LDS are BK + 8 apart (padding against bank conflicts, still 16-byte aligned).
//
// Split K: blockIdx.z takes `k_chunk` elements of K (a multiple of BK) and, when there are several such blocks,
// writes its float sums into its own slab of `partial` [splits, M, N]; `splitk_reduce` then adds the slabs in
// their fixed order (and the bias) into C.  That is for products whose output is too small to fill the device
// with tiles but whose K is long: every compute unit streams a share of the weights.
template <int BM, int BN, int BK, typename OutT, int AHEAD = 3>
__global__ void __launch_bounds__(256)
gemm_bf16_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
                 OutT* __restrict__ C, int M, int N, int K, int lda, int ldc, int k_chunk, float* __restrict__ partial) {
  constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / 32, TNI = WN / 32;
  constexpr int GB_BK = BK, GB_LDS = BK + 8, CPR = BK / 8;          // 16-byte chunks per row
  constexpr int A_CHUNKS = BM * CPR / 256, W_CHUNKS = BN * CPR / 256;   // chunks per thread and K step
  // Two LDS buffers: while one K step is multiplied, the next one's tiles (already in registers) are
  // written into the other, so a step costs one barrier.
  __shared__ __attribute__((aligned(16))) uint16_t a_s[2][BM * GB_LDS];
  __shared__ __attribute__((aligned(16))) uint16_t w_s[2][BN * GB_LDS];
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int k_begin = blockIdx.z * k_chunk, k_end = min(K, k_begin + k_chunk);
  floatx16 acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // AHEAD steps of K are on their way from memory into registers at any time: a step's products take far less
  // time than a trip to memory, so with one step in flight a tile's walk over K would be a chain of such trips.
  uint4 a_reg[AHEAD][A_CHUNKS], w_reg[AHEAD][W_CHUNKS];
  // Loads are unconditional (a row past the end reads the last row, a step past the end of K the last
  // chunk of the row: both are valid addresses), so that the compiler can count them and wait only for the
  // step it is about to use; what lies past the end of K is replaced by zeros on its way into LDS, and rows
  // past the end are never stored.
  auto fetch = [&](int k0, uint4 (&a_now)[A_CHUNKS], uint4 (&w_now)[W_CHUNKS]) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int m = min(m0 + c / CPR, M - 1), k = min(k0 + (c % CPR) * 8, K - 8);
      a_now[i] = *reinterpret_cast<const uint4*>(A + (size_t)m * lda + k);
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int n = min(n0 + c / CPR, N - 1), k = min(k0 + (c % CPR) * 8, K - 8);
      w_now[i] = *reinterpret_cast<const uint4*>(W + (size_t)n * K + k);
    }
  };
  auto stash = [&](int buf, int k0, const uint4 (&a_now)[A_CHUNKS], const uint4 (&w_now)[W_CHUNKS]) {
    const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const bool inside = k0 + (c % CPR) * 8 < k_end;
      uint4 v = a_now[i];
      if (!inside) v = zero;
      *reinterpret_cast<uint4*>(a_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = v;
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const bool inside = k0 + (c % CPR) * 8 < k_end;
      uint4 v = w_now[i];
      if (!inside) v = zero;
      *reinterpret_cast<uint4*>(w_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = v;
    }
  };

#pragma unroll
  for (int j = 0; j < AHEAD; ++j) fetch(k_begin + j * GB_BK, a_reg[j], w_reg[j]);
  stash(0, k_begin, a_reg[0], w_reg[0]);
  __syncthreads();
  int buf = 0;
  for (int k_round = k_begin; k_round < k_end; k_round += AHEAD * GB_BK) {
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {          // step k0 was fetched into registers j and sits in LDS buffer `buf`
      const int k0 = k_round + j * GB_BK;
      if (k0 < k_end) {                        // (no `break`: the register sets keep their fixed indices)
        fetch(k0 + AHEAD * GB_BK, a_reg[j], w_reg[j]);
#pragma unroll
        for (int ks = 0; ks < GB_BK; ks += 16) {
          bf16x8 af[TMI], bf[TNI];
#pragma unroll
          for (int i = 0; i < TMI; ++i)
            af[i] = *reinterpret_cast<const bf16x8*>(a_s[buf] + (wm * WM + i * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
          for (int jn = 0; jn < TNI; ++jn)
            bf[jn] = *reinterpret_cast<const bf16x8*>(w_s[buf] + (wn * WN + jn * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
          for (int i = 0; i < TMI; ++i)
#pragma unroll
            for (int jn = 0; jn < TNI; ++jn)
              acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[jn], acc[i][jn], 0, 0, 0);
        }
        // Nobody reads the other buffer now: its last readers passed the previous barrier.
        if (k0 + GB_BK < k_end) stash(buf ^ 1, k0 + GB_BK, a_reg[(j + 1) % AHEAD], w_reg[(j + 1) % AHEAD]);
        __syncthreads();
        buf ^= 1;
      }
    }
  }
  // Lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4 of each 32x32 tile.
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j) {
      const int n = n0 + wn * WN + j * 32 + (lane & 31);
      if (n >= N) continue;
      const float b = (bias && !partial) ? bias[n] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m >= M) continue;
        if (partial) partial[((size_t)blockIdx.z * M + m) * N + n] = acc[i][j][r];
        else store_out(C + (size_t)m * ldc + n, acc[i][j][r] + b);
      }
    }
}

template <int BM, int BN, int BK>
static int launch(const void* A, const void* W, const void* bias, void* C, int M, int N, int K, int lda,
                  int ldc, int out_dtype, hipStream_t stream, int splits = 1, void* partial = nullptr) {
  const int k_chunk = splits > 1 ? ((K + splits - 1) / splits + BK - 1) / BK * BK : K;
  if (splits > 1) splits = (K + k_chunk - 1) / k_chunk;      // no block without a step of its own
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, splits);
  float* slabs = splits > 1 ? (float*)partial : nullptr;
  if (out_dtype == DT_F32)
    gemm_bf16_kernel<BM, BN, BK, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (const float*)bias,
                                                              (float*)C, M, N, K, lda, ldc, k_chunk, slabs);
  else
    gemm_bf16_kernel<BM, BN, BK, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (const float*)bias,
                                                               (bf16_t*)C, M, N, K, lda, ldc, k_chunk, slabs);
  int status = LAUNCH_STATUS();
  if (status == 0 && splits > 1 && C) status = launch_splitk_reduce(slabs, bias, C, M, N, ldc, splits, out_dtype, stream);
  return status;
}

// K and lda must be multiples of 8 and the pointers 16-byte aligned (the host checks).
extern "C" int ta_gemm_bf16(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                            int lda, int ldc, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if ((K & 7) || (lda & 7)) return -1;
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (M <= 64 || tiles128 < 512) {
    // Few tiles: each step's loads are latency-bound, so a step covers more of K.
    if (K >= 256) return launch<64, 64, 64>(A, W, bias, C, M, N, K, lda, ldc, out_dtype, stream);
    return launch<64, 64, 32>(A, W, bias, C, M, N, K, lda, ldc, out_dtype, stream);
  }
  return launch<128, 128, 32>(A, W, bias, C, M, N, K, lda, ldc, out_dtype, stream);
}

// The same product with K cut into `splits` parts (at most; parts are multiples of 64) over 64 x 64 tiles, the
// parts' float sums added afterwards in a fixed order.  partial: room for splits * M * N floats; N % 4 == 0.
// With C null (and more than one part after the rounding of the parts' length) the sums are left in `partial`.
extern "C" int ta_gemm_bf16_splitk(const void* A, const void* W, const void* bias, void* C, void* partial, int M,
                                   int N, int K, int lda, int ldc, int out_dtype, int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if ((K & 7) || (lda & 7) || (N & 3) || splits < 1 || (splits > 1 && !partial)) return -1;
  if (!C && parts_of_k(K, splits, 64) < 2) return -1;
  return launch<64, 64, 64>(A, W, bias, C, M, N, K, lda, ldc, out_dtype, stream, splits, partial);
}

// The addition alone: C[M, N] (row stride ldc) = the `splits` slabs of `partial` in their order + bias.
extern "C" int ta_splitk_reduce(const void* partial, const void* bias, void* C, int M, int N, int ldc, int splits,
                                int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if ((N & 3) || splits < 1 || !partial || !C) return -1;
  return launch_splitk_reduce((const float*)partial, bias, C, M, N, ldc, splits, out_dtype, stream);
}
