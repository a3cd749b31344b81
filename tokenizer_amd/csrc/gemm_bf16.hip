// C[M,N] = A[M,K] * W[N,K]^T (+ bias): bfloat16 operands, float accumulation on the matrix cores
// (v_mfma_f32_32x32x16_bf16), output bfloat16 or float.  Tiles are staged through LDS; one block of
// four waves owns a BM x BN tile of C, each wave a quarter of it.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));


__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// BK: elements of K per step; rows in LDS are BK + 8 apart (padding against bank conflicts, still 16-byte aligned).
template <int BM, int BN, int BK, typename OutT>
__global__ void __launch_bounds__(256)
gemm_bf16_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
                 OutT* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / 32, TNI = WN / 32;
  constexpr int GB_BK = BK, GB_LDS = BK + 8, CPR = BK / 8;          // 16-byte chunks per row
  constexpr int A_CHUNKS = BM * CPR / 256, W_CHUNKS = BN * CPR / 256;   // chunks per thread and K step
  // Two LDS buffers: while one K step is multiplied, the next one's tiles (already requested from
  // memory into registers) are written into the other, so a step costs one barrier and the loads of
  // step k+1 are in flight during the products of step k.
  __shared__ __attribute__((aligned(16))) uint16_t a_s[2][BM * GB_LDS];
  __shared__ __attribute__((aligned(16))) uint16_t w_s[2][BN * GB_LDS];
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  floatx16 acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 a_reg[A_CHUNKS], w_reg[W_CHUNKS];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int r = c / CPR, kc = (c % CPR) * 8;
      const int m = m0 + r, k = k0 + kc;
      a_reg[i] = make_uint4(0, 0, 0, 0);
      if (m < M && k < K) a_reg[i] = *reinterpret_cast<const uint4*>(A + (size_t)m * lda + k);
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int r = c / CPR, kc = (c % CPR) * 8;
      const int n = n0 + r, k = k0 + kc;
      w_reg[i] = make_uint4(0, 0, 0, 0);
      if (n < N && k < K) w_reg[i] = *reinterpret_cast<const uint4*>(W + (size_t)n * K + k);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      *reinterpret_cast<uint4*>(a_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      *reinterpret_cast<uint4*>(w_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = w_reg[i];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += GB_BK) {
    const bool more = k0 + GB_BK < K;
    if (more) fetch(k0 + GB_BK);
#pragma unroll
    for (int ks = 0; ks < GB_BK; ks += 16) {
      bf16x8 af[TMI], bf[TNI];
#pragma unroll
      for (int i = 0; i < TMI; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(a_s[buf] + (wm * WM + i * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
      for (int j = 0; j < TNI; ++j)
        bf[j] = *reinterpret_cast<const bf16x8*>(w_s[buf] + (wn * WN + j * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
      for (int i = 0; i < TMI; ++i)
#pragma unroll
        for (int j = 0; j < TNI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (more) stash(buf ^ 1);      // nobody reads that buffer now: its last readers passed the previous barrier
    __syncthreads();
    buf ^= 1;
  }
  // Lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4 of each 32x32 tile.
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j) {
      const int n = n0 + wn * WN + j * 32 + (lane & 31);
      if (n >= N) continue;
      const float b = bias ? bias[n] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < M) store_out(C + (size_t)m * ldc + n, acc[i][j][r] + b);
      }
    }
}

template <int BM, int BN, int BK>
static int launch(const void* A, const void* W, const void* bias, void* C, int M, int N, int K, int lda,
                  int ldc, int out_dtype, hipStream_t stream) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (out_dtype == DT_F32)
    gemm_bf16_kernel<BM, BN, BK, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (const float*)bias,
                                                              (float*)C, M, N, K, lda, ldc);
  else
    gemm_bf16_kernel<BM, BN, BK, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (const float*)bias,
                                                               (bf16_t*)C, M, N, K, lda, ldc);
  return LAUNCH_STATUS();
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
