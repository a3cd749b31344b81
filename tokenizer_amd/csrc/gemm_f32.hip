// C[M,N] = A[M,K] * W[N,K]^T (+ bias), everything float, plain fused multiply-adds: the matrix
// product of the 32-bit path.  No matrix-core instruction is used here on purpose.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                float* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  __shared__ float a_s[TK][TM + 1];
  __shared__ float w_s[TK][TN + 1];
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // 16 x 16 threads, 4 x 4 outputs each
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += TK) {
    for (int idx = threadIdx.x; idx < TM * TK; idx += 256) {
      const int r = idx / TK, c = idx % TK;
      const int m = m0 + r, k = k0 + c;
      a_s[c][r] = (m < M && k < K) ? A[(size_t)m * lda + k] : 0.f;
      const int n = n0 + r;
      w_s[c][r] = (n < N && k < K) ? W[(size_t)n * K + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = a_s[kk][ty * 4 + i]; w[i] = w_s[kk][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = acc[i][j] + (bias ? bias[n] : 0.f);
    }
  }
}

// Few rows (M <= 16): the product is one pass over the weights, so a wave takes four weight rows and walks K
// with sixteen bytes per lane, every row of A against them; the sums are added up over the wave at the end.
// Plain multiply-adds here as well.
template <int MR>
__global__ void __launch_bounds__(256)
gemv_f32_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                float* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 4 + wave) * 4;               // this wave's four weight rows
  if (n0 >= N) return;
  float acc[4][MR];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;
  const float* w[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) w[r] = W + (size_t)min(n0 + r, N - 1) * K;
  const bool vec = (K % 4 == 0) && (lda % 4 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  if (vec) {
    for (int k = lane * 4; k < K; k += WAVE * 4) {
      float4 wv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) wv[r] = *reinterpret_cast<const float4*>(w[r] + k);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        if (m >= M) break;
        const float4 a = *reinterpret_cast<const float4*>(A + (size_t)m * lda + k);
#pragma unroll
        for (int r = 0; r < 4; ++r)
          acc[r][m] = fmaf(a.x, wv[r].x, fmaf(a.y, wv[r].y, fmaf(a.z, wv[r].z, fmaf(a.w, wv[r].w, acc[r][m]))));
      }
    }
  } else {
    for (int k = lane; k < K; k += WAVE) {
      float wv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) wv[r] = w[r][k];
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        if (m >= M) break;
        const float a = A[(size_t)m * lda + k];
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r][m] = fmaf(a, wv[r], acc[r][m]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float total = wave_sum(acc[r][m]);
      if (lane == 0 && m < M && n0 + r < N) C[(size_t)m * ldc + n0 + r] = total + (bias ? bias[n0 + r] : 0.f);
    }
}

extern "C" int ta_gemm_f32(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                           int lda, int ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M <= 16) {
    const int blocks = (N + 15) / 16;
#define GO(MR) gemv_f32_kernel<MR><<<blocks, 256, 0, stream>>>((const float*)A, (const float*)W, (const float*)bias, \
                                                              (float*)C, M, N, K, lda, ldc)
    if (M <= 1) GO(1); else if (M <= 2) GO(2); else if (M <= 4) GO(4); else if (M <= 8) GO(8); else GO(16);
#undef GO
    return LAUNCH_STATUS();
  }
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  gemm_f32_kernel<<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (const float*)bias, (float*)C,
                                            M, N, K, lda, ldc);
  return LAUNCH_STATUS();
}
