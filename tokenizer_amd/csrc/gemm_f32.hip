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

extern "C" int ta_gemm_f32(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                           int lda, int ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  gemm_f32_kernel<<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (const float*)bias, (float*)C,
                                            M, N, K, lda, ldc);
  return LAUNCH_STATUS();
}
