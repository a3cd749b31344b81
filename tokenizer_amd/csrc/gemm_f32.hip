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

// Many rows: tiles of 128 x 128 with 8 x 8 outputs a thread (two 4 x 4 quarters each way, so that LDS is read
// sixteen bytes at a time), K in steps of 16; the next step's tiles are on their way from memory while the
// current one is multiplied.  Plain multiply-adds as everywhere in this file.
#define BTM 128
#define BTN 128
#define BTK 16

__global__ void __launch_bounds__(256)
gemm_f32_big_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                    float* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  __shared__ __attribute__((aligned(16))) float a_s[BTK][BTM + 4];
  __shared__ __attribute__((aligned(16))) float w_s[BTK][BTN + 4];
  const int m0 = blockIdx.y * BTM, n0 = blockIdx.x * BTN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  // Each thread brings in two rows x four consecutive k of A and of W per step: row = id / 4 (+ 64), k = (id % 4) * 4.
  const int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
  const bool vec = (K % 4 == 0) && (lda % 4 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  float acc[8][8] = {};
  float4 a_next[2], w_next[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int m = m0 + lr + 64 * h, n = n0 + lr + 64 * h, k = k0 + lk;
      float4 av = make_float4(0.f, 0.f, 0.f, 0.f), wv = av;
      if (vec && k + 3 < K) {
        if (m < M) av = *reinterpret_cast<const float4*>(A + (size_t)m * lda + k);
        if (n < N) wv = *reinterpret_cast<const float4*>(W + (size_t)n * K + k);
      } else {
        float at[4] = {0.f, 0.f, 0.f, 0.f}, wt[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (m < M && k + i < K) at[i] = A[(size_t)m * lda + k + i];
          if (n < N && k + i < K) wt[i] = W[(size_t)n * K + k + i];
        }
        av = make_float4(at[0], at[1], at[2], at[3]);
        wv = make_float4(wt[0], wt[1], wt[2], wt[3]);
      }
      a_next[h] = av;
      w_next[h] = wv;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lr + 64 * h;
      a_s[lk][r] = a_next[h].x; a_s[lk + 1][r] = a_next[h].y; a_s[lk + 2][r] = a_next[h].z; a_s[lk + 3][r] = a_next[h].w;
      w_s[lk][r] = w_next[h].x; w_s[lk + 1][r] = w_next[h].y; w_s[lk + 2][r] = w_next[h].z; w_s[lk + 3][r] = w_next[h].w;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BTK) {
    stash();
    __syncthreads();
    if (k0 + BTK < K) fetch(k0 + BTK);
#pragma unroll
    for (int kk = 0; kk < BTK; ++kk) {
      float a[8], w[8];
      const float4 a0 = *reinterpret_cast<const float4*>(&a_s[kk][ty * 4]);
      const float4 a1 = *reinterpret_cast<const float4*>(&a_s[kk][64 + ty * 4]);
      const float4 w0 = *reinterpret_cast<const float4*>(&w_s[kk][tx * 4]);
      const float4 w1 = *reinterpret_cast<const float4*>(&w_s[kk][64 + tx * 4]);
      a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w; a[4] = a1.x; a[5] = a1.y; a[6] = a1.z; a[7] = a1.w;
      w[0] = w0.x; w[1] = w0.y; w[2] = w0.z; w[3] = w0.w; w[4] = w1.x; w[5] = w1.y; w[6] = w1.z; w[7] = w1.w;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + (i < 4 ? ty * 4 + i : 64 + ty * 4 + i - 4);
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = n0 + (j < 4 ? tx * 4 + j : 64 + tx * 4 + j - 4);
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
  if (M > 64 && N > 64) {
    dim3 big((N + BTN - 1) / BTN, (M + BTM - 1) / BTM);
    gemm_f32_big_kernel<<<big, 256, 0, stream>>>((const float*)A, (const float*)W, (const float*)bias, (float*)C,
                                                 M, N, K, lda, ldc);
    return LAUNCH_STATUS();
  }
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  gemm_f32_kernel<<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (const float*)bias, (float*)C,
                                            M, N, K, lda, ldc);
  return LAUNCH_STATUS();
}
