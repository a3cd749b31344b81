// The second step of a product whose K was cut over workgroups: the parts' float sums, one slab of
// [M, N] per part, are added in the order of the parts (so the result is the same on every run), the bias joins,
// and the result is stored in the output's type.
#pragma once
#include "common.h"

__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// C[m, n] = sum over the slabs (in their order) + bias: four columns a thread (N is a multiple of 4 here).
template <typename OutT>
__global__ void splitk_reduce(const float* __restrict__ partial, const float* __restrict__ bias, OutT* __restrict__ C,
                              int M, int N, int ldc, int splits) {
  const size_t quad = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t per_row = N / 4;
  if (quad >= (size_t)M * per_row) return;
  const int m = (int)(quad / per_row), n = (int)(quad % per_row) * 4;
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s = 0; s < splits; ++s) {
    const float4 v = *reinterpret_cast<const float4*>(partial + ((size_t)s * M + m) * N + n);
    sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
  }
  if (bias) { sum.x += bias[n]; sum.y += bias[n + 1]; sum.z += bias[n + 2]; sum.w += bias[n + 3]; }
  OutT* dst = C + (size_t)m * ldc + n;
  store_out(dst, sum.x); store_out(dst + 1, sum.y); store_out(dst + 2, sum.z); store_out(dst + 3, sum.w);
}

// Into how many parts K really falls when `splits` are asked for and a part is a multiple of `step`: no part
// without a step of its own.
static inline int parts_of_k(int K, int splits, int step) {
  if (splits <= 1) return 1;
  const int chunk = ((K + splits - 1) / splits + step - 1) / step * step;
  return (K + chunk - 1) / chunk;
}

// Launches the reduction; returns the launch status.
static inline int launch_splitk_reduce(const float* slabs, const void* bias, void* C, int M, int N, int ldc, int splits,
                                       int out_dtype, hipStream_t stream) {
  const size_t quads = (size_t)M * (N / 4);
  const int blocks = (int)((quads + 255) / 256);
  if (out_dtype == DT_F32)
    splitk_reduce<float><<<blocks, 256, 0, stream>>>(slabs, (const float*)bias, (float*)C, M, N, ldc, splits);
  else
    splitk_reduce<bf16_t><<<blocks, 256, 0, stream>>>(slabs, (const float*)bias, (bf16_t*)C, M, N, ldc, splits);
  return LAUNCH_STATUS();
}
