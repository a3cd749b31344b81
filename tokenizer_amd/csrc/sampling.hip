// Greedy pick on the device: the first maximum wins, as a scan with `>` from -inf does.
#include "common.h"

__global__ void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab) {
  __shared__ float best_s[16];
  __shared__ int at_s[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    if (v > best) { best = v; at = i; }  // ascending i per thread: the first maximum stays
  }
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, WAVE);
    const int oa = __shfl_xor(at, off, WAVE);
    if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
  }
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  if (lane == 0) { best_s[wave] = best; at_s[wave] = at; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int n_waves = blockDim.x / WAVE;
    for (int w = 1; w < n_waves; ++w)
      if (best_s[w] > best || (best_s[w] == best && at_s[w] < at)) { best = best_s[w]; at = at_s[w]; }
    out[blockIdx.x] = (at == 0x7fffffff) ? 0 : at;  // all -inf or NaN: index 0, as the scan gives
  }
}

extern "C" int ta_argmax(const void* logits, void* out, int n_rows, int vocab, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  argmax_kernel<<<n_rows, 1024, 0, stream>>>((const float*)logits, (int*)out, vocab);
  return LAUNCH_STATUS();
}
