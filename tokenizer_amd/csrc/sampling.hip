// Greedy pick on the device: the first maximum wins, as a scan with `>` from -inf does.
#include "common.h"

#define ARGMAX_THREADS 256

__device__ __forceinline__ bool better(float v, int at, float best, int best_at) {
  return v > best || (v == best && at < best_at);
}

// Block-wide (maximum, lowest index of it); the result is valid in thread 0.
__device__ __forceinline__ void block_best(float& best, int& at, float* best_s, int* at_s) {
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, WAVE);
    const int oa = __shfl_xor(at, off, WAVE);
    if (better(ob, oa, best, at)) { best = ob; at = oa; }
  }
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  if (lane == 0) { best_s[wave] = best; at_s[wave] = at; }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < ARGMAX_THREADS / WAVE; ++w)
      if (better(best_s[w], at_s[w], best, at)) { best = best_s[w]; at = at_s[w]; }
}

// Stage one: each row is cut into `chunks` pieces, one workgroup per piece; a piece's (maximum, index)
// goes to partial_v / partial_i [n_rows, chunks].  NaN never wins.
__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_pieces(const float* __restrict__ logits, float* __restrict__ partial_v, int* __restrict__ partial_i,
              int vocab, int chunks) {
  __shared__ float best_s[ARGMAX_THREADS / WAVE];
  __shared__ int at_s[ARGMAX_THREADS / WAVE];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float* src = logits + (size_t)row * vocab;
  const int per = (vocab + chunks - 1) / chunks;
  const int begin = chunk * per, end = min(vocab, begin + per);
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += ARGMAX_THREADS) {
    const float v = src[i];
    if (v > best) { best = v; at = i; }          // ascending i per thread: its first maximum stays
  }
  block_best(best, at, best_s, at_s);
  if (threadIdx.x == 0) {
    partial_v[(size_t)row * chunks + chunk] = best;
    partial_i[(size_t)row * chunks + chunk] = at;
  }
}

// Stage two: one workgroup per row reduces the pieces; a row without any maximum gives index 0.
__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_rows(const float* __restrict__ partial_v, const int* __restrict__ partial_i, int* __restrict__ out,
            int chunks) {
  __shared__ float best_s[ARGMAX_THREADS / WAVE];
  __shared__ int at_s[ARGMAX_THREADS / WAVE];
  const int row = blockIdx.x;
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += ARGMAX_THREADS) {
    const float v = partial_v[(size_t)row * chunks + c];
    const int a = partial_i[(size_t)row * chunks + c];
    if (better(v, a, best, at)) { best = v; at = a; }
  }
  block_best(best, at, best_s, at_s);
  if (threadIdx.x == 0) out[row] = (at == 0x7fffffff) ? 0 : at;
}

extern "C" int ta_argmax(const void* logits, void* out, void* partial_v, void* partial_i, int n_rows, int vocab,
                         int chunks, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (chunks < 1 || vocab < 1) return -1;
  dim3 grid(chunks, n_rows);
  argmax_pieces<<<grid, ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)partial_v, (int*)partial_i,
                                                    vocab, chunks);
  int status = LAUNCH_STATUS();
  if (status) return status;
  argmax_rows<<<n_rows, ARGMAX_THREADS, 0, stream>>>((const float*)partial_v, (const int*)partial_i, (int*)out, chunks);
  return LAUNCH_STATUS();
}
