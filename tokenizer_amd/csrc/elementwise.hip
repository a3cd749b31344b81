// Embedding gather, residual-add + RMSNorm, gated activation.
#include "common.h"

// out[t, :] = table[ids[t], :] widened to float (the residual stream is float).
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 || id >= vocab) id = 0;  // the host rejects such ids before the launch
  const T* row = table + (size_t)id * hidden;
  float* dst = out + (size_t)t * hidden;
  for (int h = threadIdx.x; h < hidden; h += blockDim.x) dst[h] = ld(row + h);
}

// The same for bfloat16 tables whose rows are a multiple of eight long: sixteen bytes a thread.
__global__ void __launch_bounds__(256)
embedding_vec_kernel(const int* __restrict__ ids, const bf16_t* __restrict__ table, float* __restrict__ out,
                     int hidden, int vocab) {
  HELD(ids, table, out, hidden, vocab);
  const int t = blockIdx.x;
  int id = scalar_int(ids + t);
  if (id < 0 || id >= vocab) id = 0;  // the host rejects such ids before the launch
  const uint4* row = reinterpret_cast<const uint4*>(table + (size_t)id * hidden);
  float* dst = out + (size_t)t * hidden;
  for (int h8 = threadIdx.x; h8 * 8 < hidden; h8 += blockDim.x) {
    const uint4 raw = row[h8];
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
    *reinterpret_cast<float4*>(dst + h8 * 8) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(dst + h8 * 8 + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
}

// For output row i: r = rows ? rows[i] : i;  x = residual[r] (+ delta[r]);
// if store_residual: residual[r] = x;  out[i] = x / sqrt(mean(x^2) + eps) * weight.
// Sum of squares, root and scaling are float.
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                   const float* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps, int store_residual) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* res = residual + (size_t)r * hidden;
  const T* del = delta ? delta + (size_t)r * hidden : nullptr;
  float sq = 0.f;
  for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
    float x = res[h];
    if (del) x += ld(del + h);
    sq += x * x;
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
  for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
    float x = res[h];
    if (del) x += ld(del + h);
    if (store_residual) res[h] = x;
    st(dst + h, x * inv * weight[h]);
  }
}

// The same for rows of up to 4096 elements (a multiple of 4): every thread keeps its four-element pieces in
// registers, so the row is read once, 16 bytes at a time.
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_bits_to_float(raw.x & 0xffffu), bf16_bits_to_float(raw.x >> 16),
                     bf16_bits_to_float(raw.y & 0xffffu), bf16_bits_to_float(raw.y >> 16));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
  uint2 raw;
  raw.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  raw.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}

// CHUNKS: runs of 1,024 floats that a row has (a thread takes four floats of each).  The old residual, the delta
// and the norm weight are all asked for at the start (a thread past the end of the row asks for the row's last
// floats and does not use them, so that no load stands behind a condition): one trip to memory where a chunk after
// the other, and the weight after the sum, were up to five.
template <typename T, int CHUNKS, bool DELTA>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ residual, const T* __restrict__ delta, const float* __restrict__ weight,
                       T* __restrict__ out, const int* __restrict__ rows, int hidden, float eps, int store_residual) {
  HELD(residual, delta, weight, out, rows, hidden, eps, store_residual);
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int r = rows ? scalar_int(rows + i) : i;
  float* res = residual + (size_t)r * hidden;
  const T* del = delta + (size_t)r * hidden;
  float4 x[CHUNKS], d[CHUNKS], gain[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = min((c * 256 + (int)threadIdx.x) * 4, hidden - 4);
    x[c] = ld4(res + h);
    if (DELTA) d[c] = ld4(del + h);
    gain[c] = ld4(weight + h);
  }
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * 256 + threadIdx.x) * 4;
    if (DELTA) { x[c].x += d[c].x; x[c].y += d[c].y; x[c].z += d[c].z; x[c].w += d[c].w; }
    if (h >= hidden) x[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    else if (DELTA && store_residual) st4(res + h, x[c]);
    sq += x[c].x * x[c].x + x[c].y * x[c].y + x[c].z * x[c].z + x[c].w * x[c].w;
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * 256 + threadIdx.x) * 4;
    if (h >= hidden) continue;
    const float4 w = gain[c];
    st4(dst + h, make_float4(x[c].x * inv * w.x, x[c].y * inv * w.y, x[c].z * inv * w.z, x[c].w * inv * w.w));
  }
}

// The same with the delta still in parts: a product whose K was cut over workgroups left `splits` slabs of
// float sums [M, hidden]; they are added in their order, the bias joins, the sum goes into the residual stream
// (stored back) and the row is normalised.  One kernel instead of the addition and the norm after it.
// CHUNKS: runs of 1,024 floats that a row has (a thread takes four floats of each).  Everything a thread needs (the
// old residual, the bias, the norm weight and the first slabs) is asked for at once and nothing is used
// before all of it is under way: asked for one after the other as they are needed, these are five trips to memory
// in a kernel that is over after one.  A thread past the end of the row asks for the row's last floats and does
// not use them (no load stands behind a condition).
template <typename T, int CHUNKS>
__global__ void __launch_bounds__(256)
splitk_add_rmsnorm_kernel(float* __restrict__ residual, const float* __restrict__ partial, int splits,
                          const float* __restrict__ bias, const float* __restrict__ weight, T* __restrict__ out,
                          int n_rows, int hidden, float eps) {
  HELD(residual, partial, splits, bias, weight, out, n_rows, hidden, eps);
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  float* res = residual + (size_t)i * hidden;
  const size_t slab_stride = (size_t)n_rows * hidden;
  const float* bias_or_any = bias ? bias : weight;           // (without a bias: loaded from a valid place, not used)
  constexpr int FIRST = CHUNKS == 1 ? 8 : 4;                 // slabs asked for at the start (registers: sixteen bytes each)
  float4 old[CHUNKS], gain[CHUNKS], extra[CHUNKS], first[CHUNKS][FIRST];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = min((c * 256 + (int)threadIdx.x) * 4, hidden - 4);
    old[c] = ld4(res + h);
    extra[c] = ld4(bias_or_any + h);
    gain[c] = ld4(weight + h);
    const float* slab = partial + (size_t)i * hidden + h;
#pragma unroll
    for (int j = 0; j < FIRST; ++j) first[c][j] = ld4(slab + (size_t)min(j, splits - 1) * slab_stride);
  }
  float4 x[CHUNKS];
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * 256 + threadIdx.x) * 4;
    const int hc = min(h, hidden - 4);
    // The slabs are added in their order, eight asked for at a time after the first ones.
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < FIRST; ++j) {
      const float4 v = j < splits ? first[c][j] : make_float4(0.f, 0.f, 0.f, 0.f);
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    const float* slab = partial + (size_t)i * hidden + hc;
    for (int s0 = FIRST; s0 < splits; s0 += 8) {
      float4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = ld4(slab + (size_t)min(s0 + j, splits - 1) * slab_stride);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float4 u = s0 + j < splits ? v[j] : make_float4(0.f, 0.f, 0.f, 0.f);
        sum.x += u.x; sum.y += u.y; sum.z += u.z; sum.w += u.w;
      }
    }
    if (bias) { sum.x += extra[c].x; sum.y += extra[c].y; sum.z += extra[c].z; sum.w += extra[c].w; }
    x[c] = make_float4(old[c].x + sum.x, old[c].y + sum.y, old[c].z + sum.z, old[c].w + sum.w);
    if (h < hidden) st4(res + h, x[c]);
    else x[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    sq += x[c].x * x[c].x + x[c].y * x[c].y + x[c].z * x[c].z + x[c].w * x[c].w;
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * 256 + threadIdx.x) * 4;
    if (h >= hidden) continue;
    const float4 w = gain[c];
    st4(dst + h, make_float4(x[c].x * inv * w.x, x[c].y * inv * w.y, x[c].z * inv * w.z, x[c].w * inv * w.w));
  }
}

// out[t, j] = silu(in[t, j]) * in[t, inner + j], silu(z) = z * sigmoid(z), in float.
template <typename T>
__global__ void silu_gate_kernel(const T* __restrict__ in, T* __restrict__ out, int inner, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inner;
    const int j = (int)(idx - t * inner);
    const float g = ld(in + t * 2 * inner + j);
    const float u = ld(in + t * 2 * inner + inner + j);
    st(out + idx, g / (1.0f + expf(-g)) * u);
  }
}

// The same for bfloat16 rows whose length is a multiple of 8: sixteen bytes of gate and of up per thread.
__global__ void silu_gate_vec_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, int inner8,
                                     unsigned total8) {
  for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += gridDim.x * blockDim.x) {
    const unsigned t = idx / (unsigned)inner8, j = idx - t * (unsigned)inner8;
    const uint4* row = reinterpret_cast<const uint4*>(in) + (size_t)t * 2 * inner8;
    const uint4 gate = row[j], up = row[inner8 + j];
    const uint32_t gw[4] = {gate.x, gate.y, gate.z, gate.w}, uw[4] = {up.x, up.y, up.z, up.w};
    uint32_t packed[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
      const float r0 = g0 / (1.0f + expf(-g0)) * u0, r1 = g1 / (1.0f + expf(-g1)) * u1;
      packed[i] = (uint32_t)float_to_bf16_bits(r0) | ((uint32_t)float_to_bf16_bits(r1) << 16);
    }
    reinterpret_cast<uint4*>(out)[idx] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
  }
}

extern "C" int ta_embedding(const void* ids, const void* table, void* out, int n_tokens, int hidden,
                            int vocab, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (dtype == DT_F32)
    embedding_kernel<float><<<n_tokens, 256, 0, stream>>>((const int*)ids, (const float*)table, (float*)out, hidden, vocab);
  else if (hidden % 8 == 0 && (((uintptr_t)table | (uintptr_t)out) & 15) == 0)
    embedding_vec_kernel<<<n_tokens, 256, 0, stream>>>((const int*)ids, (const bf16_t*)table, (float*)out, hidden, vocab);
  else
    embedding_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const int*)ids, (const bf16_t*)table, (float*)out, hidden, vocab);
  return LAUNCH_STATUS();
}

extern "C" int ta_add_rmsnorm(void* residual, const void* delta, const void* weight, void* out,
                              const void* rows, int n_rows, int hidden, float eps, int store_residual,
                              int dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (hidden % 4 == 0 && hidden <= 4096) {
#define GO(TT, CC, DD) add_rmsnorm_vec_kernel<TT, CC, DD><<<n_rows, 256, 0, stream>>>( \
    (float*)residual, (const TT*)delta, (const float*)weight, (TT*)out, (const int*)rows, hidden, eps, store_residual)
#define GO_DELTA(TT, CC) if (delta) GO(TT, CC, true); else GO(TT, CC, false)
#define GO_CHUNKS(TT) switch ((hidden + 1023) / 1024) { case 1: GO_DELTA(TT, 1); break; case 2: GO_DELTA(TT, 2); break; \
                                                        case 3: GO_DELTA(TT, 3); break; default: GO_DELTA(TT, 4); break; }
    if (dtype == DT_F32) GO_CHUNKS(float) else GO_CHUNKS(bf16_t)
#undef GO_CHUNKS
#undef GO_DELTA
#undef GO
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    add_rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>((float*)residual, (const float*)delta, (const float*)weight,
                                                          (float*)out, (const int*)rows, hidden, eps, store_residual);
  else
    add_rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((float*)residual, (const bf16_t*)delta, (const float*)weight,
                                                           (bf16_t*)out, (const int*)rows, hidden, eps, store_residual);
  return LAUNCH_STATUS();
}

// residual [n_rows, hidden] += the slabs of `partial` ([splits, n_rows, hidden] floats, added in order) + bias;
// out = rmsnorm(residual) * weight.  hidden a multiple of 4 and at most 4096.
extern "C" int ta_splitk_add_rmsnorm(void* residual, const void* partial, int splits, const void* bias,
                                     const void* weight, void* out, int n_rows, int hidden, float eps, int dtype,
                                     hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (hidden % 4 || hidden > 4096 || splits < 1 || !partial) return -1;
#define GO(TT, CC) splitk_add_rmsnorm_kernel<TT, CC><<<n_rows, 256, 0, stream>>>( \
    (float*)residual, (const float*)partial, splits, (const float*)bias, (const float*)weight, (TT*)out, n_rows, hidden, eps)
#define GO_CHUNKS(TT) switch ((hidden + 1023) / 1024) { case 1: GO(TT, 1); break; case 2: GO(TT, 2); break; \
                                                        case 3: GO(TT, 3); break; default: GO(TT, 4); break; }
  if (dtype == DT_F32) GO_CHUNKS(float) else GO_CHUNKS(bf16_t)
#undef GO_CHUNKS
#undef GO
  return LAUNCH_STATUS();
}

extern "C" int ta_silu_gate(const void* in, void* out, int n_tokens, int inner, int dtype, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * inner;
  if (total == 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  if (dtype != DT_F32 && inner % 8 == 0 && total / 8 < 0xffffffffu && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    const size_t total8 = total / 8;
    const int blocks8 = (int)((total8 + 255) / 256 < 16384 ? (total8 + 255) / 256 : 16384);
    silu_gate_vec_kernel<<<blocks8, 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, inner / 8, (unsigned)total8);
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    silu_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, (float*)out, inner, total);
  else
    silu_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, inner, total);
  return LAUNCH_STATUS();
}

// The number of compute units that the launchers plan for (the current device's).
extern "C" int ta_compute_units() { return compute_units(); }

// A yardstick, not a model kernel: reads `n16` words of sixteen bytes once, in the access pattern of the
// weight-streaming kernels (a wave instruction reads 1 KB of one run, eight such loads of a lane in flight), and
// leaves the xor of everything it read per workgroup in `out` so that no load can be dropped.  What it reaches is
// what a kernel bound by HBM can reach on this device.
typedef uint32_t word4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) read_stream_kernel(const word4* __restrict__ p, size_t n16, uint32_t* __restrict__ out) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    word4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const word4 v = __builtin_nontemporal_load(p + i);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, WAVE);
  __shared__ uint32_t parts[4];
  if ((threadIdx.x & 63) == 0) parts[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = parts[0] ^ parts[1] ^ parts[2] ^ parts[3];
}

// out: uint32 [workgroups]; bytes a multiple of 16; data 16-byte aligned.
extern "C" int ta_read_stream(const void* data, size_t bytes, void* out, int workgroups, hipStream_t stream) {
  if (bytes % 16 || workgroups <= 0 || ((uintptr_t)data & 15)) return -1;
  read_stream_kernel<<<workgroups, 256, 0, stream>>>((const word4*)data, bytes / 16, (uint32_t*)out);
  return LAUNCH_STATUS();
}
