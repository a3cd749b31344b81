// Position encoding of queries and keys (half-split rotation) fused with the write of keys and
// values into their pages.  One block per (token, head); heads are laid out q heads, k heads, v heads
// in a row of the fused projection output.
#include "common.h"

// qkv: [n_tokens, row_stride], heads of size d.  bias (float, may be null) is added first.
// cos_sin: [max_positions, d] float, cos of the d/2 angles then sin; null = no rotation.
// slots: physical slot of each token (page * page_size + offset), or null = nothing is stored.
// Key pages: [n_pages, n_kv, page_size, d]; value pages are transposed inside a page,
// [n_pages, n_kv, d, page_size], so that the keys a matrix-core lane contracts over lie side by side.
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                                  const int* __restrict__ positions, const float* __restrict__ cos_sin,
                                  const int* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                  int n_q, int n_kv, int d, int page_size) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;  // 0..n_q-1 q, then n_kv k heads, then n_kv v heads
  T* x = qkv + (size_t)t * row_stride + (size_t)head * d;
  const float* b = bias ? bias + (size_t)head * d : nullptr;
  const int half = d / 2;
  const bool is_v = head >= n_q + n_kv;
  const bool is_k = !is_v && head >= n_q;
  T* dst = nullptr;
  int dst_stride = 1;   // distance between consecutive elements of the head in the page
  if ((is_k || is_v) && slots) {
    const int slot = slots[t];
    if (slot >= 0) {
      const int page = slot / page_size, off = slot - page * page_size;
      const int kvh = is_k ? head - n_q : head - n_q - n_kv;
      T* base = (is_k ? k_pages : v_pages) + ((size_t)page * n_kv + kvh) * page_size * d;
      if (is_k) dst = base + (size_t)off * d;
      else { dst = base + off; dst_stride = page_size; }
    }
  }
  if (is_v || !cos_sin) {
    if (!b && !dst) return;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      float v = ld(x + i);
      if (b) { v += b[i]; st(x + i, v); }
      if (dst) st(dst + (size_t)i * dst_stride, v);
    }
    return;
  }
  const float* cs = cos_sin + (size_t)positions[t] * d;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float x1 = ld(x + i), x2 = ld(x + half + i);
    if (b) { x1 += b[i]; x2 += b[half + i]; }
    const float c = cs[i], s = cs[half + i];
    const float r1 = x1 * c - x2 * s;
    const float r2 = x2 * c + x1 * s;
    st(x + i, r1);
    st(x + half + i, r2);
    if (dst) { st(dst + i, r1); st(dst + half + i, r2); }
  }
}

// The same for bfloat16 with head sizes that are multiples of 16, eight elements per thread: a unit is one
// 16-byte piece of the first half of a q or k head together with its partner in the second half, or one
// 16-byte piece of a v head.  Units of all tokens are laid out on one axis.
typedef __bf16 rk_bf16x8 __attribute__((ext_vector_type(8)));

__global__ void __launch_bounds__(256)
rope_store_vec_kernel(bf16_t* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                      const int* __restrict__ positions, const float* __restrict__ cos_sin,
                      const int* __restrict__ slots, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages,
                      int n_tokens, int n_q, int n_kv, int d, int page_size) {
  const int half = d / 2, per_half = half / 8, per_head = d / 8;
  const int rot_units = (n_q + n_kv) * per_half, units = rot_units + n_kv * per_head;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n_tokens * units) return;
  const int t = (int)(idx / units), u = (int)(idx % units);
  bf16_t* row = qkv + (size_t)t * row_stride;
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  if (u < rot_units) {
    const int head = u / per_half, i = (u % per_half) * 8;
    bf16_t* x = row + (size_t)head * d + i;
    rk_bf16x8 a = *reinterpret_cast<const rk_bf16x8*>(x), b = *reinterpret_cast<const rk_bf16x8*>(x + half);
    float x1[8], x2[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x1[j] = (float)a[j];
      x2[j] = (float)b[j];
      if (bias) { x1[j] += bias[head * d + i + j]; x2[j] += bias[head * d + half + i + j]; }
    }
    if (cos_sin) {
      const float* cs = cos_sin + (size_t)positions[t] * d + i;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float c = cs[j], sn = cs[half + j];
        const float r1 = x1[j] * c - x2[j] * sn, r2 = x2[j] * c + x1[j] * sn;
        x1[j] = r1;
        x2[j] = r2;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)x1[j]; b[j] = (__bf16)x2[j]; }
    if (bias || cos_sin) {
      *reinterpret_cast<rk_bf16x8*>(x) = a;
      *reinterpret_cast<rk_bf16x8*>(x + half) = b;
    }
    if (head >= n_q && slot >= 0) {
      bf16_t* dst = k_pages + (((size_t)page * n_kv + (head - n_q)) * page_size + off) * d + i;
      *reinterpret_cast<rk_bf16x8*>(dst) = a;
      *reinterpret_cast<rk_bf16x8*>(dst + half) = b;
    }
  } else {
    const int v = u - rot_units, kvh = v / per_head, i = (v % per_head) * 8;
    bf16_t* x = row + (size_t)(n_q + n_kv + kvh) * d + i;
    rk_bf16x8 a = *reinterpret_cast<const rk_bf16x8*>(x);
    if (bias) {
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] = (__bf16)((float)a[j] + bias[(n_q + n_kv + kvh) * d + i + j]);
      *reinterpret_cast<rk_bf16x8*>(x) = a;
    }
    if (slot >= 0) {
      bf16_t* dst = v_pages + (((size_t)page * n_kv + kvh) * d + i) * page_size + off;
      union { __bf16 h; uint16_t bits; } cvt;
#pragma unroll
      for (int j = 0; j < 8; ++j) { cvt.h = a[j]; dst[(size_t)j * page_size].bits = cvt.bits; }
    }
  }
}

extern "C" int ta_rope_store(void* qkv, int row_stride, const void* bias, const void* positions,
                             const void* cos_sin, const void* slots, void* k_pages, void* v_pages,
                             int n_tokens, int n_q, int n_kv, int d, int page_size, int dtype,
                             hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (dtype == DT_BF16 && d % 16 == 0 && row_stride % 8 == 0) {
    const long units = (long)n_tokens * ((n_q + n_kv) * (d / 16) + n_kv * (d / 8));
    rope_store_vec_kernel<<<(int)((units + 255) / 256), 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, (const float*)bias, (const int*)positions, (const float*)cos_sin,
        (const int*)slots, (bf16_t*)k_pages, (bf16_t*)v_pages, n_tokens, n_q, n_kv, d, page_size);
    return LAUNCH_STATUS();
  }
  dim3 grid(n_tokens, n_q + 2 * n_kv);
  if (dtype == DT_F32)
    rope_store_kernel<float><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, (const float*)bias, (const int*)positions,
        (const float*)cos_sin, (const int*)slots, (float*)k_pages, (float*)v_pages, n_q, n_kv, d, page_size);
  else
    rope_store_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, (const float*)bias, (const int*)positions,
        (const float*)cos_sin, (const int*)slots, (bf16_t*)k_pages, (bf16_t*)v_pages, n_q, n_kv, d, page_size);
  return LAUNCH_STATUS();
}
