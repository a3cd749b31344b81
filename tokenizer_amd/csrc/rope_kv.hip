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

__device__ __forceinline__ float4 rk_ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }

// BIAS, ROTATE: whether there is a bias, an angle table (choices made when the kernel is compiled: a value loaded
// behind a condition is copied where the branches meet, and the copy waits for the load).  A thread asks for
// everything it needs at its start (slot and position; its sixteen elements; their bias, sixteen bytes a load) and
// for the angles as soon as the position is there: two trips to memory, where an element after the other they
// were a dozen.
template <bool BIAS, bool ROTATE>
__global__ void __launch_bounds__(256)
rope_store_vec_kernel(bf16_t* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                      const int* __restrict__ positions, const float* __restrict__ cos_sin,
                      const int* __restrict__ slots, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages,
                      int n_tokens, int n_q, int n_kv, int d, int page_size) {
  HELD(qkv, row_stride, bias, positions, cos_sin, slots, k_pages, v_pages, n_tokens, n_q, n_kv, d, page_size);
  const int half = d / 2, per_half = half / 8, per_head = d / 8;
  const int rot_units = (n_q + n_kv) * per_half, units = rot_units + n_kv * per_head;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n_tokens * units) return;
  const int t = (int)(idx / units), u = (int)(idx % units);
  bf16_t* row = qkv + (size_t)t * row_stride;
  const int position = ROTATE ? positions[t] : 0;
  const int slot = slots ? slots[t] : -1;
  if (u < rot_units) {
    const int head = u / per_half, i = (u % per_half) * 8;
    bf16_t* x = row + (size_t)head * d + i;
    rk_bf16x8 a = *reinterpret_cast<const rk_bf16x8*>(x), b = *reinterpret_cast<const rk_bf16x8*>(x + half);
    float4 bias1[2], bias2[2], cosine[2], sine[2];
    if (BIAS) {
      const float* at = bias + head * d + i;
      bias1[0] = rk_ld4(at); bias1[1] = rk_ld4(at + 4);
      bias2[0] = rk_ld4(at + half); bias2[1] = rk_ld4(at + half + 4);
    }
    if (ROTATE) {
      const float* cs = cos_sin + (size_t)position * d + i;
      cosine[0] = rk_ld4(cs); cosine[1] = rk_ld4(cs + 4);
      sine[0] = rk_ld4(cs + half); sine[1] = rk_ld4(cs + half + 4);
    }
    float x1[8], x2[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x1[j] = (float)a[j];
      x2[j] = (float)b[j];
    }
    if (BIAS) {
      const float add1[8] = {bias1[0].x, bias1[0].y, bias1[0].z, bias1[0].w, bias1[1].x, bias1[1].y, bias1[1].z, bias1[1].w};
      const float add2[8] = {bias2[0].x, bias2[0].y, bias2[0].z, bias2[0].w, bias2[1].x, bias2[1].y, bias2[1].z, bias2[1].w};
#pragma unroll
      for (int j = 0; j < 8; ++j) { x1[j] += add1[j]; x2[j] += add2[j]; }
    }
    if (ROTATE) {
      const float c[8] = {cosine[0].x, cosine[0].y, cosine[0].z, cosine[0].w, cosine[1].x, cosine[1].y, cosine[1].z, cosine[1].w};
      const float sn[8] = {sine[0].x, sine[0].y, sine[0].z, sine[0].w, sine[1].x, sine[1].y, sine[1].z, sine[1].w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float r1 = x1[j] * c[j] - x2[j] * sn[j], r2 = x2[j] * c[j] + x1[j] * sn[j];
        x1[j] = r1;
        x2[j] = r2;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)x1[j]; b[j] = (__bf16)x2[j]; }
    if (BIAS || ROTATE) {
      *reinterpret_cast<rk_bf16x8*>(x) = a;
      *reinterpret_cast<rk_bf16x8*>(x + half) = b;
    }
    if (head >= n_q && slot >= 0) {
      const int page = slot / page_size, off = slot % page_size;
      bf16_t* dst = k_pages + (((size_t)page * n_kv + (head - n_q)) * page_size + off) * d + i;
      *reinterpret_cast<rk_bf16x8*>(dst) = a;
      *reinterpret_cast<rk_bf16x8*>(dst + half) = b;
    }
  } else {
    const int v = u - rot_units, kvh = v / per_head, i = (v % per_head) * 8;
    bf16_t* x = row + (size_t)(n_q + n_kv + kvh) * d + i;
    rk_bf16x8 a = *reinterpret_cast<const rk_bf16x8*>(x);
    if (BIAS) {
      const float* at = bias + (n_q + n_kv + kvh) * d + i;
      const float4 lo = rk_ld4(at), hi = rk_ld4(at + 4);
      const float add[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] = (__bf16)((float)a[j] + add[j]);
      *reinterpret_cast<rk_bf16x8*>(x) = a;
    }
    if (slot >= 0) {
      const int page = slot / page_size, off = slot % page_size;
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
  if (dtype == DT_BF16 && d % 16 == 0 && row_stride % 8 == 0 && (((uintptr_t)bias | (uintptr_t)cos_sin) & 15) == 0) {
    const long units = (long)n_tokens * ((n_q + n_kv) * (d / 16) + n_kv * (d / 8));
#define GO(BB, RR) rope_store_vec_kernel<BB, RR><<<(int)((units + 255) / 256), 256, 0, stream>>>( \
        (bf16_t*)qkv, row_stride, (const float*)bias, (const int*)positions, (const float*)cos_sin, \
        (const int*)slots, (bf16_t*)k_pages, (bf16_t*)v_pages, n_tokens, n_q, n_kv, d, page_size)
    if (bias) { if (cos_sin) GO(true, true); else GO(true, false); }
    else { if (cos_sin) GO(false, true); else GO(false, false); }
#undef GO
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
