// Attention over paged keys and values, one block per (token, query head), any storage type.
// Plain float arithmetic (no matrix cores): this is the kernel of the 32-bit path and the
// yardstick for the faster bfloat16 kernels.  Softmax runs online in float.
#include "common.h"

#define ATT_WAVES 4
#define ATT_MAX_D 256

// q: rows of `q_stride` elements, head h at h*d.  out: [n_tokens, n_q*d].
// Token t at position p of entry e sees keys max(0, p-window)..p (window < 0: all from 0), whose
// pages are block_table[e, key / page_size]; a token of entry -1 is passed over (its output row is not written).  Key pages: [n_pages, n_kv, page_size, d]; value pages
// are transposed inside a page: [n_pages, n_kv, d, page_size].
template <typename T>
__global__ void __launch_bounds__(ATT_WAVES * WAVE)
paged_attention_generic(const T* __restrict__ q, int q_stride, T* __restrict__ out,
                        const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                        const int* __restrict__ positions, const int* __restrict__ entry_of_token,
                        const int* __restrict__ block_table, int table_stride,
                        int n_q, int n_kv, int d, int page_size, int window, float scale) {
  __shared__ float q_s[ATT_MAX_D];
  __shared__ float acc_s[ATT_WAVES][ATT_MAX_D];
  __shared__ float m_s[ATT_WAVES], l_s[ATT_WAVES];
  __shared__ float p_s[ATT_WAVES][WAVE];
  const int t = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int entry = entry_of_token[t];
  if (entry < 0) return;                                   // a token that only fills the batch up: it belongs to no request
  const int pos = positions[t];
  const int* table = block_table + (size_t)entry * table_stride;
  const int kvh = h / (n_q / n_kv);
  const int lo = (window >= 0 && pos > window) ? pos - window : 0;
  const int n_keys = pos - lo + 1;

  for (int i = threadIdx.x; i < d; i += blockDim.x) q_s[i] = ld(q + (size_t)t * q_stride + (size_t)h * d + i);
  __syncthreads();

  float acc[ATT_MAX_D / WAVE] = {0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  for (int base = wave * WAVE; base < n_keys; base += ATT_WAVES * WAVE) {
    const int j = lo + base + lane;
    const bool valid = base + lane < n_keys;
    int row = 0, vbase = 0;   // key row, and start of this key's column in the value page
    float s = -INFINITY;
    if (valid) {
      const int page = table[j / page_size];
      row = (page * n_kv + kvh) * page_size + (j % page_size);
      vbase = (page * n_kv + kvh) * page_size * d + (j % page_size);
      const T* kr = k_pages + (size_t)row * d;
      float dot = 0.f;
      if (sizeof(T) == 4 && d % 4 == 0) {
        // A lane walks its key's row sixteen bytes at a time (rows are 16-byte aligned: d is a multiple of 4).
        for (int i = 0; i < d; i += 4) {
          const float4 kv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(kr) + i);
          dot = fmaf(q_s[i], kv.x, fmaf(q_s[i + 1], kv.y, fmaf(q_s[i + 2], kv.z, fmaf(q_s[i + 3], kv.w, dot))));
        }
      } else {
        for (int i = 0; i < d; ++i) dot += q_s[i] * ld(kr + i);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first chunk gives 0
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int r = 0; r < ATT_MAX_D / WAVE; ++r) acc[r] *= corr;
    const int count = min(WAVE, n_keys - base);
    if (sizeof(T) == 4 && page_size % 4 == 0) {
      // Values lie transposed inside a page, [d, page_size]: lane i walks row i of the page sixteen bytes (four
      // keys) at a time, so that the wave reads the page as one contiguous block; the keys' weights come through
      // LDS.  (One key at a time, every lane's element would lie a row apart from its neighbour's.)
      p_s[wave][lane] = p;
      __builtin_amdgcn_wave_barrier();
      int jj = 0;
      while (jj < count) {
        const int j = lo + base + jj;
        const int off = j % page_size;
        const int run = min(count - jj, page_size - off);
        const float* page_v = reinterpret_cast<const float*>(v_pages) +
                              ((size_t)table[j / page_size] * n_kv + kvh) * d * page_size + off;
        if (off % 4 == 0 && run >= 4) {
          for (int q4 = 0; q4 + 4 <= run; q4 += 4) {
            const float p0 = p_s[wave][jj + q4], p1 = p_s[wave][jj + q4 + 1], p2 = p_s[wave][jj + q4 + 2],
                        p3 = p_s[wave][jj + q4 + 3];
#pragma unroll
            for (int r = 0; r < ATT_MAX_D / WAVE; ++r) {
              const int i = lane + r * WAVE;
              if (i < d) {
                const float4 v4 = *reinterpret_cast<const float4*>(page_v + (size_t)i * page_size + q4);
                acc[r] = fmaf(p0, v4.x, fmaf(p1, v4.y, fmaf(p2, v4.z, fmaf(p3, v4.w, acc[r]))));
              }
            }
          }
          jj += run / 4 * 4;
        } else {
          const float pj = p_s[wave][jj];
#pragma unroll
          for (int r = 0; r < ATT_MAX_D / WAVE; ++r) {
            const int i = lane + r * WAVE;
            if (i < d) acc[r] += pj * page_v[(size_t)i * page_size];
          }
          ++jj;
        }
      }
      __builtin_amdgcn_wave_barrier();
    } else {
      for (int jj = 0; jj < count; ++jj) {
        const float pj = __shfl(p, jj, WAVE);
        const T* vr = v_pages + (size_t)__shfl(vbase, jj, WAVE);
#pragma unroll
        for (int r = 0; r < ATT_MAX_D / WAVE; ++r) {
          const int i = lane + r * WAVE;
          if (i < d) acc[r] += pj * ld(vr + (size_t)i * page_size);
        }
      }
    }
    m = m_new;
  }
#pragma unroll
  for (int r = 0; r < ATT_MAX_D / WAVE; ++r) {
    const int i = lane + r * WAVE;
    if (i < d) acc_s[wave][i] = acc[r];
  }
  if (lane == 0) { m_s[wave] = m; l_s[wave] = l; }
  __syncthreads();
  float big = -INFINITY;
  for (int w = 0; w < ATT_WAVES; ++w) big = fmaxf(big, m_s[w]);
  float denom = 0.f;
  float weights[ATT_WAVES];
  for (int w = 0; w < ATT_WAVES; ++w) {
    weights[w] = (m_s[w] == -INFINITY) ? 0.f : expf(m_s[w] - big);
    denom += l_s[w] * weights[w];
  }
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = 0.f;
    for (int w = 0; w < ATT_WAVES; ++w) v += acc_s[w][i] * weights[w];
    st(out + (size_t)t * n_q * d + (size_t)h * d + i, v / denom);
  }
}

extern "C" int ta_paged_attention_generic(const void* q, int q_stride, void* out, const void* k_pages,
                                          const void* v_pages, const void* positions, const void* entry_of_token,
                                          const void* block_table, int table_stride, int n_tokens, int n_q,
                                          int n_kv, int d, int page_size, int window, float scale, int dtype,
                                          hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (d > ATT_MAX_D || d <= 0 || n_kv <= 0 || n_q % n_kv) return -1;
  dim3 grid(n_tokens, n_q);
  if (dtype == DT_F32)
    paged_attention_generic<float><<<grid, ATT_WAVES * WAVE, 0, stream>>>((const float*)q, q_stride, (float*)out,
        (const float*)k_pages, (const float*)v_pages, (const int*)positions, (const int*)entry_of_token,
        (const int*)block_table, table_stride, n_q, n_kv, d, page_size, window, scale);
  else
    paged_attention_generic<bf16_t><<<grid, ATT_WAVES * WAVE, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out,
        (const bf16_t*)k_pages, (const bf16_t*)v_pages, (const int*)positions, (const int*)entry_of_token,
        (const int*)block_table, table_stride, n_q, n_kv, d, page_size, window, scale);
  return LAUNCH_STATUS();
}
