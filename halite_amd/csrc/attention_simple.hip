// Paged attention, the plain way: one wavefront per (token, query head), any head
// size that is a multiple of 2 up to 512, any page size, any number of heads and
// groups, float32 or bf16 storage, float32 arithmetic throughout.  It is the whole
// attention of the 32-bit path and the fallback of the bf16 path for shapes that
// the matrix-core kernel refuses.  A row's result depends only on the row's own
// position and request: the keys are visited in order, 64 at a time.
//
// scores, mask, softmax and weighted sum as in
// src/halite/transformers/attention.py:647-714; the causal rule for a portion that
// follows cached tokens (key j visible to the query at position p iff j <= p) is
// the one of src/halite/transformers/infer/engine/flashinfer_backend.py:217-229.
#include "hal_common.h"
#include "hal_api.h"

#define SIMPLE_MAX_ACC 8  // head sizes up to 64 * 8

template <typename T>
__global__ void __launch_bounds__(HAL_WAVE)
attention_simple_kernel(const T* __restrict__ q, int q_row_stride, T* __restrict__ out,
                        int out_row_stride, const int* __restrict__ positions,
                        const int* __restrict__ token_seg, const int* __restrict__ block_table,
                        int bt_stride, const T* __restrict__ k_pages,
                        const T* __restrict__ v_pages, int H, int K, int D, int page_size,
                        int n_pages, float scale, int window) {
  extern __shared__ float smem[];
  float* q_s = smem;                            // [D]
  float* p_s = smem + D;                        // [64]
  long long* base_s = (long long*)(p_s + 64);   // [64] page * K + g, or -1
  int* off_s = (int*)(base_s + 64);             // [64]

  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / K);
  const int p = positions[t];
  const int seg = token_seg[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_table + (size_t)seg * bt_stride;

  const T* qp = q + (size_t)t * q_row_stride + (size_t)h * D;
  for (int i = lane; i < D; i += HAL_WAVE) q_s[i] = to_f32(qp[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[SIMPLE_MAX_ACC];
#pragma unroll
  for (int r = 0; r < SIMPLE_MAX_ACC; ++r) acc[r] = 0.f;

  for (int j0 = lo; j0 <= p; j0 += HAL_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= p;
    long long base = -1;
    int off = 0;
    float s = -INFINITY;
    if (valid) {
      const long long page = bt[j / page_size];
      off = j % page_size;
      if (page >= 0 && page < n_pages) {
        base = page * K + g;
        const T* kp = k_pages + ((size_t)base * page_size + off) * D;
        float dot = 0.f;
        for (int i = 0; i < D; ++i) dot += q_s[i] * to_f32(kp[i]);
        s = dot * scale;
      } else {
        s = __uint_as_float(0x7fc00000u);  // a hole in the block table must show
      }
    }
    const float m_tile = wave_max(s);
    const float m_new = fmaxf(m, m_tile);
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float pj = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(pj);
    m = m_new;
    p_s[lane] = pj;
    base_s[lane] = base;
    off_s[lane] = off;
    __syncthreads();
    const int n_valid = (p - j0 + 1) < HAL_WAVE ? (p - j0 + 1) : HAL_WAVE;
#pragma unroll
    for (int r = 0; r < SIMPLE_MAX_ACC; ++r) {
      const int i = lane + r * HAL_WAVE;
      if (i < D) {
        float a = acc[r] * alpha;
        for (int jj = 0; jj < n_valid; ++jj) {
          const long long b = base_s[jj];
          if (b >= 0)
            a += p_s[jj] * to_f32(v_pages[((size_t)b * D + i) * page_size + off_s[jj]]);
        }
        acc[r] = a;
      }
    }
    __syncthreads();
  }
  T* op = out + (size_t)t * out_row_stride + (size_t)h * D;
  const float inv = 1.0f / l;
#pragma unroll
  for (int r = 0; r < SIMPLE_MAX_ACC; ++r) {
    const int i = lane + r * HAL_WAVE;
    if (i < D) op[i] = from_f32<T>(acc[r] * inv);
  }
}

extern "C" int hal_attention_simple(const void* q, int q_row_stride, void* out,
                                    int out_row_stride, int dtype, const int* positions,
                                    const int* token_seg, const int* block_table, int bt_stride,
                                    const void* k_pages, const void* v_pages, int n_tokens, int H,
                                    int K, int D, int page_size, int n_pages, float scale,
                                    int window, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && K > 0 && D > 0 && page_size > 0 && n_pages > 0,
              "hal_attention_simple: bad sizes T=%d H=%d K=%d D=%d page=%d pages=%d", n_tokens, H,
              K, D, page_size, n_pages);
  HAL_REQUIRE(H % K == 0, "hal_attention_simple: %d query heads are not a multiple of %d kv heads",
              H, K);
  HAL_REQUIRE(D <= HAL_WAVE * SIMPLE_MAX_ACC, "hal_attention_simple: head size %d > %d", D,
              HAL_WAVE * SIMPLE_MAX_ACC);
  HAL_REQUIRE(H <= 65535, "hal_attention_simple: %d heads exceed the grid limit", H);
  HAL_REQUIRE(window >= 0, "hal_attention_simple: window %d", window);
  if (n_tokens == 0) return 0;
  const size_t smem = (size_t)D * sizeof(float) + 64 * sizeof(float) + 64 * sizeof(long long) +
                      64 * sizeof(int);
  dim3 grid(n_tokens, H);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(attention_simple_kernel<float>, grid, dim3(HAL_WAVE), smem, stream,
                       (const float*)q, q_row_stride, (float*)out, out_row_stride, positions,
                       token_seg, block_table, bt_stride, (const float*)k_pages,
                       (const float*)v_pages, H, K, D, page_size, n_pages, scale, window);
  else if (dtype == HAL_BF16)
    hipLaunchKernelGGL(attention_simple_kernel<bf16_t>, grid, dim3(HAL_WAVE), smem, stream,
                       (const bf16_t*)q, q_row_stride, (bf16_t*)out, out_row_stride, positions,
                       token_seg, block_table, bt_stride, (const bf16_t*)k_pages,
                       (const bf16_t*)v_pages, H, K, D, page_size, n_pages, scale, window);
  else
    return hal_fail("hal_attention_simple: unknown dtype %d", dtype);
  HAL_LAUNCH_CHECK();
  return 0;
}
