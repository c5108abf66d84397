// Embedding lookup, RMSNorm (with the residual add and a row gather fused in),
// SiLU-gate multiply, and rotary position encoding fused with the append of keys
// and values to their cache pages.  All arithmetic is float32; T is the element
// type of activations and cache (float or bf16).
#include "hal_common.h"
#include "hal_api.h"
#include <stdlib.h>

// ---------------------------------------------------------------------------------
// h[t, :] = table[ids[t], :]  (float32 residual stream)
// src/halite/transformers/embedding.py:36-44
// ---------------------------------------------------------------------------------
template <typename TT>
__global__ void embedding_kernel(const int* __restrict__ ids, const TT* __restrict__ table,
                                 float* __restrict__ out, int d, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* o = out + (size_t)t * d;
  if (id < 0 || id >= vocab) {
    // an id outside the table is a caller's fault; make it visible, not a fault
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const TT* row = table + (size_t)id * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = to_f32(row[i]);
}

// four elements per access; d is a multiple of 4
template <typename TT>
__global__ void embedding_vec_kernel(const int* __restrict__ ids, const TT* __restrict__ table,
                                     float* __restrict__ out, int d, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* o = out + (size_t)t * d;
  const bool ok = id >= 0 && id < vocab;
  const TT* row = table + (size_t)(ok ? id : 0) * d;
  for (int i = threadIdx.x * 4; i < d; i += blockDim.x * 4) {
    float v[4];
    load4(row + i, v);
    if (!ok) v[0] = v[1] = v[2] = v[3] = __uint_as_float(0x7fc00000u);
    store4(o + i, v);
  }
}

// Token ids that an earlier step left on the device: tokens[i] holds a row of `src` on
// entry and that row's value on return.
__global__ void take_tokens_kernel(const int* __restrict__ src, int n_src, int* __restrict__ tokens,
                                   int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r = tokens[i];
  tokens[i] = (r >= 0 && r < n_src) ? src[r] : 0;
}

extern "C" int hal_take_tokens(const int* src, int n_src, int* tokens, int n, hipStream_t stream) {
  HAL_REQUIRE(n >= 0 && n_src > 0, "hal_take_tokens: bad sizes n=%d n_src=%d", n, n_src);
  if (n == 0) return 0;
  hipLaunchKernelGGL(take_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, src, n_src,
                     tokens, n);
  HAL_LAUNCH_CHECK();
  return 0;
}

extern "C" int hal_embedding(const int* ids, const void* table, int table_dtype, float* out,
                             int n_tokens, int d, int vocab, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && d > 0 && vocab > 0, "hal_embedding: bad sizes T=%d d=%d V=%d",
              n_tokens, d, vocab);
  if (n_tokens == 0) return 0;
  HAL_REQUIRE(table_dtype == HAL_F32 || table_dtype == HAL_BF16,
              "hal_embedding: unknown table dtype %d", table_dtype);
  if (d % 4 == 0) {
    int threads = ((d / 4 + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
    if (table_dtype == HAL_F32)
      hipLaunchKernelGGL(embedding_vec_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream,
                         ids, (const float*)table, out, d, vocab);
    else
      hipLaunchKernelGGL(embedding_vec_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream,
                         ids, (const bf16_t*)table, out, d, vocab);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const int threads = d >= 1024 ? 256 : 64;
  if (table_dtype == HAL_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream, ids,
                       (const float*)table, out, d, vocab);
  else
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream, ids,
                       (const bf16_t*)table, out, d, vocab);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// RMSNorm over the float32 residual stream.
//   x = h[src] (+ delta[src]);  h[src] = x when update_h
//   out[r] = w * T(x * rsqrt(mean(x^2) + eps))
// src = rows[r] if rows is given, else r.  The statistics and the scaling are
// float32; the normalised value is rounded to T before the weight multiplies it,
// as src/halite/nn/normalization.py:43-57 does.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ delta,
                               const int* __restrict__ rows, const void* __restrict__ w,
                               int w_dtype, float eps, T* __restrict__ out, int d, int update_h) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* hr = h + (size_t)src * d;
  const T* dr = delta ? delta + (size_t)src * d : nullptr;
  T* o = out + (size_t)r * d;

  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float x = hr[i];
    if (dr) x += to_f32(dr[i]);
    ss += x * x;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float x = hr[i];
    if (dr) {
      x += to_f32(dr[i]);
      if (update_h) hr[i] = x;
    }
    const T n = from_f32<T>(x * rstd);
    o[i] = from_f32<T>(load_as_f32(w, w_dtype, i) * to_f32(n));
  }
}

// The same with the row held in registers: one pass over memory, four elements per
// access, all loads issued before the first use.  d is a multiple of 4 and at most
// 4 * RMS_MAXV * blockDim.x.
#define RMS_MAXV 8
template <typename T>
__global__ void rmsnorm_vec_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                   const int* __restrict__ rows, const void* __restrict__ w,
                                   int w_dtype, float eps, T* __restrict__ out, int d,
                                   int update_h) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* hr = h + (size_t)src * d;
  const T* dr = delta ? delta + (size_t)src * d : nullptr;
  T* o = out + (size_t)r * d;
  const int nv = d / 4;

  // the weight does not depend on the row: asked for with the row, not after the sum
  float x[RMS_MAXV][4], wv[RMS_MAXV][4];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < RMS_MAXV; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < nv) {
      load4(hr + v * 4, x[u]);
      load4_any(w, w_dtype, (size_t)v * 4, wv[u]);
    }
  }
  if (dr) {
#pragma unroll
    for (int u = 0; u < RMS_MAXV; ++u) {
      const int v = threadIdx.x + u * blockDim.x;
      if (v < nv) {
        float dv[4];
        load4(dr + v * 4, dv);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[u][i] += dv[i];
        if (update_h) store4(hr + v * 4, x[u]);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < RMS_MAXV; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < nv) {
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += x[u][i] * x[u][i];
    }
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)d + eps);
#pragma unroll
  for (int u = 0; u < RMS_MAXV; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < nv) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = wv[u][i] * to_f32(from_f32<T>(x[u][i] * rstd));
      store4(o + v * 4, y);
    }
  }
}

template <typename T>
static void launch_rmsnorm(float* h, const void* delta, const int* rows, const void* w,
                           int w_dtype, float eps, void* out, int n_rows, int d, int update_h,
                           hipStream_t stream) {
  if (d % 4 == 0 && d / 4 <= RMS_MAXV * 1024) {
    int threads = ((d / 4 + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
    // many rows: small blocks with all RMS_MAXV vectors per thread, so that a CU holds rows
    // in every phase (loading, summing, storing) at once (2,048 rows of 4,096: 19 us with 128
    // threads, 20 with 256, 23 with 512, 29 with 1,024)
    if (n_rows >= 256) threads = ((d / 4 + RMS_MAXV - 1) / RMS_MAXV + 63) / 64 * 64;
    hipLaunchKernelGGL(rmsnorm_vec_kernel<T>, dim3(n_rows), dim3(threads), 0, stream, h,
                       (const T*)delta, rows, w, w_dtype, eps, (T*)out, d, update_h);
  } else {
    const int threads = d >= 2048 ? 512 : (d >= 512 ? 256 : 64);
    hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3(n_rows), dim3(threads), 0, stream, h,
                       (const T*)delta, rows, w, w_dtype, eps, (T*)out, d, update_h);
  }
}

extern "C" int hal_rmsnorm(float* h, const void* delta, const int* rows, const void* w,
                           int w_dtype, float eps, void* out, int dtype, int n_rows, int d,
                           int update_h, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && d > 0, "hal_rmsnorm: bad sizes rows=%d d=%d", n_rows, d);
  HAL_REQUIRE(w_dtype == HAL_F32 || w_dtype == HAL_BF16, "hal_rmsnorm: weight dtype %d", w_dtype);
  HAL_REQUIRE(!(rows && update_h && delta),
              "hal_rmsnorm: a gathered call must not update the residual stream");
  if (n_rows == 0) return 0;
  if (dtype == HAL_F32)
    launch_rmsnorm<float>(h, delta, rows, w, w_dtype, eps, out, n_rows, d, update_h, stream);
  else if (dtype == HAL_BF16)
    launch_rmsnorm<bf16_t>(h, delta, rows, w, w_dtype, eps, out, n_rows, d, update_h, stream);
  else
    return hal_fail("hal_rmsnorm: unknown dtype %d", dtype);
  HAL_LAUNCH_CHECK();
  return 0;
}

// h += delta (float32 stream, delta of type T); used for the last pending delta.
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ delta, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) h[i] += to_f32(delta[i]);
}

extern "C" int hal_residual_add(float* h, const void* delta, int dtype, long long n,
                                hipStream_t stream) {
  HAL_REQUIRE(n >= 0, "hal_residual_add: n=%lld", n);
  if (n == 0) return 0;
  const int threads = 256;
  const int blocks = (int)((n + threads - 1) / threads < 4096 ? (n + threads - 1) / threads : 4096);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(residual_add_kernel<float>, dim3(blocks), dim3(threads), 0, stream, h,
                       (const float*)delta, (size_t)n);
  else if (dtype == HAL_BF16)
    hipLaunchKernelGGL(residual_add_kernel<bf16_t>, dim3(blocks), dim3(threads), 0, stream, h,
                       (const bf16_t*)delta, (size_t)n);
  else
    return hal_fail("hal_residual_add: unknown dtype %d", dtype);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// out[t, f] = up[t, f] * silu(gate[t, f]); gate and up are the two halves of one
// row of `gu` ([T, 2F], gate first).  silu(x) = x * sigmoid(x) in float32.
// src/halite/transformers/feedforward.py:204-212
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens,
                                int F) {
  const size_t n = (size_t)n_tokens * F;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const size_t t = i / F, f = i % F;
    const float g = to_f32(gu[t * 2 * F + f]);
    const float u = to_f32(gu[t * 2 * F + F + f]);
    const float s = g / (1.0f + expf(-g));
    out[i] = from_f32<T>(u * s);
  }
}

// ---- the scaling that an RMSNorm left to its reader ----------------------------------------
// A product has written x = bf16(w * bf16(h)) and, per row, partial sums of h^2 (ss
// [n_parts][row_width]); the norm's output is x * rsqrt(sum / d + eps).  Readers that
// cannot scale their own result get the rows from here.  One block per row; the partial
// sums are added in a fixed order (thread by thread, then lanes, then waves).
__global__ void __launch_bounds__(256)
scale_normed_rows_kernel(const bf16_t* __restrict__ x, int ldx, const float* __restrict__ ss,
                         int n_parts, int row_width, float eps, bf16_t* __restrict__ out, int d) {
  __shared__ float red[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  float sum = 0.f;
  for (int p = tid; p < n_parts; p += 256) sum += ss[(size_t)p * row_width + row];
  sum = block_sum(sum, red);
  const float rstd = rsqrtf(sum / (float)d + eps);
  for (int c = tid; c < d; c += 256)
    out[(size_t)row * d + c] = f32_to_bf16(bf16_to_f32(x[(size_t)row * ldx + c]) * rstd);
}

extern "C" int hal_scale_normed_rows(const void* x, int ldx, const float* ss, int n_parts,
                                     int row_width, float eps, void* out, int m, int d,
                                     hipStream_t stream) {
  HAL_REQUIRE(m >= 0 && d > 0 && ldx >= d && n_parts > 0 && eps > 0.f,
              "hal_scale_normed_rows: bad sizes m=%d d=%d ldx=%d parts=%d", m, d, ldx, n_parts);
  HAL_REQUIRE(m <= row_width, "hal_scale_normed_rows: %d rows, sums of squares for %d", m, row_width);
  if (m == 0) return 0;
  HAL_REQUIRE(x && ss && out, "hal_scale_normed_rows: arguments missing");
  hipLaunchKernelGGL(scale_normed_rows_kernel, dim3(m), dim3(256), 0, stream, (const bf16_t*)x, ldx, ss,
                     n_parts, row_width, eps, (bf16_t*)out, d);
  HAL_LAUNCH_CHECK();
  return 0;
}

// four elements per access; F is a multiple of 4
template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens,
                                    int F) {
  const int f4 = F / 4;
  const size_t n = (size_t)n_tokens * f4;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const size_t t = i / f4, f = (i % f4) * 4;
    float g[4], u[4], y[4];
    load4(gu + t * 2 * F + f, g);
    load4(gu + t * 2 * F + F + f, u);
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = u[e] * (g[e] / (1.0f + expf(-g[e])));
    store4(out + t * F + f, y);
  }
}

extern "C" int hal_silu_mul(const void* gu, void* out, int dtype, int n_tokens, int F,
                            hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && F > 0, "hal_silu_mul: bad sizes T=%d F=%d", n_tokens, F);
  if (n_tokens == 0) return 0;
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_silu_mul: unknown dtype %d", dtype);
  if (F % 4 == 0) {
    const size_t n4 = (size_t)n_tokens * (F / 4);
    const size_t want4 = (n4 + 255) / 256;
    const int blocks4 = (int)(want4 < 16384 ? want4 : 16384);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(silu_mul_vec_kernel<float>, dim3(blocks4), dim3(256), 0, stream,
                         (const float*)gu, (float*)out, n_tokens, F);
    else
      hipLaunchKernelGGL(silu_mul_vec_kernel<bf16_t>, dim3(blocks4), dim3(256), 0, stream,
                         (const bf16_t*)gu, (bf16_t*)out, n_tokens, F);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const size_t n = (size_t)n_tokens * F;
  const int threads = 256;
  const size_t want = (n + threads - 1) / threads;
  const int blocks = (int)(want < 8192 ? want : 8192);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(blocks), dim3(threads), 0, stream,
                       (const float*)gu, (float*)out, n_tokens, F);
  else if (dtype == HAL_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, dim3(blocks), dim3(threads), 0, stream,
                       (const bf16_t*)gu, (bf16_t*)out, n_tokens, F);
  else
    return hal_fail("hal_silu_mul: unknown dtype %d", dtype);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// Rotary position encoding of q and k, in place in the packed row
// [q heads | k heads | v heads], and the append of the rotated k and of v to the
// cache pages of the token's request.
//   half-split pairs (j, j + rot/2):  src/halite/transformers/position.py:287-291
//   adjacent pairs (2j, 2j + 1):      src/halite/transformers/position.py:294-300
// The angle table is float32 [table_len, rot/2] (position.py:140-167); the
// rotation is float32 and rounded once to T.
// Key pages are [page][kv head][slot in page][D]; value pages are transposed,
// [page][kv head][D][slot in page], so that the attention kernels read eight keys
// of one dimension with one load.
// src/halite/transformers/infer/engine/memory_pool.py:139-141 (append after rotation)
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void rope_append_kernel(T* __restrict__ qkv, int row_stride,
                                   const int* __restrict__ positions,
                                   const int* __restrict__ token_seg,
                                   const int* __restrict__ block_table, int bt_stride,
                                   const float* __restrict__ cos_t,
                                   const float* __restrict__ sin_t, int table_len,
                                   T* __restrict__ k_pages, T* __restrict__ v_pages, int H,
                                   int K, int D, int rot, int interleaved, int page_size,
                                   int n_pages, bool tiled) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  T* row = qkv + (size_t)t * row_stride;
  const int half = rot / 2;
  if (rot > 0 && (pos < 0 || pos >= table_len)) return;  // checked on the host; never index outside

  long long page = -1;
  int off = 0;
  if (K > 0) {
    page = block_table[(size_t)token_seg[t] * bt_stride + pos / page_size];
    off = pos % page_size;
    if (page < 0 || page >= n_pages) page = -1;  // checked on the host
  }

  const float* cp = cos_t + (size_t)pos * half;
  const float* sp = sin_t + (size_t)pos * half;
  for (int idx = threadIdx.x; idx < (H + K) * half; idx += blockDim.x) {
    const int head = idx / half, j = idx % half;
    const int i0 = interleaved ? 2 * j : j;
    const int i1 = interleaved ? 2 * j + 1 : j + half;
    T* hp = row + (size_t)head * D;
    const float c = cp[j], s = sp[j];
    const float x0 = to_f32(hp[i0]), x1 = to_f32(hp[i1]);
    const T y0 = from_f32<T>(x0 * c - x1 * s);
    const T y1 = from_f32<T>(x0 * s + x1 * c);
    hp[i0] = y0;
    hp[i1] = y1;
    if (head >= H && page >= 0) {
      const int g = head - H;
      T* kp = k_pages + ((size_t)page * K + g) * page_size * D;
      kp[kv_key_offset(tiled, page_size, D, off, i0)] = y0;
      kp[kv_key_offset(tiled, page_size, D, off, i1)] = y1;
    }
  }
  if (page < 0) return;
  // dimensions of k beyond the rotated ones pass through
  const int rest = D - rot;
  for (int idx = threadIdx.x; idx < K * rest; idx += blockDim.x) {
    const int g = idx / rest, i = rot + idx % rest;
    k_pages[((size_t)page * K + g) * page_size * D + kv_key_offset(tiled, page_size, D, off, i)] =
        row[(size_t)(H + g) * D + i];
  }
  for (int idx = threadIdx.x; idx < K * D; idx += blockDim.x) {
    const int g = idx / D, i = idx % D;
    v_pages[((size_t)page * K + g) * D * page_size + kv_value_offset(tiled, page_size, D, off, i)] =
        row[(size_t)(H + K + g) * D + i];
  }
}

// Eight elements per work item (rot a multiple of 16, or of 8 for adjacent pairs; D a
// multiple of 8): all loads of an item are issued before its arithmetic.
template <typename T>
__global__ void rope_append_vec_kernel(T* __restrict__ qkv, int row_stride,
                                       const int* __restrict__ positions,
                                       const int* __restrict__ token_seg,
                                       const int* __restrict__ block_table, int bt_stride,
                                       const float* __restrict__ cos_t,
                                       const float* __restrict__ sin_t, int table_len,
                                       T* __restrict__ k_pages, T* __restrict__ v_pages, int H,
                                       int K, int D, int rot, int interleaved, int page_size,
                                       int n_pages, bool tiled) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int seg = K > 0 ? token_seg[t] : 0;
  T* row = qkv + (size_t)t * row_stride;
  const int half = rot / 2;
  // A step of few tokens (decode) is a chain of trips to memory, so everything that does not
  // depend on the position is asked for before the position is looked at: this token's
  // values here, and the neighbours that decide further down who writes the values.
  const int d8 = D / 8;
  const bool early_values = K > 0 && gridDim.x <= 64 && K * d8 <= (int)blockDim.x;
  uint4 vpre[sizeof(T) / 2];
  if (early_values && (int)threadIdx.x < K * d8) {
    const uint4* vr = (const uint4*)(row + (size_t)(H + K) * D + (size_t)threadIdx.x * 8);
#pragma unroll
    for (int i = 0; i < (int)(sizeof(T) / 2); ++i) vpre[i] = vr[i];
  }
  if (rot > 0 && (pos < 0 || pos >= table_len)) return;
  long long page = -1;
  int off = 0;
  bool whole = false;
  if (K > 0) {
    page = block_table[(size_t)seg * bt_stride + pos / page_size];
    off = pos % page_size;
    if (page_size % 8 == 0) {
      const int t0 = t - off % 8;  // where the first token of this token's group of eight would be
      if (t0 >= 0 && t0 + 7 < (int)gridDim.x)
        whole = token_seg[t0] == seg && token_seg[t0 + 7] == seg &&
                positions[t0] == pos - off % 8 && positions[t0 + 7] == pos - off % 8 + 7;
    }
    if (page < 0 || page >= n_pages) page = -1;
  }
  const float* cp = cos_t + (size_t)pos * half;
  const float* sp = sin_t + (size_t)pos * half;

  if (!interleaved) {
    const int cph = half / 8;
    for (int idx = threadIdx.x; idx < (H + K) * cph; idx += blockDim.x) {
      const int head = idx / cph, j = (idx % cph) * 8;
      T* hp = row + (size_t)head * D;
      float a[2][4], b[2][4], c[2][4], sn[2][4], y0[2][4], y1[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        load4(hp + j + 4 * u, a[u]);
        load4(hp + j + half + 4 * u, b[u]);
        load4(cp + j + 4 * u, c[u]);
        load4(sp + j + 4 * u, sn[u]);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          y0[u][i] = a[u][i] * c[u][i] - b[u][i] * sn[u][i];
          y1[u][i] = a[u][i] * sn[u][i] + b[u][i] * c[u][i];
        }
      T* kp = (head >= H && page >= 0) ? k_pages + ((size_t)page * K + (head - H)) * page_size * D
                                       : nullptr;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        store4(hp + j + 4 * u, y0[u]);
        store4(hp + j + half + 4 * u, y1[u]);
        if (kp) {
          store4(kp + kv_key_offset(tiled, page_size, D, off, j + 4 * u), y0[u]);
          store4(kp + kv_key_offset(tiled, page_size, D, off, j + half + 4 * u), y1[u]);
        }
      }
    }
  } else {
    const int cph = rot / 8;
    for (int idx = threadIdx.x; idx < (H + K) * cph; idx += blockDim.x) {
      const int head = idx / cph, e0 = (idx % cph) * 8, j = e0 / 2;
      T* hp = row + (size_t)head * D;
      float a[2][4], c[4], sn[4], y[2][4];
      load4(hp + e0, a[0]);
      load4(hp + e0 + 4, a[1]);
      load4(cp + j, c);
      load4(sp + j, sn);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float x0 = a[i / 2][(2 * i) % 4], x1 = a[i / 2][(2 * i) % 4 + 1];
        y[i / 2][(2 * i) % 4] = x0 * c[i] - x1 * sn[i];
        y[i / 2][(2 * i) % 4 + 1] = x0 * sn[i] + x1 * c[i];
      }
      store4(hp + e0, y[0]);
      store4(hp + e0 + 4, y[1]);
      if (head >= H && page >= 0) {
        T* kp = k_pages + ((size_t)page * K + (head - H)) * page_size * D;
        store4(kp + kv_key_offset(tiled, page_size, D, off, e0), y[0]);
        store4(kp + kv_key_offset(tiled, page_size, D, off, e0 + 4), y[1]);
      }
    }
  }
  if (page < 0) return;
  const int rest8 = (D - rot) / 8;
  for (int idx = threadIdx.x; idx < K * rest8; idx += blockDim.x) {
    const int g = idx / rest8, i = rot + (idx % rest8) * 8;
    float a[2][4];
    load4(row + (size_t)(H + g) * D + i, a[0]);
    load4(row + (size_t)(H + g) * D + i + 4, a[1]);
    T* kp = k_pages + ((size_t)page * K + g) * page_size * D;
    store4(kp + kv_key_offset(tiled, page_size, D, off, i), a[0]);
    store4(kp + kv_key_offset(tiled, page_size, D, off, i + 4), a[1]);
  }
  // Values: eight consecutive slots of one dimension lie side by side in a page (both
  // layouts).  Where this token and the seven after it are one request's positions
  // 8j .. 8j+7, the block of the first writes the values of all eight, eight at a time;
  // the other seven leave theirs to it.
  if (whole) {
    if (off % 8 != 0) return;
    for (int idx = threadIdx.x; idx < K * D; idx += blockDim.x) {
      const int g = idx / D, d = idx % D;
      __attribute__((aligned(16))) T vals[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        vals[e] = qkv[(size_t)(t + e) * row_stride + (size_t)(H + K + g) * D + d];
      T* vp = v_pages + ((size_t)page * K + g) * D * page_size +
              kv_value_offset(tiled, page_size, D, off, d);
      // eight elements in one or two 16-byte stores (the offset is a multiple of 8)
      if constexpr (sizeof(T) == 2) {
        *(uint4*)vp = *(const uint4*)vals;
      } else {
        *(uint4*)vp = *(const uint4*)vals;
        *(uint4*)(vp + 4) = *(const uint4*)(vals + 4);
      }
    }
    return;
  }
  for (int idx = threadIdx.x; idx < K * d8; idx += blockDim.x) {
    const int g = idx / d8, i = (idx % d8) * 8;
    __attribute__((aligned(16))) T vals[8];
    if (early_values) {
#pragma unroll
      for (int u = 0; u < (int)(sizeof(T) / 2); ++u) ((uint4*)vals)[u] = vpre[u];
    } else {
      const uint4* vr = (const uint4*)(row + (size_t)(H + K + g) * D + i);
#pragma unroll
      for (int u = 0; u < (int)(sizeof(T) / 2); ++u) ((uint4*)vals)[u] = vr[u];
    }
    T* vp = v_pages + ((size_t)page * K + g) * D * page_size;
#pragma unroll
    for (int e = 0; e < 8; ++e) vp[kv_value_offset(tiled, page_size, D, off, i + e)] = vals[e];
  }
}

// The same for steps of many tokens (prompt portions): a workgroup takes eight consecutive
// tokens.  Their positions and pages are looked up once, by eight threads (one chain of
// trips to memory per eight tokens instead of one per token); the rotations of all eight
// are one pool of work items; and where the eight are one request's positions 8j .. 8j+7
// their values go through LDS, in with 16-byte loads and out eight slots of a dimension
// at a time (a page keeps eight consecutive slots of a dimension side by side in both
// layouts).  A token whose position lies outside the table is left alone and one whose
// page is not valid is rotated and not appended, as in the kernels above.
#define RG_TOKENS 8
#define RG_THREADS 1024
template <typename T>
__global__ void __launch_bounds__(RG_THREADS)
rope_append_group_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                         const int* __restrict__ token_seg, const int* __restrict__ block_table,
                         int bt_stride, const float* __restrict__ cos_t,
                         const float* __restrict__ sin_t, int table_len, T* __restrict__ k_pages,
                         T* __restrict__ v_pages, int n_tokens, int H, int K, int D, int rot,
                         int interleaved, int page_size, int n_pages, bool tiled) {
  __shared__ int s_pos[RG_TOKENS], s_off[RG_TOKENS];
  __shared__ int s_lead[RG_TOKENS];  // 0: the token writes its own values; 1: its run's first does; 2: it is that first
  __shared__ long long s_page[RG_TOKENS];
  extern __shared__ __align__(16) unsigned char rg_values[];  // [8 tokens][K * D] of T
  const int t0 = blockIdx.x * RG_TOKENS;
  const int n = n_tokens - t0 < RG_TOKENS ? n_tokens - t0 : RG_TOKENS;
  const int half = rot / 2;
  if (threadIdx.x < RG_TOKENS) {
    const int i = threadIdx.x;
    int pos = -1, off = 0, lead = 0;
    long long page = -1;
    if (i < n) {
      const int t = t0 + i;
      pos = positions[t];
      const int seg = token_seg[t];
      const bool ok = pos >= 0 && (rot == 0 || pos < table_len);
      if (ok) {
        page = block_table[(size_t)seg * bt_stride + pos / page_size];
        off = pos % page_size;
        if (page < 0 || page >= n_pages) page = -1;
        const int first = t - off % 8;  // where the first token of this token's run of eight would be
        if (page >= 0 && first >= 0 && first + 7 < n_tokens &&
            token_seg[first] == seg && token_seg[first + 7] == seg &&
            positions[first] == pos - off % 8 && positions[first + 7] == pos - off % 8 + 7)
          lead = off % 8 == 0 ? 2 : 1;
      } else {
        pos = -1;
      }
    }
    s_pos[i] = pos, s_off[i] = off, s_lead[i] = lead, s_page[i] = page;
  }
  __syncthreads();

  // ---- q and k: rotate in place, k also into its page --------------------------------
  const int cph = interleaved ? rot / 8 : half / 8;  // work items of a head
  const int per_token = (H + K) * cph;
  for (int item = threadIdx.x; item < n * per_token; item += blockDim.x) {
    const int i = item / per_token, idx = item % per_token;
    const int pos = s_pos[i];
    if (pos < 0) continue;
    const long long page = s_page[i];
    const int off = s_off[i];
    T* row = qkv + (size_t)(t0 + i) * row_stride;
    const float* cp = cos_t + (size_t)pos * half;
    const float* sp = sin_t + (size_t)pos * half;
    const int head = idx / cph;
    T* hp = row + (size_t)head * D;
    T* kp = (head >= H && page >= 0) ? k_pages + ((size_t)page * K + (head - H)) * page_size * D
                                     : nullptr;
    if (!interleaved) {
      const int j = (idx % cph) * 8;
      float a[2][4], b[2][4], c[2][4], sn[2][4], y0[2][4], y1[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        load4(hp + j + 4 * u, a[u]);
        load4(hp + j + half + 4 * u, b[u]);
        load4(cp + j + 4 * u, c[u]);
        load4(sp + j + 4 * u, sn[u]);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          y0[u][e] = a[u][e] * c[u][e] - b[u][e] * sn[u][e];
          y1[u][e] = a[u][e] * sn[u][e] + b[u][e] * c[u][e];
        }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        store4(hp + j + 4 * u, y0[u]);
        store4(hp + j + half + 4 * u, y1[u]);
        if (kp) {
          store4(kp + kv_key_offset(tiled, page_size, D, off, j + 4 * u), y0[u]);
          store4(kp + kv_key_offset(tiled, page_size, D, off, j + half + 4 * u), y1[u]);
        }
      }
    } else {
      const int e0 = (idx % cph) * 8, j = e0 / 2;
      float a[2][4], c[4], sn[4], y[2][4];
      load4(hp + e0, a[0]);
      load4(hp + e0 + 4, a[1]);
      load4(cp + j, c);
      load4(sp + j, sn);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x0 = a[e / 2][(2 * e) % 4], x1 = a[e / 2][(2 * e) % 4 + 1];
        y[e / 2][(2 * e) % 4] = x0 * c[e] - x1 * sn[e];
        y[e / 2][(2 * e) % 4 + 1] = x0 * sn[e] + x1 * c[e];
      }
      store4(hp + e0, y[0]);
      store4(hp + e0 + 4, y[1]);
      if (kp) {
        store4(kp + kv_key_offset(tiled, page_size, D, off, e0), y[0]);
        store4(kp + kv_key_offset(tiled, page_size, D, off, e0 + 4), y[1]);
      }
    }
  }
  // dimensions of k beyond the rotated ones pass through
  const int rest8 = (D - rot) / 8;
  for (int item = threadIdx.x; item < n * K * rest8; item += blockDim.x) {
    const int i = item / (K * rest8), idx = item % (K * rest8);
    if (s_pos[i] < 0 || s_page[i] < 0) continue;
    const int g = idx / rest8, d = rot + (idx % rest8) * 8;
    const T* row = qkv + (size_t)(t0 + i) * row_stride;
    float a[2][4];
    load4(row + (size_t)(H + g) * D + d, a[0]);
    load4(row + (size_t)(H + g) * D + d + 4, a[1]);
    T* kp = k_pages + ((size_t)s_page[i] * K + g) * page_size * D;
    store4(kp + kv_key_offset(tiled, page_size, D, s_off[i], d), a[0]);
    store4(kp + kv_key_offset(tiled, page_size, D, s_off[i], d + 4), a[1]);
  }

  // ---- values ---------------------------------------------------------------------
  // A token whose run of eight positions (from a multiple of eight on) is all in this step
  // leaves its values to the run's first token; that token's workgroup brings the eight rows
  // into LDS and writes eight slots of every dimension at a time.  (The run's other tokens
  // may be the next workgroup's: their values are only read.)
  const int KD = K * D;
  for (int i = 0; i < n; ++i) {
    if (s_lead[i] != 2) continue;  // the same for the whole workgroup
    T* staged = (T*)rg_values;
    constexpr int PER = 16 / sizeof(T);  // elements of a 16-byte piece
    __syncthreads();  // (the run before this one has been written)
    for (int c = threadIdx.x; c < RG_TOKENS * KD / PER; c += blockDim.x) {
      const int r = c / (KD / PER), e = (c % (KD / PER)) * PER;
      *(uint4*)(staged + (size_t)r * KD + e) =
          *(const uint4*)(qkv + (size_t)(t0 + i + r) * row_stride + (size_t)(H + K) * D + e);
    }
    __syncthreads();
    const long long page = s_page[i];
    const int off = s_off[i];
    for (int idx = threadIdx.x; idx < KD; idx += blockDim.x) {
      const int g = idx / D, d = idx % D;
      __attribute__((aligned(16))) T vals[RG_TOKENS];
#pragma unroll
      for (int r = 0; r < RG_TOKENS; ++r) vals[r] = staged[(size_t)r * KD + idx];
      T* vp = v_pages + ((size_t)page * K + g) * D * page_size +
              kv_value_offset(tiled, page_size, D, off, d);
      if constexpr (sizeof(T) == 2) {
        *(uint4*)vp = *(const uint4*)vals;
      } else {
        *(uint4*)vp = *(const uint4*)vals;
        *(uint4*)(vp + 4) = *(const uint4*)(vals + 4);
      }
    }
  }
  const int d8 = D / 8;
  for (int item = threadIdx.x; item < n * K * d8; item += blockDim.x) {
    const int i = item / (K * d8), idx = item % (K * d8);
    if (s_pos[i] < 0 || s_page[i] < 0 || s_lead[i] != 0) continue;
    const int g = idx / d8, d = (idx % d8) * 8;
    __attribute__((aligned(16))) T vals[8];
    const uint4* vr = (const uint4*)(qkv + (size_t)(t0 + i) * row_stride + (size_t)(H + K + g) * D + d);
#pragma unroll
    for (int u = 0; u < (int)(sizeof(T) / 2); ++u) ((uint4*)vals)[u] = vr[u];
    T* vp = v_pages + ((size_t)s_page[i] * K + g) * D * page_size;
#pragma unroll
    for (int e = 0; e < 8; ++e) vp[kv_value_offset(tiled, page_size, D, s_off[i], d + e)] = vals[e];
  }
}

extern "C" int hal_rope_append(void* qkv, int dtype, int row_stride, const int* positions,
                               const int* token_seg, const int* block_table, int bt_stride,
                               const float* cos_t, const float* sin_t, int table_len,
                               void* k_pages, void* v_pages, int n_tokens, int H, int K, int D,
                               int rot, int interleaved, int page_size, int n_pages, int tiled,
                               hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H >= 0 && K >= 0 && D > 0, "hal_rope_append: bad sizes");
  HAL_REQUIRE(rot >= 0 && rot <= D && rot % 2 == 0, "hal_rope_append: rotary dim %d of %d", rot, D);
  HAL_REQUIRE(row_stride >= (H + 2 * K) * D, "hal_rope_append: row stride %d < %d", row_stride,
              (H + 2 * K) * D);
  HAL_REQUIRE(K == 0 || (k_pages && v_pages && block_table && token_seg && page_size > 0),
              "hal_rope_append: cache arguments missing");
  if (n_tokens == 0) return 0;
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_rope_append: unknown dtype %d", dtype);
  HAL_REQUIRE(!tiled || (page_size % 32 == 0 && D % 32 == 0),
              "hal_rope_append: the tiled page layout needs pages and heads of a multiple of 32 "
              "(page %d, head %d)", page_size, D);
  const bool vec = D % 8 == 0 && row_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0 &&
                   (interleaved ? rot % 8 == 0 : rot % 16 == 0);
  // many tokens: eight to a workgroup (the values of eight tokens must fit LDS)
  const size_t group_lds = (size_t)RG_TOKENS * K * D * (dtype == HAL_F32 ? 4 : 2);
  // (measured with 32 + 8 + 8 heads of 128: the same at 1,024 tokens, 14 against 18 us at
  // 2,048, 42 against 62 us at 8,192; below that the kernels above, which have more
  // workgroups in flight, are faster)
  if (vec && K > 0 && n_tokens >= 1536 && page_size % 8 == 0 && rot > 0 && group_lds <= 48 * 1024) {
    const dim3 grid((n_tokens + RG_TOKENS - 1) / RG_TOKENS);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(rope_append_group_kernel<float>, grid, dim3(RG_THREADS), group_lds, stream,
                         (float*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                         cos_t, sin_t, table_len, (float*)k_pages, (float*)v_pages, n_tokens, H, K,
                         D, rot, interleaved, page_size, n_pages, tiled != 0);
    else
      hipLaunchKernelGGL(rope_append_group_kernel<bf16_t>, grid, dim3(RG_THREADS), group_lds, stream,
                         (bf16_t*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                         cos_t, sin_t, table_len, (bf16_t*)k_pages, (bf16_t*)v_pages, n_tokens, H,
                         K, D, rot, interleaved, page_size, n_pages, tiled != 0);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  if (vec) {
    int items = (H + K) * (rot / 8) / (interleaved ? 1 : 2);
    if (K * (D / 8) > items) items = K * (D / 8);
    int threads = ((items + 63) / 64) * 64;
    threads = threads < 64 ? 64 : (threads > 512 ? 512 : threads);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(rope_append_vec_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream,
                         (float*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                         cos_t, sin_t, table_len, (float*)k_pages, (float*)v_pages, H, K, D, rot,
                         interleaved, page_size, n_pages, tiled != 0);
    else
      hipLaunchKernelGGL(rope_append_vec_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream,
                         (bf16_t*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                         cos_t, sin_t, table_len, (bf16_t*)k_pages, (bf16_t*)v_pages, H, K, D,
                         rot, interleaved, page_size, n_pages, tiled != 0);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const int work = (H + K) * (rot / 2) > K * D ? (H + K) * (rot / 2) : K * D;
  const int threads = work >= 1024 ? 256 : (work >= 256 ? 128 : 64);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(rope_append_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream,
                       (float*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                       cos_t, sin_t, table_len, (float*)k_pages, (float*)v_pages, H, K, D, rot,
                       interleaved, page_size, n_pages, tiled != 0);
  else if (dtype == HAL_BF16)
    hipLaunchKernelGGL(rope_append_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream,
                       (bf16_t*)qkv, row_stride, positions, token_seg, block_table, bt_stride,
                       cos_t, sin_t, table_len, (bf16_t*)k_pages, (bf16_t*)v_pages, H, K, D, rot,
                       interleaved, page_size, n_pages, tiled != 0);
  else
    return hal_fail("hal_rope_append: unknown dtype %d", dtype);
  HAL_LAUNCH_CHECK();
  return 0;
}
