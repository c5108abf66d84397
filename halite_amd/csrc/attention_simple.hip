// Paged attention, the plain way: float32 arithmetic on the vector units throughout, any
// head size that is a multiple of 2 up to 512, any page size, any number of heads and
// groups, float32 or bf16 storage.  It is the whole attention of the 32-bit path and the
// fallback of the bf16 path for shapes that the matrix-core kernel refuses.
//
// A workgroup of up to four waves serves one (token, query head).  The row's keys, from the
// start of its window to its own position, go in blocks of 64; wave w takes the blocks w,
// w + waves, ... and keeps a running maximum, denominator and weighted sum of its own, and
// at the end the waves' results are joined in wave order by the log-sum-exp rule.  A row's
// result therefore depends on the row's own position and request alone, not on the batch.
// Within a block a lane is a key for the scores (the block's keys lie in LDS, transposed on
// the way in, so that global loads are contiguous and a lane walks its key's dimensions in
// order) and a dimension for the weighted sum (the block's values in LDS likewise, a lane
// walks the keys in order).
//
// scores, mask, softmax and weighted sum as in
// src/halite/transformers/attention.py:647-714; the causal rule for a portion that
// follows cached tokens (key j visible to the query at position p iff j <= p) is
// the one of src/halite/transformers/infer/engine/flashinfer_backend.py:217-229.
#include "hal_common.h"
#include "hal_api.h"

#define SIMPLE_MAX_ACC 8  // head sizes up to 64 * 8
#define SIMPLE_MAX_WAVES 4

// floats of LDS that one wave needs: a tile of 64 keys x D (rows padded by one) that holds
// the keys and then the values of a block, and the block's 64 probabilities
static inline size_t simple_wave_floats(int D) { return (size_t)HAL_WAVE * (D + 1) + D + HAL_WAVE; }

// LDS that one lane of a wave writes and another reads: the wave's LDS operations are done
// in the order they were issued; this keeps the compiler from moving them across
__device__ __forceinline__ void simple_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// R: 64-wide pieces of a head (head sizes up to 64 * R)
template <typename T, int R>
__global__ void __launch_bounds__(SIMPLE_MAX_WAVES * HAL_WAVE)
attention_simple_kernel(const T* __restrict__ q, int q_row_stride, T* __restrict__ out,
                        int out_row_stride, const int* __restrict__ positions,
                        const int* __restrict__ token_seg, const int* __restrict__ block_table,
                        int bt_stride, const T* __restrict__ k_pages,
                        const T* __restrict__ v_pages, int H, int K, int D, int page_size,
                        int n_pages, float scale, int window) {
  extern __shared__ float smem[];
  const int n_waves = blockDim.x / HAL_WAVE;
  const int lane = threadIdx.x % HAL_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / HAL_WAVE);
  float* q_s = smem;  // [D], shared by the waves
  float* mine = smem + D + (size_t)wave * ((size_t)HAL_WAVE * (D + 1) + D + HAL_WAVE);
  float* tile = mine;                                  // keys [64][D + 1], then values [D][65]
  float* p_s = mine + (size_t)HAL_WAVE * (D + 1) + D;  // [64]  (D * 65 <= 64 * (D + 1) + D)

  const int t = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / K);
  const int p = positions[t];
  const int seg = token_seg[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_table + (size_t)seg * bt_stride;

  const T* qp = q + (size_t)t * q_row_stride + (size_t)h * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) q_s[i] = to_f32(qp[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;

  for (int j0 = lo + wave * HAL_WAVE; j0 <= p; j0 += n_waves * HAL_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= p;
    const int n_valid = (p - j0 + 1) < HAL_WAVE ? (p - j0 + 1) : HAL_WAVE;
    // this lane's key: where it lies (a hole in the block table must show)
    long long base = -1;
    int off = 0;
    if (valid) {
      const long long page = bt[j / page_size];
      off = j % page_size;
      if (page >= 0 && page < n_pages) base = page * K + g;
    }
    // the block's keys into LDS, the lanes along the dimensions; eight keys' loads are
    // issued before the first is stored, so that the trips to memory overlap
    constexpr int KEYS_AT_ONCE = R <= 2 ? 16 : (R <= 4 ? 8 : 4);
    for (int jj0 = 0; jj0 < n_valid; jj0 += KEYS_AT_ONCE) {
      float kv[KEYS_AT_ONCE][R];
#pragma unroll
      for (int u = 0; u < KEYS_AT_ONCE; ++u) {
        const int jj = jj0 + u < n_valid ? jj0 + u : n_valid - 1;
        const int b_lo = __builtin_amdgcn_readlane((int)(base & 0xffffffffll), jj);
        const int b_hi = __builtin_amdgcn_readlane((int)(base >> 32), jj);
        const long long b = ((long long)b_hi << 32) | (unsigned int)b_lo;
        const int o = __builtin_amdgcn_readlane(off, jj);
        const T* kp = k_pages + ((size_t)(b < 0 ? 0 : b) * page_size + o) * D;  // (a hole: any row)
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int i = lane + r * HAL_WAVE;
          kv[u][r] = i < D ? to_f32(kp[i]) : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < KEYS_AT_ONCE; ++u) {
        if (jj0 + u >= n_valid) break;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int i = lane + r * HAL_WAVE;
          if (i < D) tile[(size_t)(jj0 + u) * (D + 1) + i] = kv[u][r];
        }
      }
    }
    simple_wave_sync();  // the rows are written by other lanes than the one that reads them
    float s = -INFINITY;
    if (valid) {
      if (base >= 0) {
        const float* kr = tile + (size_t)lane * (D + 1);
        float dot = 0.f;
        for (int i = 0; i < D; ++i) dot += q_s[i] * kr[i];
        s = dot * scale;
      } else {
        s = __uint_as_float(0x7fc00000u);
      }
    }
    const float m_tile = wave_max(s);
    const float m_new = fmaxf(m, m_tile);
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float pj = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(pj);
    m = m_new;
    simple_wave_sync();  // every lane has read its key's row
    p_s[lane] = pj;
    // the block's values into the same tile, [dimension][key], the lanes along the keys
    // (every lane has read its key's row by now: a wave runs in step)
    {
      const bool have = valid && base >= 0;
      const T* vp = v_pages + (size_t)(have ? base : 0) * D * page_size + off;
      for (int i0 = 0; i0 < D; i0 += 32) {  // 32 dimensions' loads at a time
        float vv[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          const int i = i0 + u < D ? i0 + u : D - 1;
          vv[u] = to_f32(vp[(size_t)i * page_size]);
        }
#pragma unroll
        for (int u = 0; u < 32; ++u)
          if (i0 + u < D) tile[(size_t)(i0 + u) * (HAL_WAVE + 1) + lane] = have ? vv[u] : 0.f;
      }
    }
    simple_wave_sync();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = lane + r * HAL_WAVE;
      if (i < D) {
        const float* vr = tile + (size_t)i * (HAL_WAVE + 1);
        float a = acc[r] * alpha;
        for (int jj = 0; jj < n_valid; ++jj) a += p_s[jj] * vr[jj];
        acc[r] = a;
      }
    }
    simple_wave_sync();  // before the next block's keys overwrite the tile
  }

  // join the waves' results in wave order: every wave leaves (m, l, sums) in its own LDS,
  // the first wave adds them up
  __syncthreads();
  if (lane == 0) {
    p_s[0] = m;
    p_s[1] = l;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = lane + r * HAL_WAVE;
    if (i < D) tile[i] = acc[r];
  }
  __syncthreads();
  if (wave != 0) return;
  const size_t per_wave = (size_t)HAL_WAVE * (D + 1) + D + HAL_WAVE;
  float m_all = -INFINITY;
  for (int w = 0; w < n_waves; ++w) m_all = fmaxf(m_all, smem[D + w * per_wave + (size_t)HAL_WAVE * (D + 1) + D]);
  float l_all = 0.f;
  float tot[R];
#pragma unroll
  for (int r = 0; r < R; ++r) tot[r] = 0.f;
  for (int w = 0; w < n_waves; ++w) {
    const float* theirs = smem + D + w * per_wave;
    const float mw = theirs[(size_t)HAL_WAVE * (D + 1) + D], lw = theirs[(size_t)HAL_WAVE * (D + 1) + D + 1];
    const float wgt = mw == -INFINITY ? 0.f : expf(mw - m_all);
    l_all += wgt * lw;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = lane + r * HAL_WAVE;
      if (i < D) tot[r] += wgt * theirs[i];
    }
  }
  T* op = out + (size_t)t * out_row_stride + (size_t)h * D;
  const float inv = 1.0f / l_all;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = lane + r * HAL_WAVE;
    if (i < D) op[i] = from_f32<T>(tot[r] * inv);
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
  // as many waves as fit the LDS of a CU with their tiles, four at most
  int waves = SIMPLE_MAX_WAVES;
  while (waves > 1 && ((size_t)D + waves * simple_wave_floats(D)) * sizeof(float) > 150 * 1024) waves /= 2;
  const size_t smem = ((size_t)D + waves * simple_wave_floats(D)) * sizeof(float);
  HAL_REQUIRE(smem <= 160 * 1024, "hal_attention_simple: head size %d needs %zu bytes of LDS", D, smem);
  dim3 grid(n_tokens, H);
#define SIMPLE_LAUNCH(T_, R_)                                                                        \
  do {                                                                                              \
    static bool raised = false; /* more than 64 KB of LDS has to be asked for, once per kernel */    \
    if (!raised) {                                                                                  \
      HAL_CHECK_HIP(hipFuncSetAttribute((const void*)attention_simple_kernel<T_, R_>,               \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));   \
      raised = true;                                                                                \
    }                                                                                               \
    hipLaunchKernelGGL((attention_simple_kernel<T_, R_>), grid, dim3(waves * HAL_WAVE), smem, stream, \
                       (const T_*)q, q_row_stride, (T_*)out, out_row_stride, positions, token_seg,  \
                       block_table, bt_stride, (const T_*)k_pages, (const T_*)v_pages, H, K, D,      \
                       page_size, n_pages, scale, window);                                          \
  } while (0)
#define SIMPLE_BY_SIZE(T_)                   \
  do {                                       \
    if (D <= 64) SIMPLE_LAUNCH(T_, 1);       \
    else if (D <= 128) SIMPLE_LAUNCH(T_, 2); \
    else if (D <= 256) SIMPLE_LAUNCH(T_, 4); \
    else SIMPLE_LAUNCH(T_, 8);               \
  } while (0)
  if (dtype == HAL_F32)
    SIMPLE_BY_SIZE(float);
  else if (dtype == HAL_BF16)
    SIMPLE_BY_SIZE(bf16_t);
  else
    return hal_fail("hal_attention_simple: unknown dtype %d", dtype);
#undef SIMPLE_BY_SIZE
#undef SIMPLE_LAUNCH
  HAL_LAUNCH_CHECK();
  return 0;
}
