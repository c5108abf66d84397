// C[M, N] = X[M, K] * W[N, K]^T for few rows of X (decode batches): bf16 operands,
// float32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16), bound by the
// one pass over W.  W is a linear layer's weight as stored ([out, in]); it is read
// straight from memory into the MFMA operand layout, 64 contiguous bytes of a row
// per load instruction, and never staged.
//
// A wavefront owns 16*NT rows of W and 16*MT rows of X and a share of K; the waves
// of a workgroup split K among them and their partial sums are added in wave order
// through LDS, so the result is deterministic.  The epilogue writes bf16 or float32,
// can add into a float32 destination (the residual stream), and in the gated form
// computes up * silu(gate) from two weights at once
// (src/halite/transformers/feedforward.py:204-212).
#include "hal_common.h"
#include "hal_api.h"
#include <stdlib.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* p, bool valid) {
  u32x4 raw = {0u, 0u, 0u, 0u};
  if (valid) raw = *(const u32x4*)p;
  return __builtin_bit_cast(bf16x8, raw);
}

enum { SK_OUT_BF16 = 0, SK_OUT_F32 = 1, SK_OUT_F32_ADD = 2 };

// Two things around the product that save a launch each when a layer is a chain of
// small-batch products (src/halite/transformers/block.py:56-74 is the chain):
// * the rows of X are RMSNorm(xh) computed while they are loaded: xh is the float32
//   stream, the sums of squares of its rows come in as `ss_parts` partial sums, and the
//   formula is the norm kernel's (src/halite/nn/normalization.py:48-55);
// * after adding into the float32 stream (SK_OUT_F32_ADD) a block writes the sums of
//   squares of its part of the new rows, which are such partial sums for the next norm.
struct SkinnyFuse {
  const float* xh;  // [M, ldxh] or null
  int ldxh;
  const float* ss_in;  // [ss_parts][ss_ld]
  int ss_parts, ss_ld;
  const void* norm_w;  // [K]
  int norm_w_dtype;
  float eps;
  float* ss_out;  // [blocks][ss_out_ld] or null
  int ss_out_ld;
};

// eight elements of a normalised row (two groups of four): the norm's value rounded to
// bf16, times the weight
__device__ __forceinline__ bf16x8 norm_frag(const float (&hv)[2][4], const float (&wv)[2][4],
                                            float rstd) {
  u32x4 raw;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int g = i / 2, e = (i % 2) * 2;
    const float a = wv[g][e] * bf16_to_f32(f32_to_bf16(hv[g][e] * rstd));
    const float b = wv[g][e + 1] * bf16_to_f32(f32_to_bf16(hv[g][e + 1] * rstd));
    raw[i] = pack_bf16x2(a, b);
  }
  return __builtin_bit_cast(bf16x8, raw);
}

template <int NT, int MT, bool GATED, int U, bool NORMX>
__global__ void skinny_gemm_kernel(const bf16_t* __restrict__ X, int ldx,
                                   const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
                                   int ldw, void* __restrict__ C, int ldc, int out_mode, int M,
                                   int N, int K, int slots, SkinnyFuse fuse) {
  extern __shared__ float red[];  // [waves][sets][NT*MT][64][4]
  const int tid = threadIdx.x, lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const int n_waves = blockDim.x / HAL_WAVE;
  const int r = lane % 16, q = lane / 16;
  const int n_base = blockIdx.x * 16 * NT;
  constexpr int SETS = GATED ? 2 : 1;

  const int steps = (K + 31) / 32;
  const int per_wave = (steps + n_waves - 1) / n_waves;
  const int s_begin = wave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;

  f32x4 acc[SETS][NT][MT];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int f = 0; f < NT; ++f)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[s][f][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[NT];
  const bf16_t* w2row[NT];
#pragma unroll
  for (int f = 0; f < NT; ++f) {
    if (ldw == 0) {
      // tiled weights: [16-row tile][32-column step][lane][8], zero-padded, so that a
      // wave's load instruction reads one contiguous KiB
      int tile = blockIdx.x * NT + f;
      const int n_tiles = (N + 15) / 16;
      if (tile >= n_tiles) tile = n_tiles - 1;
      wrow[f] = W + ((size_t)tile * steps * 64 + lane) * 8;
      w2row[f] = GATED ? W2 + ((size_t)tile * steps * 64 + lane) * 8 : nullptr;
    } else {
      int n = n_base + f * 16 + r;
      if (n >= N) n = N - 1;  // rows past the end are computed and dropped
      wrow[f] = W + (size_t)n * ldw + q * 8;
      w2row[f] = GATED ? W2 + (size_t)n * ldw + q * 8 : nullptr;
    }
  }
  const int kstride = ldw == 0 ? 512 : 32;  // elements from one step to the next
  const bf16_t* xrow[MT];
  const float* hrow[MT];
  float rstd[MT];
  bool xvalid[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    xvalid[t] = m < M;
    xrow[t] = X + (size_t)(xvalid[t] ? m : 0) * ldx + q * 8;
    hrow[t] = nullptr;
    rstd[t] = 0.f;
    if constexpr (NORMX) {
      hrow[t] = fuse.xh + (size_t)(xvalid[t] ? m : 0) * fuse.ldxh + q * 8;
      // the row's sum of squares: the four lanes of a row take every fourth partial sum
      float ss = 0.f;
      if (xvalid[t])
        for (int p = q; p < fuse.ss_parts; p += 4) ss += fuse.ss_in[(size_t)p * fuse.ss_ld + m];
      ss += __shfl_xor(ss, 16, HAL_WAVE);
      ss += __shfl_xor(ss, 32, HAL_WAVE);
      rstd[t] = 1.0f / sqrtf(ss / (float)K + fuse.eps);
    }
  }

  // U steps of 32 columns at a time: every load of the group is issued before the
  // first multiply, so a wave keeps U * (NT + MT) 16-byte loads in flight
  for (int step = s_begin; step < s_end; step += U) {
    bf16x8 a[U][NT], a2[U][NT], b[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (step + u) * 32;
      const bool kv = (step + u) < s_end && k + q * 8 < K;  // K is a multiple of 8
      const size_t kw = (size_t)(step + u) * kstride;
#pragma unroll
      for (int f = 0; f < NT; ++f) {
        a[u][f] = load_frag(wrow[f] + kw, kv);
        if (GATED) a2[u][f] = load_frag(w2row[f] + kw, kv);
      }
      if constexpr (!NORMX) {
#pragma unroll
        for (int t = 0; t < MT; ++t) b[u][t] = load_frag(xrow[t] + k, kv && xvalid[t]);
      }
    }
    if constexpr (NORMX) {
      // the stream's rows and the norm's weight: loaded for the whole group, then turned
      // into operands (the loads of W above are on their way meanwhile)
      float hv[U][MT][2][4], wv[U][2][4];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = (step + u) * 32 + q * 8;
        const bool kv = (step + u) < s_end && k < K;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
          for (int i = 0; i < 4; ++i) wv[u][g][i] = 0.f;
          if (kv) load4_any(fuse.norm_w, fuse.norm_w_dtype, (size_t)k + 4 * g, wv[u][g]);
#pragma unroll
          for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int i = 0; i < 4; ++i) hv[u][t][g][i] = 0.f;
            if (kv && xvalid[t]) load4(hrow[t] + (size_t)(step + u) * 32 + 4 * g, hv[u][t][g]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < MT; ++t) b[u][t] = norm_frag(hv[u][t], wv[u], rstd[t]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int f = 0; f < NT; ++f)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[0][f][t] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][f], b[u][t], acc[0][f][t], 0, 0, 0);
          if (GATED)
            acc[1][f][t] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[u][f], b[u][t], acc[1][f][t], 0, 0, 0);
        }
  }

  // every wave's partial sums -> LDS; then each output element is the sum over the
  // waves in wave order (deterministic).  `slots` < n_waves means that LDS holds only
  // that many partial tiles: in rounds, the next `slots` waves hand their sums to the
  // first `slots` waves (wave w + r*slots to wave w, same lanes) before those write.
  constexpr int TILE = SETS * NT * MT * 256;
  for (int base = slots; base < n_waves; base += slots) {
    if (wave >= base && wave < base + slots) {
      float* theirs = red + (size_t)(wave - base) * TILE;
#pragma unroll
      for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int f = 0; f < NT; ++f)
#pragma unroll
          for (int t = 0; t < MT; ++t)
            *(f32x4*)(theirs + ((s * NT + f) * MT + t) * 256 + lane * 4) = acc[s][f][t];
    }
    __syncthreads();
    if (wave < slots && wave + base < n_waves) {
      const float* from = red + (size_t)wave * TILE;
#pragma unroll
      for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int f = 0; f < NT; ++f)
#pragma unroll
          for (int t = 0; t < MT; ++t)
            acc[s][f][t] += *(const f32x4*)(from + ((s * NT + f) * MT + t) * 256 + lane * 4);
    }
    __syncthreads();
  }
  if (wave < slots) {
    float* mine = red + (size_t)wave * TILE;
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int f = 0; f < NT; ++f)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          *(f32x4*)(mine + ((s * NT + f) * MT + t) * 256 + lane * 4) = acc[s][f][t];
  }
  __syncthreads();

  // element (f, t, lane, i) of the accumulator tile is row n_base + f*16 + (lane/16)*4 + i
  // of W (column of C) and row t*16 + lane%16 of X (row of C)
  float my_ss = 0.f;
  for (int idx = tid; idx < NT * MT * 256; idx += blockDim.x) {
    const int i = idx % 4, ln = (idx / 4) % 64, ft = idx / 256;
    const int f = ft / MT, t = ft % MT;
    const int n = n_base + f * 16 + (ln / 16) * 4 + i;
    const int m = t * 16 + ln % 16;
    if (n >= N || m >= M) continue;
    float v = 0.f, v2 = 0.f;
    for (int w = 0; w < slots; ++w) {
      v += red[(size_t)w * TILE + idx];
      if (GATED) v2 += red[(size_t)w * TILE + NT * MT * 256 + idx];
    }
    if (GATED) v = v2 * (v / (1.0f + expf(-v)));  // set 0 is the gate, set 1 is up
    const size_t o = (size_t)m * ldc + n;
    if (out_mode == SK_OUT_BF16) {
      ((bf16_t*)C)[o] = f32_to_bf16(v);
    } else if (out_mode == SK_OUT_F32) {
      ((float*)C)[o] = v;
    } else {
      const float sum = ((float*)C)[o] + v;
      ((float*)C)[o] = sum;
      my_ss += sum * sum;
    }
  }
  if (fuse.ss_out) {
    // (MT == 1) a thread's elements all belong to row (tid / 4) % 16; the row's sum over
    // this block's columns is added up by one thread in the order of the threads
    __syncthreads();
    red[tid] = my_ss;
    __syncthreads();
    if (tid < 16 && tid < M) {
      float total = 0.f;
      for (int j = tid * 4; j < (int)blockDim.x; j += 64)
        total += (red[j] + red[j + 1]) + (red[j + 2] + red[j + 3]);
      fuse.ss_out[(size_t)blockIdx.x * fuse.ss_out_ld + tid] = total;
    }
  }
}

template <int NT, int MT, bool GATED, int U>
static int launch_skinny(const bf16_t* X, int ldx, const bf16_t* W, const bf16_t* W2, int ldw,
                         void* C, int ldc, int out_mode, int M, int N, int K, int waves,
                         const SkinnyFuse& fuse, hipStream_t stream) {
  constexpr int SETS = GATED ? 2 : 1;
  // LDS for the partial sums of all waves, or of a half, a quarter ... if that is too much
  const size_t per_wave = (size_t)SETS * NT * MT * 256 * sizeof(float);
  int slots = waves;
  while (slots > 1 && (size_t)slots * per_wave > 64 * 1024) slots /= 2;
  size_t smem = (size_t)slots * per_wave;
  if (fuse.ss_out && smem < (size_t)waves * HAL_WAVE * sizeof(float))
    smem = (size_t)waves * HAL_WAVE * sizeof(float);  // one float per thread for the rows' sums
  const int blocks = (N + 16 * NT - 1) / (16 * NT);
  if (fuse.xh) {
    if constexpr (MT == 1 && U <= 4) {
      hipLaunchKernelGGL((skinny_gemm_kernel<NT, MT, GATED, U, true>), dim3(blocks),
                         dim3(waves * HAL_WAVE), smem, stream, X, ldx, W, W2, ldw, C, ldc,
                         out_mode, M, N, K, slots, fuse);
    } else {
      return hal_fail("hal_gemm_bf16_skinny: a normalised X needs at most 16 rows");
    }
  } else {
    hipLaunchKernelGGL((skinny_gemm_kernel<NT, MT, GATED, U, false>), dim3(blocks),
                       dim3(waves * HAL_WAVE), smem, stream, X, ldx, W, W2, ldw, C, ldc, out_mode,
                       M, N, K, slots, fuse);
  }
  HAL_LAUNCH_CHECK();
  return 0;
}

// Blocks of the product (and so partial sums of squares per row that it writes).
extern "C" int hal_gemm_bf16_skinny_blocks(int M, int N, int gated) {
  (void)gated;
  const int mt = (M + 15) / 16;
  int nt = mt >= 3 ? 2 : mt;
  if (nt < 1) nt = 1;
  return (N + 16 * nt - 1) / (16 * nt);
}

static int skinny_dispatch(const void* X, int ldx, const void* W, const void* W2, int ldw, void* C,
                           int ldc, int out_mode, int M, int N, int K, const SkinnyFuse& fuse,
                           hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && M <= 64, "hal_gemm_bf16_skinny: M=%d (at most 64 rows)", M);
  HAL_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "hal_gemm_bf16_skinny: N=%d K=%d (K in steps of 8)", N,
              K);
  HAL_REQUIRE((fuse.xh || ldx >= K) && (ldw >= K || ldw == 0) && ldc >= N && ldx % 8 == 0 &&
                  ldw % 8 == 0,
              "hal_gemm_bf16_skinny: leading dimensions %d %d %d", ldx, ldw, ldc);
  HAL_REQUIRE(out_mode >= 0 && out_mode <= 2, "hal_gemm_bf16_skinny: out_mode %d", out_mode);
  HAL_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)W2 % 16) == 0,
              "hal_gemm_bf16_skinny: operands must be 16-byte aligned");
  if (fuse.xh) {
    HAL_REQUIRE(M <= 16 && fuse.ldxh >= K && fuse.ldxh % 4 == 0 && ((uintptr_t)fuse.xh % 16) == 0 &&
                    fuse.ss_in && fuse.ss_parts > 0 && fuse.ss_ld >= M && fuse.norm_w &&
                    (fuse.norm_w_dtype == HAL_F32 || fuse.norm_w_dtype == HAL_BF16) &&
                    ((uintptr_t)fuse.norm_w % 16) == 0,
                "hal_gemm_bf16_skinny: a normalised X needs at most 16 rows of an aligned float32 "
                "stream, partial sums and a weight (M=%d)", M);
  }
  if (fuse.ss_out)
    HAL_REQUIRE(M <= 16 && out_mode == SK_OUT_F32_ADD && fuse.ss_out_ld >= M && !W2,
                "hal_gemm_bf16_skinny: sums of squares come with at most 16 rows added into float32");
  if (M == 0) return 0;
  const bf16_t* x = (const bf16_t*)X;
  const bf16_t* w = (const bf16_t*)W;
  const bf16_t* w2 = (const bf16_t*)W2;
  const int mt = (M + 15) / 16;
  const int sets = w2 ? 2 : 1;
  // Rows of W per wave (16 * nt): more of them mean that a fragment of X, which every
  // block reads again, serves more of W.  The waves of a block split K, more of them
  // when there are few blocks.  Tunable through the environment for measurements.
  int nt = mt >= 3 ? 2 : mt;
  int u = 0, waves = 0;
  if (!fuse.ss_out) {  // the count of blocks is promised to the caller otherwise
    if (const char* e = getenv("HAL_SKINNY_NT")) nt = atoi(e);
  }
  if (const char* e = getenv("HAL_SKINNY_U")) u = atoi(e);
  if (const char* e = getenv("HAL_SKINNY_WAVES")) waves = atoi(e);
  if (nt != 1 && nt != 2 && nt != 4) nt = 2;
  if (mt >= 2 && nt < 2) nt = 2;
  const int blocks = (N + 16 * nt - 1) / (16 * nt);
  const int steps = (K + 31) / 32;
  if (waves <= 0) {
    waves = 4;
    while (waves < 16 && blocks * waves < 4096 && steps / (waves * 2) >= 4) waves *= 2;
  }
  while (waves > 1 && (size_t)sets * nt * mt * 1024 > 64 * 1024) waves /= 2;  // one tile must fit
  // loads in flight per wave: about 16 fragments of 16 bytes
  if (u <= 0) u = 8 / (sets * nt);
  if (fuse.xh && u > 4) u = 4;  // the stream's rows take registers too
  u = u >= 8 ? 8 : (u >= 4 ? 4 : (u >= 2 ? 2 : 1));

#define SK_LAUNCH(NT_, MT_, U_)                                                               \
  do {                                                                                        \
    if (w2)                                                                                   \
      return launch_skinny<NT_, MT_, true, U_>(x, ldx, w, w2, ldw, C, ldc, out_mode, M, N, K, \
                                               waves, fuse, stream);                          \
    return launch_skinny<NT_, MT_, false, U_>(x, ldx, w, nullptr, ldw, C, ldc, out_mode, M,   \
                                              N, K, waves, fuse, stream);                     \
  } while (0)
#define SK_CASE(NT_, MT_)                                      \
  if (nt == NT_ && mt == MT_) {                                \
    if (u == 8) SK_LAUNCH(NT_, MT_, ((NT_ + MT_) <= 2 ? 8 : 4)); \
    if (u == 4) SK_LAUNCH(NT_, MT_, ((NT_ + MT_) <= 5 ? 4 : 2)); \
    if (u == 2) SK_LAUNCH(NT_, MT_, 2);                        \
    SK_LAUNCH(NT_, MT_, 1);                                    \
  }
  SK_CASE(1, 1)
  SK_CASE(2, 1)
  SK_CASE(4, 1)
  SK_CASE(2, 2)
  SK_CASE(4, 2)
  SK_CASE(2, 3)
  SK_CASE(2, 4)
  SK_CASE(4, 3)
  SK_CASE(4, 4)
#undef SK_LAUNCH
#undef SK_CASE
  return hal_fail("hal_gemm_bf16_skinny: no kernel for nt=%d mt=%d", nt, mt);
}

// X [M, K] bf16 (M <= 64), W [N, K] bf16, optional W2 [N, K] (gated form: W is the
// gate's weight, W2 is up's).  out_mode: 0 bf16, 1 float32, 2 add into float32.
extern "C" int hal_gemm_bf16_skinny(const void* X, int ldx, const void* W, const void* W2,
                                    int ldw, void* C, int ldc, int out_mode, int M, int N, int K,
                                    hipStream_t stream) {
  SkinnyFuse none = {};
  return skinny_dispatch(X, ldx, W, W2, ldw, C, ldc, out_mode, M, N, K, none, stream);
}

// The same for at most 16 rows with what surrounds the product in a layer folded in: if
// xh is given, X is RMSNorm(xh) with weight norm_w, computed from the float32 stream xh
// [M, ldxh] and the partial sums of squares of its rows ss_in [ss_parts][ss_ld]; if ss_out
// is given (out_mode 2), block b of hal_gemm_bf16_skinny_blocks(M, N, 0) writes the sums of
// squares of its columns of the new C to ss_out[b][0..M).
extern "C" int hal_gemm_bf16_skinny_fused(const void* W, const void* W2, int ldw, void* C, int ldc,
                                          int out_mode, int M, int N, int K, const void* X, int ldx,
                                          const float* xh, int ldxh, const float* ss_in,
                                          int ss_parts, int ss_ld, const void* norm_w,
                                          int norm_w_dtype, float eps, float* ss_out,
                                          int ss_out_ld, hipStream_t stream) {
  SkinnyFuse fuse = {xh, ldxh, ss_in, ss_parts, ss_ld, norm_w, norm_w_dtype, eps, ss_out, ss_out_ld};
  HAL_REQUIRE(xh || X, "hal_gemm_bf16_skinny_fused: no X");
  return skinny_dispatch(xh ? (const void*)nullptr : X, xh ? 0 : ldx, W, W2, ldw, C, ldc, out_mode,
                         M, N, K, fuse, stream);
}
