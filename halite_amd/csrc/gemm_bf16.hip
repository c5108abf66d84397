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
//
// A third epilogue serves the packed q, k, v projection of few tokens: it rotates q and k
// by the tokens' positions and appends the rotated k and v to the cache pages, which
// otherwise is a kernel of its own between this one and attention
// (src/halite/transformers/position.py:287-291, infer/engine/memory_pool.py:139-141).  The
// two elements of a rotation pair lie half a head apart; the weight's rows are reordered
// for this epilogue so that a tile of 16 rows holds eight pairs.
//
// With at most 32 rows the RMSNorm between two products (src/halite/nn/normalization.py:
// 43-57, src/halite/transformers/block.py:56-74) needs no kernel of its own.  The product
// before it (PREP) adds its result into the float32 residual stream h, writes
// bf16(w * bf16(h)) for the norm's weight w, and leaves one sum of h^2 per row and
// workgroup; the product after it (SCALED) adds those sums up in a fixed order and
// multiplies its float32 accumulators by rsqrt(mean(h^2) + eps), which is the same number
// up to the place of one bf16 rounding (the norm's kernel rounds h * rstd, this way rounds h).
// Up to 16 rows always, 17 to 32 rows (two row tiles per wave) where the host finds it the
// faster way.
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

// What the rotating epilogue needs beside the product.  Row r' = head * D + 16 * j + c of
// the reordered weight is row head * D + 8 * j + c of the stored one for c < 8 and row
// head * D + D / 2 + 8 * j + (c - 8) for c >= 8: a tile holds dimensions 8j .. 8j + 7 and
// their partners.  Heads [0, H) are q, [H, H + K) k, [H + K, H + 2K) v.
struct RopeEpilogue {
  const int* positions;    // [M]
  const int* token_seg;    // [M] row of the block table
  const int* block_table;  // [segments, bt_stride] page numbers
  int bt_stride;
  const float* cos_t;  // [table_len, D / 2]
  const float* sin_t;
  int table_len;
  bf16_t* k_pages;
  bf16_t* v_pages;
  int H, K, D, page_size, n_pages, tiled;
};

// The norm folded into the products around it (at most 32 rows; RW below is 16 for up to
// 16 rows of X and 32 beyond, the same in the product before the norm and the one after).
struct NormFusion {
  // SCALED: X holds bf16(w * bf16(h)); sums of h^2, [n_parts][RW], one part per
  // workgroup of the product before; the norm's eps (its size is this product's K)
  const float* ss_in;
  int n_parts;
  float eps;
  // PREP: C is h (float32, added into); the next norm's weight [N], where bf16(w * bf16(h))
  // goes ([M, N] bf16) and where this workgroup's sums of h^2 go ([workgroups][RW])
  const void* norm_w;
  int norm_w_dtype;
  bf16_t* xw_out;
  float* ss_out;
};
enum { SK_ROPE = 1, SK_SCALED = 2, SK_PREP = 4 };
#define SK_MAX_PART_LOADS 4  // float4 loads of partial sums per thread that are asked for ahead

// PL: float4 loads of partial sums per thread (SCALED), held in registers through the loop
template <int NT, int MT, bool GATED, int U, int FLAGS = 0, int PL = 1>
__global__ void skinny_gemm_kernel(const bf16_t* __restrict__ X, int ldx,
                                   const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
                                   int ldw, void* __restrict__ C, int ldc, int out_mode, int M,
                                   int N, int K, int slots, RopeEpilogue rope = RopeEpilogue{},
                                   NormFusion nf = NormFusion{}) {
  constexpr bool ROPE = (FLAGS & SK_ROPE) != 0, SCALED = (FLAGS & SK_SCALED) != 0,
                 PREP = (FLAGS & SK_PREP) != 0;
  static_assert(!(SCALED || PREP || ROPE) || (MT <= 2 && NT <= 2),
                "the extra epilogues serve at most 32 rows");
  static_assert(!PREP || (NT == 1 && !GATED && !ROPE && !SCALED), "PREP takes one plain tile");
  constexpr int RW = 16 * MT;  // rows of X a workgroup holds, and floats per part of the sums
  __shared__ float row_sums[16][RW];  // SCALED: [wave][row]; PREP: [column of the tile][row]
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

  // SCALED: this thread's share of the partial sums is asked for before anything else, so
  // that it has arrived long before the epilogue; with QW = RW / 4, float4 f holds rows
  // 4 (f % QW) .. + 3 of part f / QW, and f % QW == lane % QW for every f of a thread
  // (a load past the end is clamped here and dropped where the sums are added)
  float4 my_parts[PL];
  if constexpr (SCALED) {
    const float4* pp = (const float4*)nf.ss_in;
    const int last = nf.n_parts * (RW / 4) - 1;
#pragma unroll
    for (int k = 0; k < PL; ++k) {
      const int f = tid + k * (int)blockDim.x;
      my_parts[k] = pp[f < last ? f : last];
    }
  }

  // What the norm-preparing epilogue reads from memory beside the sums is asked for here too
  // (a workgroup has at least 256 threads): behind the last product that trip to memory would
  // be the kernel's tail (0.7 us of 16 on the o-proj and down products of a 4,096-wide model).
  // PREP, element e = tid + i * threads: column c of the tile, row m
  constexpr int PREPS = (MT * 256 + 255) / 256;
  float prep_h[PREP ? PREPS : 1], prep_w[PREP ? PREPS : 1];
  if constexpr (PREP) {
#pragma unroll
    for (int i = 0; i < PREPS; ++i) {
      const int e = tid + i * (int)blockDim.x;
      prep_h[i] = 0.f, prep_w[i] = 0.f;
      if (e >= MT * 256) continue;
      const int t = e / 256, c = (e % 256) / 16, m = t * 16 + e % 16, n = n_base + c;
      if (n < N && m < M) {
        prep_h[i] = ((const float*)C)[(size_t)m * ldc + n];
        prep_w[i] = load_as_f32(nf.norm_w, nf.norm_w_dtype, n);
      }
    }
  }

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
  bool xvalid[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    xvalid[t] = m < M;
    xrow[t] = X + (size_t)(xvalid[t] ? m : 0) * ldx + q * 8;
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
#pragma unroll
      for (int t = 0; t < MT; ++t) b[u][t] = load_frag(xrow[t] + k, kv && xvalid[t]);
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
  if constexpr (SCALED) {
    // sums over the parts in a fixed order: this thread's loads, then the lanes that hold
    // the same rows (a butterfly), then the waves (by whoever needs a row, in wave order)
    float4 sum = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < PL; ++k) {
      if (tid + k * (int)blockDim.x < nf.n_parts * (RW / 4))
        sum.x += my_parts[k].x, sum.y += my_parts[k].y, sum.z += my_parts[k].z, sum.w += my_parts[k].w;
    }
    // more parts than the loads ahead cover (a very wide model): the rest is read here
    for (int f = tid + PL * (int)blockDim.x; f < nf.n_parts * (RW / 4); f += blockDim.x) {
      const float4 more = ((const float4*)nf.ss_in)[f];
      sum.x += more.x, sum.y += more.y, sum.z += more.z, sum.w += more.w;
    }
#pragma unroll
    for (int off = RW / 4; off < HAL_WAVE; off <<= 1) {
      sum.x += __shfl_xor(sum.x, off, HAL_WAVE), sum.y += __shfl_xor(sum.y, off, HAL_WAVE);
      sum.z += __shfl_xor(sum.z, off, HAL_WAVE), sum.w += __shfl_xor(sum.w, off, HAL_WAVE);
    }
    if (lane < RW / 4) *(float4*)&row_sums[wave][lane * 4] = sum;
  }
  __syncthreads();
  // rsqrt(mean(h^2) + eps) of row m, as the norm's own kernel computes it
  auto row_scale = [&](int m) {
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += row_sums[w][m];
    return 1.0f / sqrtf(total / (float)K + nf.eps);
  };

  if constexpr (ROPE) {
    static_assert(!GATED, "the rotating epilogue is not the gated one");
    // pair p: elements c and c + 8 of tile f, for token m; C is q alone, [M, H * D]
    const int D = rope.D, half = D / 2, tiles_per_head = D / 16;
    for (int p = tid; p < NT * MT * 128; p += blockDim.x) {
      const int f = p / (MT * 128), t = (p / 128) % MT, c = (p % 128) / 16, m = t * 16 + p % 16;
      const int tile = blockIdx.x * NT + f;
      if (m >= M || tile * 16 >= N) continue;
      const int idx0 = (f * MT + t) * 256 + ((c / 4) * 16 + p % 16) * 4 + c % 4, idx1 = idx0 + 128;
      float v0 = 0.f, v1 = 0.f;
      for (int w = 0; w < slots; ++w) {
        v0 += red[(size_t)w * TILE + idx0];
        v1 += red[(size_t)w * TILE + idx1];
      }
      if constexpr (SCALED) {
        const float rs = row_scale(m);
        v0 *= rs, v1 *= rs;
      }
      // the product is rounded to bf16 before the rotation, as the unfused way stores it
      const float x0 = bf16_to_f32(f32_to_bf16(v0)), x1 = bf16_to_f32(f32_to_bf16(v1));
      const int head = tile / tiles_per_head, d0 = (tile % tiles_per_head) * 8 + c;
      const int d1 = d0 + half;
      const int pos = rope.positions[m];
      if (pos < 0 || pos >= rope.table_len) continue;  // checked on the host
      float y0 = x0, y1 = x1;
      if (head < rope.H + rope.K) {
        const float cs = rope.cos_t[(size_t)pos * half + d0], sn = rope.sin_t[(size_t)pos * half + d0];
        y0 = x0 * cs - x1 * sn;
        y1 = x0 * sn + x1 * cs;
      }
      if (head < rope.H) {
        bf16_t* q = (bf16_t*)C + (size_t)m * ldc + (size_t)head * D;
        q[d0] = f32_to_bf16(y0);
        q[d1] = f32_to_bf16(y1);
        continue;
      }
      const long long page =
          rope.block_table[(size_t)rope.token_seg[m] * rope.bt_stride + pos / rope.page_size];
      if (page < 0 || page >= rope.n_pages) continue;  // checked on the host
      const int off = pos % rope.page_size;
      if (head < rope.H + rope.K) {
        bf16_t* kp = rope.k_pages + ((size_t)page * rope.K + (head - rope.H)) * rope.page_size * D;
        kp[kv_key_offset(rope.tiled, rope.page_size, D, off, d0)] = f32_to_bf16(y0);
        kp[kv_key_offset(rope.tiled, rope.page_size, D, off, d1)] = f32_to_bf16(y1);
      } else {
        bf16_t* vp =
            rope.v_pages + ((size_t)page * rope.K + (head - rope.H - rope.K)) * D * rope.page_size;
        vp[kv_value_offset(rope.tiled, rope.page_size, D, off, d0)] = f32_to_bf16(y0);
        vp[kv_value_offset(rope.tiled, rope.page_size, D, off, d1)] = f32_to_bf16(y1);
      }
    }
    return;
  }
  if constexpr (PREP) {
    // thread (column c of the tile, row m): h += product (rounded to bf16 first, as the
    // unfused way hands it on), the next norm's input, and h^2 for the row's sum
#pragma unroll
    for (int i = 0; i < PREPS; ++i) {
      const int e = tid + i * (int)blockDim.x;
      if (e >= MT * 256) continue;
      const int t = e / 256, c = (e % 256) / 16, m = t * 16 + e % 16, n = n_base + c;
      const int idx = t * 256 + ((c / 4) * 16 + e % 16) * 4 + c % 4;
      float sq = 0.f;
      if (n < N && m < M) {
        float v = 0.f;
        for (int w = 0; w < slots; ++w) v += red[(size_t)w * TILE + idx];
        const float h = prep_h[i] + bf16_to_f32(f32_to_bf16(v));
        ((float*)C)[(size_t)m * ldc + n] = h;
        nf.xw_out[(size_t)m * N + n] = f32_to_bf16(prep_w[i] * bf16_to_f32(f32_to_bf16(h)));
        sq = h * h;
      }
      row_sums[c][m] = sq;
    }
    __syncthreads();
    if (tid < RW) {
      float total = 0.f;
#pragma unroll
      for (int c = 0; c < 16; ++c) total += row_sums[c][tid];
      nf.ss_out[(size_t)blockIdx.x * RW + tid] = total;
    }
    return;
  }
  // element (f, t, lane, i) of the accumulator tile is row n_base + f*16 + (lane/16)*4 + i
  // of W (column of C) and row t*16 + lane%16 of X (row of C)
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
    if constexpr (SCALED) {
      const float rs = row_scale(m);
      v *= rs, v2 *= rs;
    }
    if (GATED) v = v2 * (v / (1.0f + expf(-v)));  // set 0 is the gate, set 1 is up
    const size_t o = (size_t)m * ldc + n;
    if (out_mode == SK_OUT_BF16)
      ((bf16_t*)C)[o] = f32_to_bf16(v);
    else if (out_mode == SK_OUT_F32)
      ((float*)C)[o] = v;
    else
      ((float*)C)[o] += v;
  }
}

template <int NT, int MT, bool GATED, int U, int FLAGS = 0, int PL = 1>
static int launch_skinny(const bf16_t* X, int ldx, const bf16_t* W, const bf16_t* W2, int ldw,
                         void* C, int ldc, int out_mode, int M, int N, int K, int waves,
                         hipStream_t stream, RopeEpilogue rope = RopeEpilogue{},
                         NormFusion nf = NormFusion{}) {
  constexpr int SETS = GATED ? 2 : 1;
  HAL_REQUIRE((FLAGS & SK_PREP) == 0 || waves >= 4,
              "small-batch product: the norm-preparing epilogue takes at least four waves (%d)", waves);
  // LDS for the partial sums of all waves, or of a half, a quarter ... if that is too much
  const size_t per_wave = (size_t)SETS * NT * MT * 256 * sizeof(float);
  int slots = waves;
  while (slots > 1 && (size_t)slots * per_wave > 64 * 1024) slots /= 2;
  const size_t smem = (size_t)slots * per_wave;
  const int blocks = (N + 16 * NT - 1) / (16 * NT);
  // (two row tiles: the accumulators need the registers, and what the loads ahead do not
  // cover is read in the epilogue)
  if constexpr ((FLAGS & SK_SCALED) != 0 && PL < (MT == 1 ? SK_MAX_PART_LOADS : 2)) {
    if (nf.n_parts * 4 * MT > PL * waves * HAL_WAVE)  // more loads per thread
      return launch_skinny<NT, MT, GATED, U, FLAGS, PL * 2>(X, ldx, W, W2, ldw, C, ldc, out_mode, M,
                                                            N, K, waves, stream, rope, nf);
  }
  hipLaunchKernelGGL((skinny_gemm_kernel<NT, MT, GATED, U, FLAGS, PL>), dim3(blocks),
                     dim3(waves * HAL_WAVE), smem, stream, X, ldx, W, W2, ldw, C, ldc, out_mode,
                     M, N, K, slots, rope, nf);
  HAL_LAUNCH_CHECK();
  return 0;
}

// Waves per workgroup, which split K among them: more where there are few workgroups, up
// to about 1,536 waves in all (measured on the projections of a 4,096-wide model at 1 and
// 8 rows: beyond that the products of 256 to 384 workgroups get 1 to 2 us slower).
static int skinny_waves(int blocks, int steps) {
  int waves = 4;
  while (waves < 16 && blocks * waves < 1536 && steps / (waves * 2) >= 4) waves *= 2;
  return waves;
}

// X [M, K] bf16 (M <= 64), W [N, K] bf16, optional W2 [N, K] (gated form: W is the
// gate's weight, W2 is up's).  out_mode: 0 bf16, 1 float32, 2 add into float32.
extern "C" int hal_gemm_bf16_skinny(const void* X, int ldx, const void* W, const void* W2,
                                    int ldw, void* C, int ldc, int out_mode, int M, int N, int K,
                                    hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && M <= 64, "hal_gemm_bf16_skinny: M=%d (at most 64 rows)", M);
  HAL_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "hal_gemm_bf16_skinny: N=%d K=%d (K in steps of 8)", N,
              K);
  HAL_REQUIRE(ldx >= K && (ldw >= K || ldw == 0) && ldc >= N && ldx % 8 == 0 && ldw % 8 == 0,
              "hal_gemm_bf16_skinny: leading dimensions %d %d %d", ldx, ldw, ldc);
  HAL_REQUIRE(out_mode >= 0 && out_mode <= 2, "hal_gemm_bf16_skinny: out_mode %d", out_mode);
  HAL_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)W2 % 16) == 0,
              "hal_gemm_bf16_skinny: operands must be 16-byte aligned");
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
  if (const char* e = getenv("HAL_SKINNY_NT")) nt = atoi(e);
  if (const char* e = getenv("HAL_SKINNY_U")) u = atoi(e);
  if (const char* e = getenv("HAL_SKINNY_WAVES")) waves = atoi(e);
  if (nt != 1 && nt != 2 && nt != 4) nt = 2;
  if (mt >= 2 && nt < 2) nt = 2;
  const int blocks = (N + 16 * nt - 1) / (16 * nt);
  const int steps = (K + 31) / 32;
  if (waves <= 0) {
    waves = skinny_waves(blocks, steps);
  }
  while (waves > 1 && (size_t)sets * nt * mt * 1024 > 64 * 1024) waves /= 2;  // one tile must fit
  // loads in flight per wave: about 16 fragments of 16 bytes
  if (u <= 0) u = 8 / (sets * nt);
  u = u >= 8 ? 8 : (u >= 4 ? 4 : (u >= 2 ? 2 : 1));

#define SK_LAUNCH(NT_, MT_, U_)                                                               \
  do {                                                                                        \
    if (w2)                                                                                   \
      return launch_skinny<NT_, MT_, true, U_>(x, ldx, w, w2, ldw, C, ldc, out_mode, M, N, K, \
                                               waves, stream);                                \
    return launch_skinny<NT_, MT_, false, U_>(x, ldx, w, nullptr, ldw, C, ldc, out_mode, M,   \
                                              N, K, waves, stream);                           \
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

// The same product for at most 32 rows with the RMSNorm before or after it folded in.
// The sums of h^2 come in parts of 16 floats (up to 16 rows) or 32 floats (17 to 32 rows).
// ss_in (or null): X holds bf16(w * bf16(h)) of the norm before this product and ss_in
// [n_parts, 16 or 32] the partial sums of h^2 that the product before left; the result is scaled
// by rsqrt(sum / K + eps) per row.  norm_w (or null, not with W2): C is the float32 stream
// h [M, N]; the result is added into it, xw_out [M, N] receives bf16(norm_w * bf16(h)) and
// ss_out [ceil(N / 16), 16 or 32] this product's partial sums of h^2 for the product after.
// Without norm_w the result goes to C as bf16.
extern "C" int hal_gemm_bf16_skinny_norm(const void* X, int ldx, const void* W, const void* W2,
                                         int ldw, void* C, int ldc, int M, int N, int K,
                                         const float* ss_in, int n_parts, float eps,
                                         const void* norm_w, int norm_w_dtype, void* xw_out,
                                         float* ss_out, hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && M <= 32, "hal_gemm_bf16_skinny_norm: M=%d (at most 32 rows)", M);
  HAL_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "hal_gemm_bf16_skinny_norm: N=%d K=%d", N, K);
  HAL_REQUIRE(ldx >= K && (ldw >= K || ldw == 0) && ldc >= N && ldx % 8 == 0 && ldw % 8 == 0,
              "hal_gemm_bf16_skinny_norm: leading dimensions %d %d %d", ldx, ldw, ldc);
  HAL_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)W2 % 16) == 0 &&
                  ((uintptr_t)ss_in % 16) == 0,
              "hal_gemm_bf16_skinny_norm: operands must be 16-byte aligned");
  HAL_REQUIRE((ss_in != nullptr) != (norm_w != nullptr),
              "hal_gemm_bf16_skinny_norm: the norm before the product or the one after it");
  HAL_REQUIRE(!ss_in || (n_parts > 0 && eps > 0.f), "hal_gemm_bf16_skinny_norm: parts %d", n_parts);
  HAL_REQUIRE(!norm_w || (!W2 && xw_out && ss_out && (norm_w_dtype == HAL_F32 || norm_w_dtype == HAL_BF16)),
              "hal_gemm_bf16_skinny_norm: arguments of the norm after the product");
  if (M == 0) return 0;
  const int blocks = (N + 15) / 16, steps = (K + 31) / 32;
  const int waves = skinny_waves(blocks, steps);
  NormFusion nf{ss_in, n_parts, eps, norm_w, norm_w_dtype, (bf16_t*)xw_out, ss_out};
  const bf16_t* x = (const bf16_t*)X;
  const bf16_t* w = (const bf16_t*)W;
  const bf16_t* w2 = (const bf16_t*)W2;
  // 17 to 32 rows: two row tiles per wave, half as many steps of K in flight
#define SK_NORM_LAUNCH(MT_, GATED_, U_, FLAGS_, W2_, MODE_)                                        \
  return launch_skinny<1, MT_, GATED_, U_, FLAGS_>(x, ldx, w, W2_, ldw, C, ldc, MODE_, M, N, K,    \
                                                   waves, stream, RopeEpilogue{}, nf)
  if (M <= 16) {
    if (w2) SK_NORM_LAUNCH(1, true, 4, SK_SCALED, w2, SK_OUT_BF16);
    if (norm_w) SK_NORM_LAUNCH(1, false, 8, SK_PREP, nullptr, SK_OUT_F32_ADD);
    SK_NORM_LAUNCH(1, false, 8, SK_SCALED, nullptr, SK_OUT_BF16);
  }
  if (norm_w) SK_NORM_LAUNCH(2, false, 4, SK_PREP, nullptr, SK_OUT_F32_ADD);
#undef SK_NORM_LAUNCH
  // the products that read the normed rows take two tiles of W as well (fewer, larger
  // workgroups read X less often), as hal_gemm_bf16_skinny does at these sizes
  const int waves2 = skinny_waves((N + 31) / 32, steps);
  if (w2)
    return launch_skinny<2, 2, true, 2, SK_SCALED>(x, ldx, w, w2, ldw, C, ldc, SK_OUT_BF16, M, N, K,
                                                   waves2, stream, RopeEpilogue{}, nf);
  return launch_skinny<2, 2, false, 4, SK_SCALED>(x, ldx, w, nullptr, ldw, C, ldc, SK_OUT_BF16, M, N,
                                                  K, waves2, stream, RopeEpilogue{}, nf);
}

// The packed q, k, v projection of at most 32 tokens with rotation and append in its
// epilogue.  W is the projection's weight with its rows reordered (see RopeEpilogue) and
// then laid out in tiles as for hal_gemm_bf16_skinny with ldw == 0; q_out [M, H * D]
// receives the rotated queries; rotated keys and the values go to the pages of each
// token's request.  Pairs are (j, j + D/2) and the whole head is rotated.
extern "C" int hal_qkv_rope_append(const void* X, int ldx, const void* W, void* q_out, int M,
                                   int K_in, const int* positions, const int* token_seg,
                                   const int* block_table, int bt_stride, const float* cos_t,
                                   const float* sin_t, int table_len, void* k_pages,
                                   void* v_pages, int H, int K, int D, int page_size, int n_pages,
                                   int tiled, const float* ss_in, int n_parts, float eps,
                                   hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && M <= 32, "hal_qkv_rope_append: M=%d (at most 32 tokens)", M);
  HAL_REQUIRE(!ss_in || (n_parts > 0 && eps > 0.f && ((uintptr_t)ss_in % 16) == 0),
              "hal_qkv_rope_append: partial sums of the norm before");
  HAL_REQUIRE(H > 0 && K > 0 && D > 0 && D % 16 == 0, "hal_qkv_rope_append: heads %d, %d, size %d",
              H, K, D);
  HAL_REQUIRE(K_in > 0 && K_in % 8 == 0 && ldx >= K_in && ldx % 8 == 0,
              "hal_qkv_rope_append: inner size %d, leading dimension %d", K_in, ldx);
  HAL_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0,
              "hal_qkv_rope_append: operands must be 16-byte aligned");
  HAL_REQUIRE(positions && token_seg && block_table && cos_t && sin_t && k_pages && v_pages &&
                  q_out && page_size > 0 && n_pages > 0 && table_len > 0,
              "hal_qkv_rope_append: arguments missing");
  HAL_REQUIRE(!tiled || (page_size % 32 == 0 && D % 32 == 0),
              "hal_qkv_rope_append: the tiled page layout needs pages and heads of a multiple "
              "of 32 (page %d, head %d)", page_size, D);
  if (M == 0) return 0;
  const int N = (H + 2 * K) * D;
  const int blocks = N / 16, steps = (K_in + 31) / 32;
  const int waves = skinny_waves(blocks, steps);
  RopeEpilogue rope{positions, token_seg, block_table, bt_stride, cos_t, sin_t, table_len,
                    (bf16_t*)k_pages, (bf16_t*)v_pages, H, K, D, page_size, n_pages, tiled};
  NormFusion nf{ss_in, n_parts, eps, nullptr, 0, nullptr, nullptr};
#define SK_ROPE_LAUNCH(MT_, U_, FLAGS_)                                                            \
  return launch_skinny<1, MT_, false, U_, FLAGS_>((const bf16_t*)X, ldx, (const bf16_t*)W, nullptr, \
                                                  0, q_out, H * D, SK_OUT_BF16, M, N, K_in, waves,  \
                                                  stream, rope, nf)
  if (M <= 16) {
    if (ss_in) SK_ROPE_LAUNCH(1, 8, SK_ROPE | SK_SCALED);
    SK_ROPE_LAUNCH(1, 8, SK_ROPE);
  }
#undef SK_ROPE_LAUNCH
  const int waves2 = skinny_waves((N + 31) / 32, steps);
  if (ss_in)
    return launch_skinny<2, 2, false, 4, SK_ROPE | SK_SCALED>(
        (const bf16_t*)X, ldx, (const bf16_t*)W, nullptr, 0, q_out, H * D, SK_OUT_BF16, M, N, K_in,
        waves2, stream, rope, nf);
  return launch_skinny<2, 2, false, 4, SK_ROPE>((const bf16_t*)X, ldx, (const bf16_t*)W, nullptr, 0,
                                                q_out, H * D, SK_OUT_BF16, M, N, K_in, waves2,
                                                stream, rope, nf);
}
