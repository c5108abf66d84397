// Paged attention in float32 arithmetic throughout: any head size that is a multiple of 4 up
// to 512, any page size, any number of heads and groups, float32 or bf16 storage.  It is the
// whole attention of the 32-bit path and the fallback of the bf16 path for shapes that the
// bf16 matrix-core kernel refuses.  Two kernels: the plain one on the vector units, described
// first, which serves every step, and further down one on the matrix cores' float32
// instruction for steps in which every request brings many tokens (prompts).
//
// A workgroup of four waves serves up to 16 rows that share their keys: a few neighbouring
// tokens of one request times the query heads of one key/value head, so the keys and values
// are read once for all of them.  It walks the keys in blocks of 64 (32 for heads above
// 256), always cut at multiples of the block size counted from the request's first key:
// all threads bring a block's keys [key][D] and values [D][key] into LDS together (the next
// block's loads are in flight while this one is worked on), then wave w takes the rows w,
// w + 4, ...: a lane is a key for the scores and a dimension for the weighted sum.
//
// A row's keys are summed in pieces of 512 (of 256 or 128 where a step has so few rows and
// keys that pieces of 512 would leave the chip empty): a piece starts from nothing, and the
// pieces' sums are joined in the order of the keys by the log-sum-exp rule.  Where a step has
// few rows (decoding) every piece is a workgroup of its own and a second kernel joins them;
// where it has many, one workgroup walks all of a row's pieces and joins as it goes.  Both
// do the same arithmetic in the same order, and every sum over keys is cut at fixed
// multiples counted from the request's first key, so a row's result depends on the row's
// own position, window and request alone, not on what else the step holds.  (Between steps
// that are cut differently the same row differs by rounding: the kernel has two builds,
// blocks of 32 keys for steps of few tokens and of 64 for the others, and the size of the
// pieces follows the size of the step.)
//
// scores, mask, softmax and weighted sum as in
// src/halite/transformers/attention.py:647-714; the causal rule for a portion that
// follows cached tokens (key j visible to the query at position p iff j <= p) is
// the one of src/halite/transformers/infer/engine/flashinfer_backend.py:217-229.
#include "hal_common.h"
#include "hal_api.h"

#define PLAIN_THREADS 256
#define PLAIN_WAVES 4
#define PLAIN_PIECE_SHIFT 9  // a piece has 512 keys,
#define PLAIN_PIECE_LEAST 7  // or 256 or 128 where pieces are workgroups of their own and that many fit
#define PLAIN_PAD 4         // floats between two rows of a tile: 16-byte rows, no bank conflicts

// LDS that one lane of a wave writes and another reads: the wave's LDS operations are done
// in the order they were issued; this keeps the compiler from moving them across
__device__ __forceinline__ void plain_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Maximum and sum over the wave on the vector unit itself (data-parallel moves within a row
// of 16 lanes, then the swaps of register halves between rows): a shuffle would be a trip
// through the LDS hardware each, six in a row that the wave waits for.
template <int CTRL>
__device__ __forceinline__ float plain_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ void plain_swap_16(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void plain_swap_32(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float plain_wave_max(float v) {
  v = fmaxf(v, plain_dpp<0xB1>(v));   // lanes 1 apart (quad_perm 1,0,3,2)
  v = fmaxf(v, plain_dpp<0x4E>(v));   // 2 apart (quad_perm 2,3,0,1)
  v = fmaxf(v, plain_dpp<0x141>(v));  // the mirrored half row
  v = fmaxf(v, plain_dpp<0x140>(v));  // the mirrored row
  float a = v, b = v;
  plain_swap_16(a, b);
  v = fmaxf(a, b);
  a = b = v;
  plain_swap_32(a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float plain_wave_sum(float v) {
  v += plain_dpp<0xB1>(v);
  v += plain_dpp<0x4E>(v);
  v += plain_dpp<0x141>(v);
  v += plain_dpp<0x140>(v);
  float a = v, b = v;
  plain_swap_16(a, b);
  v = a + b;
  a = b = v;
  plain_swap_32(a, b);
  return a + b;
}

// The join of two partial softmax sums, (M, L, A) with (m, l, a): one definition for the
// kernel that walks and the kernel that merges, written without contraction so that both
// compile to the same operations.
__device__ __forceinline__ void plain_join_weights(float M, float m, float& M_new, float& w_old, float& w_new) {
  M_new = fmaxf(M, m);
  w_old = (M == -INFINITY) ? 0.f : expf(M - M_new);
  w_new = (m == -INFINITY) ? 0.f : expf(m - M_new);
}
__device__ __forceinline__ float plain_join(float A, float w_old, float a, float w_new) {
  return __fadd_rn(__fmul_rn(A, w_old), __fmul_rn(a, w_new));
}

// The pieces of a row whose keys are lo .. p, where every piece is a workgroup of its own and
// a row has room for `slots` of them: the smallest pieces that fit (so that a short range
// still spreads over the chip), cut at multiples of their size counted from key 0.
__device__ __forceinline__ int plain_piece_shift(int lo, int p, int slots) {
  int s = PLAIN_PIECE_LEAST;
  while (s < PLAIN_PIECE_SHIFT && (p >> s) - (lo >> s) + 1 > slots) ++s;
  return s;
}

static inline size_t plain_lds_floats(int D, int keys, int rows) {
  return (size_t)keys * (D + PLAIN_PAD) + (size_t)D * (keys + PLAIN_PAD) + (size_t)rows * D +
         (size_t)PLAIN_WAVES * keys + (size_t)2 * 2 * keys;  // tiles, rows, probabilities, places
}

// A block's keys and values on their way to LDS, for both kernels below.  Where a key lies
// (its page's part for this key/value head, its slot) is looked up once per key, by the
// block's first threads, two blocks ahead, and left in LDS.  Keys outside [lo_min, p_max] are
// not read (their pages may not be held) and count as zero; a hole in the block table inside
// that range gives NaN keys, so that it shows.  Of the keys, thread `tid` brings vector kc of
// the rows kr0, kr0 + rows_per_pass, ...; of the values, four keys of a dimension each time.
// (the entry of the block table is asked for in one step of the walk and put down in the
// next, when the wave waits for its loads anyway)
// NV: 16-byte vectors of a tile that a thread brings (KEYS * ceil(D / 64) / 16).
template <typename T, int KEYS, int NV>
struct plain_tiles {
  const T* k_pages;
  const T* v_pages;
  const int* bt;      // the request's row of the block table
  float* k_tile;      // [KEYS][KS]
  float* v_tile;      // [D][VS]
  int2* key_place;    // [2][KEYS]: (page * K + key/value head, slot); -1: a hole, -2: not read
  int KS, VS, D, dv, page_size, page_shift, n_pages, K, g, lo_min, p_max, tid, kc, kr0, rows_per_pass;
  int asked_page, asked_slot;
  float kreg[NV][4], vreg[NV][4];

  __device__ __forceinline__ void ask_place(int j0) {
    asked_slot = -1;
    if (tid < KEYS) {
      const int j = j0 + tid;
      if (j >= lo_min && j <= p_max) {
        const int pg = page_shift >= 0 ? j >> page_shift : j / page_size;
        asked_page = bt[pg];
        asked_slot = j - pg * page_size;
      }
    }
  }
  __device__ __forceinline__ void put_place(int buf) {
    if (tid < KEYS) {
      int2 where = make_int2(-2, 0);  // not read
      if (asked_slot >= 0) {
        where.y = asked_slot;
        where.x = (asked_page >= 0 && asked_page < n_pages) ? asked_page * K + g : -1;  // -1: a hole
      }
      key_place[buf * KEYS + tid] = where;
    }
  }
  __device__ __forceinline__ void fetch(int buf) {
    const int2* place = key_place + buf * KEYS;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      kreg[u][0] = kreg[u][1] = kreg[u][2] = kreg[u][3] = 0.f;
      vreg[u][0] = vreg[u][1] = vreg[u][2] = vreg[u][3] = 0.f;
      const int row = kr0 + u * rows_per_pass;
      if (row < KEYS && kc < dv) {
        const int2 w = place[row];
        if (w.x >= 0) load4(k_pages + ((size_t)w.x * page_size + w.y) * D + kc * 4, kreg[u]);
        else if (w.x == -1) kreg[u][0] = kreg[u][1] = kreg[u][2] = kreg[u][3] = __uint_as_float(0x7fc00000u);
      }
      const int e = tid + u * PLAIN_THREADS;
      const int d = e / (KEYS / 4), jj = (e % (KEYS / 4)) * 4;
      if (d < D) {
        if (page_size % 4 == 0) {  // the four keys lie side by side in one page
          const int2 w = place[jj];
          if (w.x >= 0) {
            load4(v_pages + ((size_t)w.x * D + d) * page_size + w.y, vreg[u]);
            if (place[jj + 3].x < 0) {  // (some of the four are outside the range: their slots may hold anything)
#pragma unroll
              for (int x = 1; x < 4; ++x)
                if (place[jj + x].x < 0) vreg[u][x] = 0.f;
            }
          } else {  // the range may begin among the four
#pragma unroll
            for (int x = 1; x < 4; ++x) {
              const int2 wx = place[jj + x];
              if (wx.x >= 0) vreg[u][x] = to_f32(v_pages[((size_t)wx.x * D + d) * page_size + wx.y]);
            }
          }
        } else {
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            const int2 wx = place[jj + x];
            if (wx.x >= 0) vreg[u][x] = to_f32(v_pages[((size_t)wx.x * D + d) * page_size + wx.y]);
          }
        }
      }
    }
  }
  __device__ __forceinline__ void commit() {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int row = kr0 + u * rows_per_pass;
      if (row < KEYS && kc < dv) store4(k_tile + (size_t)row * KS + kc * 4, kreg[u]);
      const int e = tid + u * PLAIN_THREADS;
      const int d = e / (KEYS / 4), jj = (e % (KEYS / 4)) * 4;
      if (d < D) store4(v_tile + (size_t)d * VS + jj, vreg[u]);
    }
  }
};

// R: 64-wide pieces of a head (head sizes up to 64 * R); KEYS: keys of a block; RW: rows of
// a wave (a workgroup has 4 RW rows at most).  Steps of few tokens run RW = 1 with blocks of
// 32 keys (less LDS and fewer registers, so four workgroups share a compute unit and one's
// loads fly while the others compute), the others RW = 4 with blocks of 64.
// Grid: x = groups of `tq` tokens, y = key/value head times chunk of 4 RW heads of its
// group, z = piece (split) or 1.
// (the build for few tokens is held to the registers that let four workgroups share a
// compute unit, where its LDS allows as many)
template <typename T, int R, int KEYS, int RW>
__global__ void __launch_bounds__(PLAIN_THREADS, (RW == 1 && R <= 2) ? 4 : 1)
attention_plain_kernel(const T* __restrict__ q, int q_row_stride, T* __restrict__ out,
                       int out_row_stride, const int* __restrict__ positions,
                       const int* __restrict__ token_seg, const int* __restrict__ block_table,
                       int bt_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                       float* __restrict__ part, int n_tokens, int H, int K, int D, int page_size,
                       int n_pages, float scale, int window, int tq, int chunks, int split,
                       int max_pieces, int page_shift, int cw_shift) {
  constexpr int NV = KEYS * R / 16;  // 16-byte vectors of a tile that a thread brings
  constexpr int ROWS_MOST = RW * PLAIN_WAVES;
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int lane = tid % HAL_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / HAL_WAVE);
  const int KS = D + PLAIN_PAD, VS = KEYS + PLAIN_PAD;
  float* k_tile = smem;                                // [KEYS][D + pad]
  float* v_tile = k_tile + (size_t)KEYS * KS;           // [D][KEYS + pad]
  float* q_rows = v_tile + (size_t)D * VS;              // [rows][D]
  float* p_mine = q_rows + (size_t)ROWS_MOST * D + (size_t)wave * KEYS;  // [KEYS] per wave
  int2* key_place = (int2*)(q_rows + (size_t)ROWS_MOST * D + (size_t)PLAIN_WAVES * KEYS);  // [2][KEYS]

  const int G = H / K;
  const int g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int heads_here = min(ROWS_MOST, G - chunk * ROWS_MOST);  // heads of this chunk
  const int h_first = g * G + chunk * ROWS_MOST;
  const int t_first = blockIdx.x * tq;
  const int t_end = min(n_tokens, t_first + tq);
  const int dv = D / 4;  // 16-byte vectors of a key's row

  // the tokens of the group go in runs of one request; each run is a walk of its own
  for (int ta = t_first; ta < t_end;) {
    const int seg = token_seg[ta];
    int tb = ta + 1;
    while (tb < t_end && token_seg[tb] == seg) ++tb;
    int p_max = -1, lo_min = 0x7fffffff;
    for (int t = ta; t < tb; ++t) {
      const int p = positions[t];
      const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
      p_max = max(p_max, p);
      lo_min = min(lo_min, lo);
    }
    const int* bt = block_table + (size_t)seg * bt_stride;
    const int n_rows = (tb - ta) * heads_here;
    // the keys this workgroup walks for the run
    int j_begin = lo_min / KEYS * KEYS, j_end = p_max + 1;
    // (pieces as workgroups: a token a workgroup, so the run's range is the range of its rows)
    const int piece_shift = split ? plain_piece_shift(lo_min, p_max, max_pieces) : PLAIN_PIECE_SHIFT;
    if (split) {
      const int pc = (lo_min >> piece_shift) + (int)blockIdx.z;
      j_begin = max(j_begin, pc << piece_shift);
      j_end = min(j_end, (pc + 1) << piece_shift);
    }
    if (j_begin >= j_end) {  // (the same for every thread)
      ta = tb;
      continue;
    }

    __syncthreads();  // the walk before is done with the tiles and the rows
    for (int e = tid; e < n_rows * dv; e += PLAIN_THREADS) {
      const int r = e / dv, i = (e % dv) * 4;
      const T* qp = q + (size_t)(ta + r / heads_here) * q_row_stride + (size_t)(h_first + r % heads_here) * D + i;
      float v[4];
      load4(qp, v);
      store4(q_rows + (size_t)r * D + i, v);
    }

    // this wave's rows: r = wave + 4 * rr
    int row_p[RW], row_lo[RW];
    float M[RW], L[RW], A[RW][R];    // the pieces so far
    float m[RW], l[RW], acc[RW][R];  // the piece at hand
#pragma unroll
    for (int rr = 0; rr < RW; ++rr) {
      const int r = wave + PLAIN_WAVES * rr;
      const int p = r < n_rows ? positions[ta + r / heads_here] : -1;
      row_p[rr] = p;
      row_lo[rr] = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
      M[rr] = m[rr] = -INFINITY;
      L[rr] = l[rr] = 0.f;
#pragma unroll
      for (int c = 0; c < R; ++c) A[rr][c] = acc[rr][c] = 0.f;
    }

    plain_tiles<T, KEYS, NV> tiles;  // (see there for what is read and what counts as zero)
    tiles.k_pages = k_pages, tiles.v_pages = v_pages, tiles.bt = bt;
    tiles.k_tile = k_tile, tiles.v_tile = v_tile, tiles.key_place = key_place;
    tiles.KS = KS, tiles.VS = VS, tiles.D = D, tiles.dv = dv, tiles.page_size = page_size, tiles.page_shift = page_shift;
    tiles.n_pages = n_pages, tiles.K = K, tiles.g = g, tiles.lo_min = lo_min, tiles.p_max = p_max, tiles.tid = tid;
    tiles.kc = tid & ((1 << cw_shift) - 1), tiles.kr0 = tid >> cw_shift, tiles.rows_per_pass = PLAIN_THREADS >> cw_shift;
    tiles.asked_page = 0, tiles.asked_slot = -1;

    tiles.ask_place(j_begin);
    tiles.put_place(0);
    tiles.ask_place(j_begin + KEYS);
    tiles.put_place(1);
    __syncthreads();
    tiles.fetch(0);
    tiles.ask_place(j_begin + 2 * KEYS);
    int buf = 0;
    for (int j0 = j_begin; j0 < j_end; j0 += KEYS, buf ^= 1) {
      __syncthreads();  // every wave has read the block before
      tiles.commit();
      tiles.put_place(buf);  // of the block after the next
      if (j0 + KEYS < j_end) tiles.fetch(buf ^ 1);
      tiles.ask_place(j0 + 3 * KEYS);
      __syncthreads();
      const bool piece_ends = ((j0 + KEYS) & ((1 << piece_shift) - 1)) == 0 || j0 + KEYS >= j_end;
#pragma unroll
      for (int rr = 0; rr < RW; ++rr) {
        const int r = wave + PLAIN_WAVES * rr;
        const bool have_row = r < n_rows;  // (the same for the whole wave)
        const int p = row_p[rr], lo = row_lo[rr];
        if (have_row && j0 <= p && j0 + KEYS > lo) {  // the block holds keys of this row
          // ---- scores: a lane is a key (blocks of 32: the two halves of the wave take a
          // half of the dimensions each, where that is a whole number of vectors) ----
          const int key_lane = lane % KEYS;
          const int j = j0 + key_lane;
          const bool valid = j >= lo && j <= p;
          float s = -INFINITY;
          {
            const bool halves = KEYS == 32 && D % 8 == 0;  // (the same for every lane)
            const int n = halves ? D / 2 : D, from = halves ? (lane / 32) * (D / 2) : 0;
            const float* kr = k_tile + (size_t)key_lane * KS + from;
            const float* qr = q_rows + (size_t)r * D + from;
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll 4
            for (int i = 0; i < n; i += 4) {
              const float4 kk = *(const float4*)(kr + i);
              const float4 qq = *(const float4*)(qr + i);
              d0 = fmaf(kk.x, qq.x, d0);
              d1 = fmaf(kk.y, qq.y, d1);
              d2 = fmaf(kk.z, qq.z, d2);
              d3 = fmaf(kk.w, qq.w, d3);
            }
            float dot = (d0 + d1) + (d2 + d3);
            if constexpr (KEYS == 32) {
              if (!halves && lane >= 32) dot = 0.f;  // (the upper half did the lower half's work again)
              float other = dot;
              plain_swap_32(dot, other);  // (one of the two is this lane's, the other its partner's)
              dot = dot + other;
            }
            if (valid) s = dot * scale;
          }
          const float m_new = fmaxf(m[rr], plain_wave_max(s));
          // (a NaN score makes every sum NaN, as it must; m_new is -inf only if no key is valid)
          const float alpha = (m[rr] == -INFINITY) ? 0.f : expf(m[rr] - m_new);
          const float pj = (valid && lane < KEYS) ? expf(s - m_new) : 0.f;  // (a key counts once)
          l[rr] = l[rr] * alpha + plain_wave_sum(pj);
          m[rr] = m_new;
          if (lane < KEYS) p_mine[lane] = pj;
          plain_wave_sync();
          // ---- weighted sum: a lane is a dimension ----
#pragma unroll
          for (int c = 0; c < R; ++c) {
            const int d = lane + c * HAL_WAVE;
            if (d < D) {
              const float* vr = v_tile + (size_t)d * VS;
              float t0 = 0.f, t1 = 0.f;
#pragma unroll 4
              for (int jj = 0; jj < KEYS; jj += 4) {
                const float4 vv = *(const float4*)(vr + jj);
                const float4 pp = *(const float4*)(p_mine + jj);
                t0 = fmaf(pp.x, vv.x, t0);
                t1 = fmaf(pp.y, vv.y, t1);
                t0 = fmaf(pp.z, vv.z, t0);
                t1 = fmaf(pp.w, vv.w, t1);
              }
              acc[rr][c] = __fadd_rn(__fmul_rn(acc[rr][c], alpha), __fadd_rn(t0, t1));
            }
          }
          plain_wave_sync();  // before the next row's probabilities overwrite these
        }
        if (have_row && piece_ends) {
          // Only pieces that hold keys of the row count (the others would join as nothing,
          // but where pieces are workgroups of their own nobody computes them).
          const int pc = j0 >> piece_shift;
          const bool mine = pc >= (lo >> piece_shift) && pc <= (p >> piece_shift);
          const bool only_piece = (lo >> piece_shift) == (p >> piece_shift);
          if (mine && split && !only_piece) {
            float* dst = part + (((size_t)(ta + r / heads_here) * H + h_first + r % heads_here) * max_pieces + blockIdx.z) * (D + 2);
#pragma unroll
            for (int c = 0; c < R; ++c) {
              const int d = lane + c * HAL_WAVE;
              if (d < D) dst[d] = acc[rr][c];
            }
            if (lane == 0) {
              dst[D] = m[rr];
              dst[D + 1] = l[rr];
            }
          } else if (mine) {
            float M_new, w_old, w_new;
            plain_join_weights(M[rr], m[rr], M_new, w_old, w_new);
            L[rr] = plain_join(L[rr], w_old, l[rr], w_new);
            M[rr] = M_new;
#pragma unroll
            for (int c = 0; c < R; ++c) A[rr][c] = plain_join(A[rr][c], w_old, acc[rr][c], w_new);
          }
          m[rr] = -INFINITY;
          l[rr] = 0.f;
#pragma unroll
          for (int c = 0; c < R; ++c) acc[rr][c] = 0.f;
        }
      }
    }

    // rows whose pieces were all joined here are done
#pragma unroll
    for (int rr = 0; rr < RW; ++rr) {
      const int r = wave + PLAIN_WAVES * rr;
      const int p = row_p[rr], lo = row_lo[rr];
      const bool only_piece = (lo >> piece_shift) == (p >> piece_shift);
      if (r >= n_rows || (split && !(only_piece && blockIdx.z == 0))) continue;
      T* op = out + (size_t)(ta + r / heads_here) * out_row_stride + (size_t)(h_first + r % heads_here) * D;
      const float inv = 1.0f / L[rr];
#pragma unroll
      for (int c = 0; c < R; ++c) {
        const int d = lane + c * HAL_WAVE;
        if (d < D) op[d] = from_f32<T>(__fmul_rn(A[rr][c], inv));
      }
    }
    ta = tb;
  }
}

// The pieces of a row, joined in the order of the keys: one wave per (token, head) whose
// keys lie in more than one piece.
template <typename T, int R>
__global__ void __launch_bounds__(HAL_WAVE)
attention_plain_merge_kernel(T* __restrict__ out, int out_row_stride, const int* __restrict__ positions,
                             const float* __restrict__ part, int H, int D, int window, int max_pieces) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int piece_shift = plain_piece_shift(lo, p, max_pieces);
  const int first = lo >> piece_shift, last = p >> piece_shift;
  if (first == last) return;  // written by the piece's own workgroup
  float M = -INFINITY, L = 0.f, A[R];
#pragma unroll
  for (int c = 0; c < R; ++c) A[c] = 0.f;
  // eight pieces are asked for at once (the joins wait for each other, the loads need not)
  constexpr int AHEAD = 8;
  const float* row = part + ((size_t)t * H + h) * max_pieces * (D + 2);
  for (int base = first; base <= last; base += AHEAD) {
    float mm[AHEAD], ll[AHEAD], aa[AHEAD][R];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const float* src = row + (size_t)(min(base + u, last) - first) * (D + 2);
      mm[u] = src[D];
      ll[u] = src[D + 1];
#pragma unroll
      for (int c = 0; c < R; ++c) {
        const int d = lane + c * HAL_WAVE;
        aa[u][c] = d < D ? src[d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      if (base + u > last) break;
      float M_new, w_old, w_new;
      plain_join_weights(M, mm[u], M_new, w_old, w_new);
      L = plain_join(L, w_old, ll[u], w_new);
      M = M_new;
#pragma unroll
      for (int c = 0; c < R; ++c) A[c] = plain_join(A[c], w_old, aa[u][c], w_new);
    }
  }
  T* op = out + (size_t)t * out_row_stride + (size_t)h * D;
  const float inv = 1.0f / L;
#pragma unroll
  for (int c = 0; c < R; ++c) {
    const int d = lane + c * HAL_WAVE;
    if (d < D) op[d] = from_f32<T>(__fmul_rn(A[c], inv));
  }
}

// ---- steps of many rows a request: the matrix cores' float32 instruction -----------------
// Prompts and their portions.  v_mfma_f32_32x32x2_f32 multiplies and adds in float32 at
// twice the rate of the vector units; scores, softmax and weighted sum stay float32
// throughout.  A workgroup serves up to 128 rows that share their keys (neighbouring tokens
// of one request times the query heads of one key/value head), a wave 32 of them, and walks
// the keys in blocks of 32, cut at multiples of 32 counted from the request's first key.
//
// Both products are computed transposed, so that a lane is a query row in each of them:
//   S^T [key][row] = K [key][d] Q^T [d][row]       (A: the block's keys from LDS, B: q in registers)
//   O^T [d][row]  += V^T [d][key] P^T [key][row]   (A: the block's values from LDS, B: the probabilities)
// The instruction leaves S^T with lane l holding row l % 32 and the 16 keys
// 8 (v / 4) + 4 (l / 32) + v % 4, v = 0 .. 15, which is the order in which the second
// product takes P^T from lane l if its sixteen calls take their two keys each in that
// order too (which keys a call sums is free as long as both operands agree).  So the
// softmax of a row is a loop over a lane's registers and one exchange between the wave's
// halves, and the probabilities never leave the registers.  Likewise the first product's
// calls pair the dimensions d and D / 2 + d: the lower half of the lanes holds q[0 .. D/2),
// the upper half the rest.
//
// A row's maximum and sums are updated block by block; blocks outside a row's range change
// nothing, so a row's result depends on its own position, window and request alone.
// DB: blocks of 32 dimensions of a head (head sizes that are multiples of 8, up to 32 DB).
// Grid: x = groups of `tq` tokens, y = key/value head times chunk of 128 heads of its group.
typedef __attribute__((ext_vector_type(16))) float plain_f32x16;
#define ROWS_KEYS 32
#define ROWS_MOST 128

static inline size_t rows_lds_floats(int D, int db) {
  return (size_t)ROWS_KEYS * (D + PLAIN_PAD) + (size_t)db * 32 * (ROWS_KEYS + PLAIN_PAD) + (size_t)2 * 2 * ROWS_KEYS;
}

template <typename T, int DB>
__global__ void __launch_bounds__(PLAIN_THREADS, 2)
attention_rows_kernel(const T* __restrict__ q, int q_row_stride, T* __restrict__ out, int out_row_stride,
                      const int* __restrict__ positions, const int* __restrict__ token_seg,
                      const int* __restrict__ block_table, int bt_stride, const T* __restrict__ k_pages,
                      const T* __restrict__ v_pages, int n_tokens, int H, int K, int D, int page_size,
                      int n_pages, float scale, int window, int tq, int chunks, int page_shift,
                      int cw_shift) {
  constexpr int KEYS = ROWS_KEYS;
  constexpr int NV = KEYS * ((DB + 1) / 2) / 16;
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int lane = tid % HAL_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / HAL_WAVE);
  const int half = lane / 32, col = lane % 32;
  const int KS = D + PLAIN_PAD, VS = KEYS + PLAIN_PAD;
  float* k_tile = smem;                             // [KEYS][D + pad]
  float* v_tile = k_tile + (size_t)KEYS * KS;        // [32 DB][KEYS + pad], zero from row D on
  int2* key_place = (int2*)(v_tile + (size_t)DB * 32 * VS);  // [2][KEYS]
  for (int e = D * VS + tid; e < DB * 32 * VS; e += PLAIN_THREADS) v_tile[e] = 0.f;

  const int G = H / K;
  const int g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int heads_here = min(ROWS_MOST, G - chunk * ROWS_MOST);
  const int h_first = g * G + chunk * ROWS_MOST;
  const int t_first = blockIdx.x * tq;
  const int t_end = min(n_tokens, t_first + tq);
  const int hd = D / 2;  // dimensions of a half of the lanes

  for (int ta = t_first; ta < t_end;) {  // runs of one request, as above
    const int seg = token_seg[ta];
    int tb = ta + 1;
    while (tb < t_end && token_seg[tb] == seg) ++tb;
    // (a request's tokens follow each other, so do their positions)
    const int p_first = positions[ta], p_max = positions[tb - 1];
    const int lo_min = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int* bt = block_table + (size_t)seg * bt_stride;
    const int n_rows = (tb - ta) * heads_here;
    const int j_begin = lo_min / KEYS * KEYS, j_end = p_max + 1;

    // this lane's row (both halves of the wave have the same 32 rows)
    const int r = wave * 32 + col;
    const bool have_row = r < n_rows;
    const int token = ta + (have_row ? r / heads_here : 0), head = h_first + (have_row ? r % heads_here : 0);
    const int p = have_row ? positions[token] : -1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    // what the wave's rows see between them
    const bool wave_has_rows = wave * 32 < n_rows;
    int wave_lo = 0, wave_p = -1;
    if (wave_has_rows) {
      const int p0 = positions[ta + wave * 32 / heads_here];
      wave_lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
      wave_p = positions[ta + min(wave * 32 + 31, n_rows - 1) / heads_here];
    }
    float qreg[DB * 16];
#pragma unroll
    for (int i = 0; i < DB * 4; ++i) {
      float t[4] = {0.f, 0.f, 0.f, 0.f};
      if (have_row && i * 4 < hd) load4(q + (size_t)token * q_row_stride + (size_t)head * D + half * hd + i * 4, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) qreg[i * 4 + x] = t[x];
    }
    float m = -INFINITY, l = 0.f;  // (l: of this half's keys)
    plain_f32x16 acc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;

    plain_tiles<T, KEYS, NV> tiles;
    tiles.k_pages = k_pages, tiles.v_pages = v_pages, tiles.bt = bt;
    tiles.k_tile = k_tile, tiles.v_tile = v_tile, tiles.key_place = key_place;
    tiles.KS = KS, tiles.VS = VS, tiles.D = D, tiles.dv = D / 4, tiles.page_size = page_size, tiles.page_shift = page_shift;
    tiles.n_pages = n_pages, tiles.K = K, tiles.g = g, tiles.lo_min = lo_min, tiles.p_max = p_max, tiles.tid = tid;
    tiles.kc = tid & ((1 << cw_shift) - 1), tiles.kr0 = tid >> cw_shift, tiles.rows_per_pass = PLAIN_THREADS >> cw_shift;
    tiles.asked_page = 0, tiles.asked_slot = -1;

    __syncthreads();  // the walk before is done with the tiles and the places
    tiles.ask_place(j_begin);
    tiles.put_place(0);
    tiles.ask_place(j_begin + KEYS);
    tiles.put_place(1);
    __syncthreads();
    tiles.fetch(0);
    tiles.ask_place(j_begin + 2 * KEYS);
    int buf = 0;
    for (int j0 = j_begin; j0 < j_end; j0 += KEYS, buf ^= 1) {
      __syncthreads();  // every wave has read the block before
      tiles.commit();
      tiles.put_place(buf);  // of the block after the next
      if (j0 + KEYS < j_end) tiles.fetch(buf ^ 1);
      tiles.ask_place(j0 + 3 * KEYS);
      __syncthreads();
      if (!wave_has_rows || j0 > wave_p || j0 + KEYS <= wave_lo) continue;  // (the same for the whole wave)
      // ---- S^T: lane = (key col, half) for the keys, (row col, half) for q ----
      plain_f32x16 st;
#pragma unroll
      for (int v = 0; v < 16; ++v) st[v] = 0.f;
      const float* kr = k_tile + (size_t)col * KS + half * hd;
#pragma unroll
      for (int i = 0; i < DB * 4; ++i) {
        if (i * 4 < hd) {
          const float4 kk = *(const float4*)(kr + i * 4);
          st = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.x, qreg[i * 4 + 0], st, 0, 0, 0);
          st = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.y, qreg[i * 4 + 1], st, 0, 0, 0);
          st = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.z, qreg[i * 4 + 2], st, 0, 0, 0);
          st = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.w, qreg[i * 4 + 3], st, 0, 0, 0);
        }
      }
      // ---- this row's 16 keys of the block (the other half of the wave has the other 16) ----
      float mx = -INFINITY;
      bool valid[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 8 * (v / 4) + 4 * half + v % 4;
        valid[v] = j >= lo && j <= p;
        st[v] = valid[v] ? st[v] * scale : -INFINITY;
        mx = fmaxf(mx, st[v]);
      }
      {
        float other = mx;
        plain_swap_32(mx, other);  // (one of the two is this lane's, the other its partner's)
        mx = fmaxf(mx, other);
      }
      const float m_new = fmaxf(m, mx);
      // (a NaN score makes every sum NaN, as it must; m_new is -inf only if no key is valid yet)
      const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        st[v] = valid[v] ? expf(st[v] - m_new) : 0.f;
        sum += st[v];
      }
      l = l * alpha + sum;
      m = m_new;
      // ---- O^T: lane = (dimension col of a block, half) for the values, (row col, half) for P^T ----
#pragma unroll
      for (int b = 0; b < DB; ++b) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] *= alpha;
        const float* vr = v_tile + (size_t)(b * 32 + col) * VS + 4 * half;
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          const float4 vv = *(const float4*)(vr + 8 * t4);
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, st[4 * t4 + 0], acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, st[4 * t4 + 1], acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.z, st[4 * t4 + 2], acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.w, st[4 * t4 + 3], acc[b], 0, 0, 0);
        }
      }
    }

    {
      float other = l;
      plain_swap_32(l, other);
      l = l + other;
    }
    if (have_row) {  // element v of a block's 16: dimension 32 b + 8 (v / 4) + 4 half + v % 4
      T* op = out + (size_t)token * out_row_stride + (size_t)head * D;
      const float inv = 1.0f / l;
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          const int d = b * 32 + 8 * v4 + 4 * half;
          if (d < D) {
            const float t[4] = {acc[b][4 * v4] * inv, acc[b][4 * v4 + 1] * inv, acc[b][4 * v4 + 2] * inv, acc[b][4 * v4 + 3] * inv};
            store4(op + d, t);
          }
        }
    }
    ta = tb;
  }
}

// How `hal_attention_simple` cuts a step of `n_tokens` tokens whose longest key range is
// `max_kv_len` and whose requests have `min_q_len` tokens or more each (1 if not known):
// tokens per workgroup, whether pieces are workgroups of their own, the rows of a wave (32:
// the kernel for many rows a request), the pieces' number and the floats of partial sums that
// the caller must bring then.  The two numbers decide how fast a step is, never a result.
static bool rows_kernel_serves(int G, int D, int min_q_len) {
  // a wave's 32 rows are there in every request, and the head fits the registers
  return D % 8 == 0 && D <= 128 && (long long)min_q_len * G >= 32;
}

extern "C" int hal_attention_simple_plan(int n_tokens, int H, int K, int D, int max_kv_len, int min_q_len,
                                         int* tq, int* split, int* rows_per_wave, int* max_pieces,
                                         long long* part_floats) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && K > 0 && D > 0 && H % K == 0 && max_kv_len >= 0 && min_q_len >= 0,
              "hal_attention_simple_plan: bad sizes T=%d H=%d K=%d D=%d keys=%d tokens a request=%d", n_tokens, H,
              K, D, max_kv_len, min_q_len);
  const int G = H / K;
  if (rows_kernel_serves(G, D, min_q_len)) {
    *tq = G >= ROWS_MOST ? 1 : ROWS_MOST / G;
    *split = 0;
    *rows_per_wave = 32;
    *max_pieces = 1;
    *part_floats = 0;
    return 0;
  }
  const int rows_most = D > 256 ? PLAIN_WAVES : 4 * PLAIN_WAVES;
  const int chunks = (G + rows_most - 1) / rows_most;
  int together = G >= rows_most ? 1 : rows_most / G;  // tokens whose rows fill a workgroup
  const long long groups = ((long long)n_tokens + together - 1) / together * K * chunks;
  // Few workgroups: a token each, and a piece each.  A workgroup's walk waits for memory block
  // after block (4 us a block of 32 keys where it has a compute unit to itself), so a row gets
  // as many slots for pieces as it takes for 1024 workgroups (at most 64, and no more than
  // pieces of 128 keys could fill), and the kernel cuts each row's own range into the smallest
  // pieces that fit its slots.  Pieces of 512 keys always fit (one more where a window's range
  // begins inside a piece).
  const int whole = (max_kv_len + (1 << PLAIN_PIECE_SHIFT) - 1) / (1 << PLAIN_PIECE_SHIFT) + 1;
  const int least = (max_kv_len + (1 << PLAIN_PIECE_LEAST) - 1) / (1 << PLAIN_PIECE_LEAST) + 1;
  const long long alone = (long long)n_tokens * K * ((G + PLAIN_WAVES - 1) / PLAIN_WAVES);  // groups of a token each
  const int wanted = alone > 0 ? (int)min((1024 + alone - 1) / alone, (long long)64) : 1;
  const int pieces = max(whole, min(wanted, least));
  *split = (groups < 512 && max_kv_len > (1 << PLAIN_PIECE_LEAST)) ? 1 : 0;
  *tq = *split ? 1 : together;
  // a token whose heads are at most four: a row a wave
  *rows_per_wave = (*tq == 1 && G <= PLAIN_WAVES) || D > 256 ? 1 : 4;
  *max_pieces = pieces;
  *part_floats = *split ? (long long)n_tokens * H * pieces * (D + 2) : 0;
  return 0;
}

extern "C" int hal_attention_simple(const void* q, int q_row_stride, void* out,
                                    int out_row_stride, int dtype, const int* positions,
                                    const int* token_seg, const int* block_table, int bt_stride,
                                    const void* k_pages, const void* v_pages, float* part,
                                    int n_tokens, int H, int K, int D, int page_size, int n_pages,
                                    float scale, int window, int max_kv_len, int min_q_len,
                                    hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && K > 0 && D > 0 && page_size > 0 && n_pages > 0,
              "hal_attention_simple: bad sizes T=%d H=%d K=%d D=%d page=%d pages=%d", n_tokens, H,
              K, D, page_size, n_pages);
  HAL_REQUIRE(H % K == 0, "hal_attention_simple: %d query heads are not a multiple of %d kv heads",
              H, K);
  HAL_REQUIRE(D % 4 == 0 && D <= 512, "hal_attention_simple: head size %d is not a multiple of 4 up to 512", D);
  HAL_REQUIRE(window >= 0 && max_kv_len >= 0, "hal_attention_simple: window %d, keys %d", window, max_kv_len);
  HAL_REQUIRE(q_row_stride % 4 == 0 && out_row_stride % 4 == 0,
              "hal_attention_simple: rows of %d and %d elements are not multiples of 4", q_row_stride, out_row_stride);
  if (n_tokens == 0) return 0;
  int tq, split, rw, max_pieces;
  long long part_floats;
  if (hal_attention_simple_plan(n_tokens, H, K, D, max_kv_len, min_q_len, &tq, &split, &rw, &max_pieces, &part_floats))
    return 1;
  HAL_REQUIRE(!split || part != nullptr, "hal_attention_simple: %lld floats of partial sums are needed", part_floats);
  const int G = H / K;
  int page_shift = -1;  // pages of a power of two need no division
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  int cw_shift = 0;  // a key's row of D / 4 vectors goes to the next power of two of threads
  while ((1 << cw_shift) < D / 4) ++cw_shift;
  HAL_REQUIRE((long long)n_pages * K < (1ll << 31), "hal_attention_simple: %d pages of %d heads exceed the index range", n_pages, K);
  if (rw == 32) {
    const int chunks = (G + ROWS_MOST - 1) / ROWS_MOST, db = (D + 31) / 32;
    const size_t smem = rows_lds_floats(D, db) * sizeof(float);
    const long long gy = (long long)K * chunks;
    HAL_REQUIRE(gy <= 65535, "hal_attention_simple: %lld head chunks exceed the grid limit", gy);
    dim3 grid((n_tokens + tq - 1) / tq, (unsigned)gy);
#define ROWS_LAUNCH(T_, DB_)                                                                          \
  hipLaunchKernelGGL((attention_rows_kernel<T_, DB_>), grid, dim3(PLAIN_THREADS), smem, stream,        \
                     (const T_*)q, q_row_stride, (T_*)out, out_row_stride, positions, token_seg,       \
                     block_table, bt_stride, (const T_*)k_pages, (const T_*)v_pages, n_tokens, H, K, D, \
                     page_size, n_pages, scale, window, tq, chunks, page_shift, cw_shift)
#define ROWS_BY_SIZE(T_)                  \
  do {                                    \
    if (db == 1) ROWS_LAUNCH(T_, 1);      \
    else if (db == 2) ROWS_LAUNCH(T_, 2); \
    else if (db == 3) ROWS_LAUNCH(T_, 3); \
    else ROWS_LAUNCH(T_, 4);              \
  } while (0)
    if (dtype == HAL_F32)
      ROWS_BY_SIZE(float);
    else if (dtype == HAL_BF16)
      ROWS_BY_SIZE(bf16_t);
    else
      return hal_fail("hal_attention_simple: unknown dtype %d", dtype);
#undef ROWS_BY_SIZE
#undef ROWS_LAUNCH
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const int rows_most = rw * PLAIN_WAVES;
  const int chunks = (G + rows_most - 1) / rows_most;
  const int keys = rw == 1 ? 32 : 64;
  const size_t smem = plain_lds_floats(D, keys, rows_most) * sizeof(float);
  HAL_REQUIRE(smem <= 160 * 1024, "hal_attention_simple: head size %d needs %zu bytes of LDS", D, smem);
  const long long gy = (long long)K * chunks;
  HAL_REQUIRE(gy <= 65535 && max_pieces <= 65535, "hal_attention_simple: %lld head chunks or %d pieces exceed the grid limit", gy, max_pieces);
  dim3 grid((n_tokens + tq - 1) / tq, (unsigned)gy, split ? max_pieces : 1);
  dim3 merge_grid(n_tokens, H);
#define PLAIN_LAUNCH(T_, R_, KEYS_, RW_)                                                                  \
  do {                                                                                              \
    static bool raised = false; /* more than 64 KB of LDS has to be asked for, once per kernel */    \
    if (!raised) {                                                                                  \
      HAL_CHECK_HIP(hipFuncSetAttribute((const void*)attention_plain_kernel<T_, R_, KEYS_, RW_>,         \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));   \
      raised = true;                                                                                \
    }                                                                                               \
    hipLaunchKernelGGL((attention_plain_kernel<T_, R_, KEYS_, RW_>), grid, dim3(PLAIN_THREADS), smem,     \
                       stream, (const T_*)q, q_row_stride, (T_*)out, out_row_stride, positions,      \
                       token_seg, block_table, bt_stride, (const T_*)k_pages, (const T_*)v_pages,    \
                       part, n_tokens, H, K, D, page_size, n_pages, scale, window, tq, chunks,       \
                       split, max_pieces, page_shift, cw_shift);                                     \
    if (split)                                                                                      \
      hipLaunchKernelGGL((attention_plain_merge_kernel<T_, R_>), merge_grid, dim3(HAL_WAVE), 0,      \
                         stream, (T_*)out, out_row_stride, positions, part, H, D, window,            \
                         max_pieces);                                                                \
  } while (0)
#define PLAIN_BY_ROWS(T_, R_)                    \
  do {                                           \
    if (rw == 1) PLAIN_LAUNCH(T_, R_, 32, 1);    \
    else PLAIN_LAUNCH(T_, R_, 64, 4);            \
  } while (0)
#define PLAIN_BY_SIZE(T_)                        \
  do {                                           \
    if (D <= 64) PLAIN_BY_ROWS(T_, 1);           \
    else if (D <= 128) PLAIN_BY_ROWS(T_, 2);     \
    else if (D <= 256) PLAIN_BY_ROWS(T_, 4);     \
    else PLAIN_LAUNCH(T_, 8, 32, 1);             \
  } while (0)
  if (dtype == HAL_F32)
    PLAIN_BY_SIZE(float);
  else if (dtype == HAL_BF16)
    PLAIN_BY_SIZE(bf16_t);
  else
    return hal_fail("hal_attention_simple: unknown dtype %d", dtype);
#undef PLAIN_BY_SIZE
#undef PLAIN_BY_ROWS
#undef PLAIN_LAUNCH
  HAL_LAUNCH_CHECK();
  return 0;
}
