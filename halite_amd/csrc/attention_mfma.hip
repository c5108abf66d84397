// Paged attention on the matrix cores (bf16 operands, float32 accumulation and
// softmax), for prefill portions and decode tokens alike.  Compiled for one head size,
// HAL_HEAD_DIM (a multiple of 16, at most 256).
//
// The unit of work is a wavefront with one *item*: 16 query rows of one request and
// one key/value head, against a range of that request's keys.  A query row is a
// (token, head-in-group) pair, token-major, so the heads that share a key/value head
// sit in the same tile and every key is loaded once for all of them.  The host lists
// the items; an item whose key range is not the row's whole range writes a partial
// result (unnormalised sum, running maximum, running denominator) that the merge
// kernel combines with the log-sum-exp rule, the same rule that joins two partial
// attentions in src/halite/transformers/tokainfer/attention_fn.py:147-167.
//
// Per 32 keys a wave computes S^T = K Q^T with v_mfma_f32_16x16x32_bf16 (A = 16 keys x
// 32 dims of K straight from the key page, B = Q^T), the online softmax on the
// accumulator layout (a lane owns one query row and eight keys), and O^T += V^T P^T
// (A = 16 dims x 32 keys straight from the transposed value page, B = the lane's own
// eight probabilities).  The keys of the two 16-key MFMA tiles are interleaved so that
// a lane's eight probabilities are eight consecutive keys, which is one 16-byte load of
// the transposed values.
//
// Two kernels come from one file.  Decode tokens (segments of at most 16 rows) run one
// item per wave and keys and values do not go through LDS: a workgroup takes a piece of a
// tile's key range, its four waves a quarter of the piece each (four items), and their
// sums are joined through LDS at the end, so that a range of one piece needs neither partial
// results in memory nor the merge kernel, and a long range, cut into about as many pieces
// as there are compute units to take them, a quarter as many partial results as waves; the
// workgroup that finishes a tile's last piece merges the partial results in the same launch.
// Prompt portions run four items per workgroup (up to RT_BIG tiles
// each): the waves walk the union of their key ranges together, and each block of keys and
// values goes once from global memory straight into LDS, a step ahead.  Such a workgroup has
// eight waves in two halves: both halves hold the same four items, the first takes the even
// steps of the key walk and the second the odd ones (so the causal work splits evenly), each
// with LDS buffers of its own, and at the end the second half hands its sums to the first
// through LDS, where they are joined by the log-sum-exp rule.  A workgroup then has a CU to
// itself and is done in half the time, and since the host lists the longest walks first the
// workgroups that start late are the short ones.  The halves run half a step apart: the
// softmax of one (vector units) against the products of the other (matrix cores); see the
// loop.
//
// The pages are read in one of three ways: pages in the kernel's fragment order (TILED:
// one contiguous KB per MFMA operand, see kv_key_offset in hal_common.h), row-major pages
// of a power of two of at least 32 tokens (PAGE32: the page number of a block is the
// same for the whole wave), and any other page size (a lane looks its own keys up).
//
// scores, causal rule and grouped heads as in src/halite/transformers/attention.py:
// 647-714 and src/halite/transformers/infer/engine/flashinfer_backend.py:217-261.
#include "hal_common.h"
#include "hal_api.h"

#ifndef HAL_HEAD_DIM
#error "compile with -DHAL_HEAD_DIM=<head size>"
#endif
static_assert(HAL_HEAD_DIM % 16 == 0 && HAL_HEAD_DIM >= 16 && HAL_HEAD_DIM <= 256,
              "head size must be a multiple of 16 up to 256");

#define D HAL_HEAD_DIM
#define KT ((D + 31) / 32)  // 32-wide steps over the head dimension for Q K^T
#define DT (D / 16)         // 16-wide tiles of the head dimension for P V
#define ITEM_INTS 8        // merge items
#define SMALL_ITEM_INTS 12  // items of the kernel for segments of one tile
#define BIG_ITEM_INTS 16  // items of the kernel for long segments
#define RESCALE_SLACK 8.0f  // in powers of two
#define MERGE_FEW_PARTS 8   // up to here a merge item is one wave's work

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 ld16(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8, *(const u32x4*)p);
}
__device__ __forceinline__ bf16x8 zero8() {
  u32x4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
// 2^x for x <= 0 (results below the normal range may flush to zero)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The larger of x in this lane and in the lane 32 (16) places away: the swap instructions
// exchange register halves (quarters) between two registers on the vector unit itself,
// where a shuffle is a trip through the LDS hardware that the wave waits for.
__device__ __forceinline__ float max_across_32(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}
__device__ __forceinline__ float max_across_16(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}
// 16 bytes of every lane from global memory straight into LDS: the wave's 64 pieces land
// one after the other from `lds` on (the same address for the whole wave).
__device__ __forceinline__ void load_to_lds(const bf16_t* src, void* lds) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// item: {segment, first row of tile 0, first key, end key, first partial slot or -1,
//        first row of tile 1, of tile 2, of tile 3 (or -1)}
// An item of the one-tile kernel (12 ints) carries its segment's first token, number of
// tokens and number of keys in the last three of the eight instead, so that the wave need
// not wait for the item before it can ask for them; then the first partial slot of its tile
// and the number of pieces of the tile's key range, if the kernel is to merge them itself
// (else 0, 0), and two unused.
// A wave works on up to RT tiles of 16 rows of one segment; the keys and values it
// loads serve all of them.  The tiles need not be neighbours (the host lists neighbours:
// they share nearly all of their keys).  A tile skips the steps whose keys lie wholly
// outside its own range.  Row tile rt of an
// item writes partial slot `first partial slot + rt`.
#define N_XCD 8
#define WAVES 4  // per workgroup
// Two waves per SIMD leave 256 registers each, which keeps the accumulators in VGPRs (no
// copies to and from AGPRs around every MFMA); the largest head sizes need more.
#define MIN_WAVES_PER_SIMD (D > 160 ? 1 : 2)
template <int RT, bool POW2, bool PAGE32, bool SHARED, bool TILED, int KB, int HALVES>
__global__ void __launch_bounds__(256 * HALVES, MIN_WAVES_PER_SIMD)
attention_mfma_kernel(const bf16_t* __restrict__ q, int q_row_stride, bf16_t* __restrict__ out,
                      int out_row_stride, const int* __restrict__ items,
                      const int* __restrict__ n_items_ptr, const int* __restrict__ seg_q_start,
                      const int* __restrict__ seg_q_len, const int* __restrict__ seg_kv_len,
                      const int* __restrict__ block_table, int bt_stride,
                      const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                      float* __restrict__ part_o, float* __restrict__ part_ml,
                      int* __restrict__ counters, int H, int K, int page_size, int page_shift,
                      float scale_log2e, int window, int max_items) {
  static_assert(HALVES == 1 || (SHARED && HALVES == 2), "only the kernel with LDS has two halves");
  // JOIN (the kernel without LDS for keys): the four items of a workgroup are four pieces of
  // one tile's key range (the host lists them so, in whole runs of four, the last may be
  // empty); their sums are joined through LDS at the end and the first wave writes the
  // result, to the output or to the partial slot that its item names.
  constexpr bool JOIN = !SHARED;
  static_assert(!JOIN || RT == 1, "pieces are joined in the kernel for one tile per wave");
  // wave: within its half (it names the item and the fragments the wave loads)
  const int lane = threadIdx.x % HAL_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane((threadIdx.x / HAL_WAVE) % WAVES);
  const int half_id = __builtin_amdgcn_readfirstlane(threadIdx.x / (HAL_WAVE * WAVES));
  // Workgroups go to the eight XCDs in turn (linear id modulo 8) and each XCD has an L2 of
  // its own: the ids are renumbered so that an XCD gets a contiguous run of (kv head, item
  // block) pairs, i.e. the tiles that read one head's keys meet in one L2.
  int bx = blockIdx.x, g = blockIdx.y;
  {
    const int nx = gridDim.x, n_blocks = nx * gridDim.y;
    if (n_blocks % N_XCD == 0) {
      const int linear = bx + nx * g;
      const int v = (linear % N_XCD) * (n_blocks / N_XCD) + linear / N_XCD;
      g = v / nx;
      bx = v % nx;
    }
  }
  // everything that describes the item is the same for the whole wave: kept in scalar
  // registers, so that loop control, block-level masks and page lookups cost no vector work
  auto uniform = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
  const int item = uniform(bx * WAVES + wave);
  // the item is asked for together with the live count (an index past the list's end is
  // clamped for the address only): one trip to memory instead of two
  // (the kernel for long segments finds in its items of 16 what the other looks up: the
  // segment's scalars and the key range that the workgroup's four items walk together)
  constexpr bool INLINE_SEG = SHARED || RT == 1;
  constexpr int STRIDE_INTS = SHARED ? BIG_ITEM_INTS : SMALL_ITEM_INTS;
  constexpr int PRE_INTS = SHARED ? 13 : 10;
  int pre[PRE_INTS];
  if constexpr (INLINE_SEG) {
    const int* ip = items + (size_t)(item < max_items ? item : max_items - 1) * STRIDE_INTS;
#pragma unroll
    for (int i = 0; i < PRE_INTS; ++i) pre[i] = ip[i];
  }
  const int n_items = *n_items_ptr;
  // SHARED: the four waves of a workgroup have items of one segment (the host lists them
  // so, in whole runs of four, padded with items that have no rows and no keys) and walk
  // the union of their key ranges together; the keys and values of a block are loaded once,
  // by all four, into LDS.  A wave whose item is padding still loads and waits at the
  // barriers.
  if (bx * WAVES >= n_items) return;  // items come in whole runs of four
  const bool have_item = item < n_items;
  const int* it = items + (size_t)(have_item ? item : bx * WAVES) * STRIDE_INTS;
  auto iv = [&](int i) {
    if constexpr (INLINE_SEG) return pre[i];
    else return it[i];
  };
  const int seg = uniform(iv(0));
  const int rho0 = have_item ? uniform(iv(1)) : -1;
  const int kv_begin = have_item ? uniform(iv(2)) : 0, kv_end = have_item ? uniform(iv(3)) : 0;
  const int partial = have_item ? uniform(iv(4)) : -1;
  int walk_begin = kv_begin, walk_end = kv_end;  // the keys this wave walks through
  if constexpr (SHARED) {
    walk_begin = uniform(pre[11]), walk_end = uniform(pre[12]);
    if (walk_begin >= walk_end) return;  // the same for all four waves
  }
  const int G = H / K;
  int q_start, q_len, kv_len;
  if constexpr (SHARED) {
    q_start = uniform(pre[8]), q_len = uniform(pre[9]), kv_len = uniform(pre[10]);
  } else if constexpr (INLINE_SEG) {
    q_start = uniform(pre[5]), q_len = uniform(pre[6]), kv_len = uniform(pre[7]);
  } else {
    q_start = uniform(seg_q_start[seg]), q_len = uniform(seg_q_len[seg]);
    kv_len = uniform(seg_kv_len[seg]);
  }
  const int pos0 = kv_len - q_len;  // position of the segment's first token
  const int* bt = block_table + (size_t)seg * bt_stride;

  // A step of the walk takes KB keys: 32 without LDS, 32 or 64 with it (SUBS blocks of 32).
  static_assert(KB == 32 || (SHARED && KB == 64), "keys per step");
  constexpr int SUBS = KB / 32;
  const int j_first = walk_begin & ~31;
  // PAGE32: page numbers are looked up (scalar loads) well before the loads that need them
  auto page_at = [&](int j0) {
    // (an entry of a page that a window has passed is -1: never an address)
    if constexpr (PAGE32) return max(uniform(bt[(j0 < walk_end ? j0 : j_first) >> page_shift]), 0);
    else return 0;
  };
  // with LDS: the pages of this half's first three steps are asked for here, so that they
  // are on their way while the query rows' addresses are worked out
  int pages_0[SHARED ? SUBS : 1], pages_1[SHARED ? SUBS : 1], pages_2[SHARED ? SUBS : 1];
  if constexpr (SHARED) {
#pragma unroll
    for (int u = 0; u < SUBS; ++u) {
      const int j_mine = j_first + half_id * KB + 32 * u;
      pages_0[u] = page_at(j_mine);
      pages_1[u] = page_at(j_mine + KB * HALVES);
      pages_2[u] = page_at(j_mine + 2 * KB * HALVES);
    }
  }

  const int col = lane % 16, quad = lane / 16;
  // this lane's query row in every row tile
  bool row_ok[RT];
  int qi[RT], head[RT], p_row[RT], lo_row[RT];
  bf16x8 bq[RT][KT];  // Q^T as the B operand: lane holds Q[row][ks*32 + quad*8 .. +8]
  f32x4 o[RT][DT];
  float m[RT], l[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int tile0 = rt == 0 ? rho0 : (have_item ? uniform(iv(4 + rt)) : -1);
    const int rho = tile0 + col;
    row_ok[rt] = tile0 >= 0 && rho < q_len * G;
    qi[rt] = row_ok[rt] ? rho / G : 0;
    head[rt] = g * G + (row_ok[rt] ? rho % G : 0);
    p_row[rt] = pos0 + qi[rt];  // the row's position: it sees keys <= p_row
    lo_row[rt] = (window > 0 && p_row[rt] - window + 1 > 0) ? p_row[rt] - window + 1 : 0;
    const bf16_t* qp = q + (size_t)(q_start + qi[rt]) * q_row_stride + (size_t)head[rt] * D;
#pragma unroll
    for (int ks = 0; ks < KT; ++ks) {
      const int d0 = ks * 32 + quad * 8;
      bq[rt][ks] = (row_ok[rt] && (D % 32 == 0 || d0 < D)) ? ld16(qp + d0) : zero8();
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[rt] = -INFINITY;
    l[rt] = 0.f;
  }

  const int last_key = kv_len - 1;  // keys beyond it are not written yet
  // page and slot of a key; pages of a power of two (page_shift >= 0) need no division
  auto page_of = [&](int j) { return POW2 ? j >> page_shift : j / page_size; };
  auto slot_of = [&](int j) { return POW2 ? j & (page_size - 1) : j % page_size; };
  // per row tile, the positions of its first and last row (uniform over the wave): a
  // block of keys wholly below the first row's position needs no mask
  int p_first[RT], p_last[RT], lo_first[RT], lo_last[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r_first = rt == 0 ? rho0 : (have_item ? uniform(iv(4 + rt)) : -1);
    int r_last = r_first + 15;
    if (r_last > q_len * G - 1) r_last = q_len * G - 1;
    if (r_last < r_first) r_last = r_first;
    p_first[rt] = pos0 + r_first / G;
    p_last[rt] = r_first >= 0 ? pos0 + r_last / G : -1;  // no tile: no key is in range
    lo_first[rt] = (window > 0 && p_first[rt] - window + 1 > 0) ? p_first[rt] - window + 1 : 0;
    lo_last[rt] = (window > 0 && p_last[rt] - window + 1 > 0) ? p_last[rt] - window + 1 : 0;
  }

  // This lane's key of tile t in the block of 32 keys at j0: row `col` of tile t is
  // key j0 + (col/4)*8 + t*4 + col%4; its eight keys for the values are j0 + quad*8 .. +8.
  //
  // PAGE32 (pages of a power of two, at least 32 tokens): a block of 32 keys lies in one
  // page, so the page number and the block's base addresses are the same for the whole
  // wave (scalar registers) and a lane adds constants of its own.  Keys of the page that
  // are outside the item's range or not written yet are loaded like the others (the page
  // is held), their scores are masked and their values cleared.
  //
  // Otherwise every lane looks its keys' pages up itself; keys outside
  // [walk_begin, last_key] are clamped for the address only.
  const int koff0 = ((col / 4) * 8 + (col % 4)) * D + quad * 8;  // tile 1 is 4 keys on
  const int voff = col * page_size + quad * 8;
  auto key_index = [&](int j0, int t) {
    const int j = j0 + (col / 4) * 8 + t * 4 + (col % 4);
    return j < walk_begin ? walk_begin : (j > last_key ? last_key : j);
  };
  auto value_index = [&](int j0) {
    int jv = j0 + quad * 8;
    if constexpr (!PAGE32) {
      if (jv < (walk_begin & ~7)) jv = walk_begin & ~7;
      if (jv > (last_key & ~7)) jv = last_key & ~7;
    }
    return jv;
  };
  // One fragment is what one MFMA takes from the block of 32 keys, 16 bytes a lane:
  // (t, ks) of the keys, dt of the values.
  // (a lane whose 8 dimensions lie past a head size that is no multiple of 32 is pointed
  // at the 16 before them: what it reads meets zeros of Q)
  auto key_frag_ptr = [&](int j0, int page, int t, int ks) -> const bf16_t* {
    int d0 = ks * 32 + quad * 8;
    if (D % 32 != 0 && d0 >= D) d0 -= 16;
    if constexpr (TILED) {  // the fragment is one contiguous KB
      const bf16_t* base =
          k_pages + (((size_t)page * K + g) * page_size + (j0 & (page_size - 1))) * D;
      return base + (t * KT + ks) * 512 + lane * 8;
    } else if constexpr (PAGE32) {
      const bf16_t* base =
          k_pages + (((size_t)page * K + g) * page_size + (j0 & (page_size - 1))) * D;
      return base + (koff0 - quad * 8) + t * 4 * D + d0;
    } else {
      const int j = key_index(j0, t);
      const long long pg = bt[page_of(j)];
      return k_pages + (((size_t)pg * K + g) * page_size + slot_of(j)) * D + d0;
    }
  };
  auto load_key_frag = [&](int j0, int page, int t, int ks) -> bf16x8 {
    if (D % 32 != 0 && ks * 32 + quad * 8 >= D) return zero8();
    return ld16(key_frag_ptr(j0, page, t, ks));
  };
  auto value_frag_ptr = [&](int j0, int page, int dt) -> const bf16_t* {
    // lane loads V^T[dim dt*16 + col][keys jv .. jv+8]
    if constexpr (TILED) {
      const bf16_t* base =
          v_pages + (((size_t)page * K + g) * page_size + (j0 & (page_size - 1))) * D;
      return base + dt * 512 + lane * 8;
    } else if constexpr (PAGE32) {
      const bf16_t* base =
          v_pages + ((size_t)page * K + g) * D * page_size + (j0 & (page_size - 1));
      return base + voff + (size_t)dt * 16 * page_size;
    } else {
      const int jv = value_index(j0);
      const long long pg = bt[page_of(jv)];
      return v_pages + ((size_t)pg * K + g) * D * page_size + slot_of(jv) +
             (size_t)(dt * 16 + col) * page_size;
    }
  };
  auto load_value_frag = [&](int j0, int page, int dt) -> bf16x8 {
    return ld16(value_frag_ptr(j0, page, dt));
  };
  // unwritten slots may hold anything, NaN included, and 0 * NaN must not get in: in the
  // last block of the request the values of keys past the end are cleared
  auto clear_unwritten = [&](int j0, bf16x8 v) -> bf16x8 {
    const int jv = value_index(j0);
    u32x4 raw = __builtin_bit_cast(u32x4, v);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int ja = jv + 2 * w;
      raw[w] &= (ja <= last_key ? 0x0000ffffu : 0u) | (ja + 1 <= last_key ? 0xffff0000u : 0u);
    }
    return __builtin_bit_cast(bf16x8, raw);
  };

  // ---- one step's mask and online softmax, for every row tile: scores in, probabilities
  // (as the B operand of the second product) and the factor for the old sums out.  Of every
  // block of 32 keys this lane has the keys quad*8 + e, e = 0..7.  Raw scores; the scale
  // (positive) goes into the exponent's multiply-add.
  auto softmax_step = [&](int j0, const f32x4 (&s)[RT][SUBS][2], const bool (&active)[RT],
                          bf16x8 (&pb)[RT][SUBS], float (&alpha)[RT]) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      alpha[rt] = 1.f;
#pragma unroll
      for (int u = 0; u < SUBS; ++u) pb[rt][u] = zero8();
      if (!active[rt]) continue;
      float sv[SUBS * 8];
      float m_raw = -INFINITY;
      const bool full = j0 >= kv_begin && j0 + KB <= kv_end && j0 + KB - 1 <= p_first[rt] &&
                        j0 >= lo_last[rt];
      if (full) {  // every key of the step is visible to every row of the tile
#pragma unroll
        for (int e = 0; e < SUBS * 8; ++e) {
          sv[e] = s[rt][e / 8][(e % 8) / 4][e % 4];
          m_raw = fmaxf(m_raw, sv[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < SUBS * 8; ++e) {
          const int j = j0 + (e / 8) * 32 + quad * 8 + e % 8;
          const bool ok =
              row_ok[rt] && j >= kv_begin && j < kv_end && j >= lo_row[rt] && j <= p_row[rt];
          sv[e] = ok ? s[rt][e / 8][(e % 8) / 4][e % 4] : -INFINITY;
          m_raw = fmaxf(m_raw, sv[e]);
        }
      }
      m_raw = max_across_16(max_across_32(m_raw));
      const float m_tile = m_raw * scale_log2e;
      // The running maximum only has to keep exp2(s - m) in range, so it is raised
      // only when the step's maximum exceeds it by more than 2^RESCALE_SLACK: then
      // the accumulated sums are rarely rescaled (and a partial result's m, l and sums
      // stay consistent with each other, which is all the merge needs).
      const float m_new = m_tile > m[rt] + RESCALE_SLACK ? m_tile : m[rt];
      // a row that has seen no key yet keeps m = -inf; subtracting 0 instead of -inf
      // gives exp2(-inf) = 0 everywhere without a branch
      const float m_sub = m_new == -INFINITY ? 0.f : m_new;
      alpha[rt] = fast_exp2(m[rt] - m_sub);
      float pv[SUBS * 8];
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < SUBS * 8; ++e) {
        pv[e] = fast_exp2(__builtin_fmaf(sv[e], scale_log2e, -m_sub));
        psum += pv[e];
      }
      l[rt] = l[rt] * alpha[rt] + psum;
      m[rt] = m_new;
#pragma unroll
      for (int u = 0; u < SUBS; ++u) {
        u32x4 praw = {pack2(pv[u * 8 + 0], pv[u * 8 + 1]), pack2(pv[u * 8 + 2], pv[u * 8 + 3]),
                      pack2(pv[u * 8 + 4], pv[u * 8 + 5]), pack2(pv[u * 8 + 6], pv[u * 8 + 7])};
        pb[rt][u] = __builtin_bit_cast(bf16x8, praw);
      }
    }
    // rescale the sums only if some row of the tile raised its maximum
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (__builtin_amdgcn_ballot_w64(alpha[rt] != 1.f) != 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[rt][dt][r] *= alpha[rt];
      }
    }
  };
  // a step wholly after the tile's last row or before its first row's window does nothing
  // for this tile
  auto tile_active = [&](int j0, int rt) {
    return j0 <= p_last[rt] && j0 + KB - 1 >= lo_first[rt] && j0 < kv_end && j0 + KB > kv_begin &&
           j0 < walk_end;
  };

  constexpr int FK = 2 * KT;                       // key fragments of a block of 32 keys
  constexpr int NFK = SUBS * FK, NFV = SUBS * DT;  // key and value fragments of a step
  constexpr int XCH_VALUES = RT * DT * 4 + 2 * RT;
  constexpr int XCH_BYTES = HALVES == 2 ? WAVES * XCH_VALUES * HAL_WAVE * 4 : 0;
  // With LDS: [half of the workgroup][keys: two buffers of NFK fragments, values: two of
  // NFV][lane]: a fragment lies there in lane order, as the MFMA wants it back.  At the end,
  // with two halves, the same memory carries the second half's sums to the first:
  // [wave][value][lane] floats.
  constexpr int FRAG_BYTES = SHARED ? HALVES * 2 * (NFK + NFV) * HAL_WAVE * 16 : 16;
  __shared__ __align__(16) unsigned char lds_raw[FRAG_BYTES > XCH_BYTES ? FRAG_BYTES : XCH_BYTES];

  if constexpr (SHARED) {
    // Fragment f of a step is brought in by wave f % 4, straight from global memory into
    // LDS (every lane names its own 16 bytes; they land in lane order).  The steps of the
    // walk go to the halves in turn: STRIDE keys from one step of a half to its next; both
    // halves make the same number of steps (the second may have a last one without keys).
    //
    // A step of a half is two blocks of instructions with a barrier before each:
    //   barrier 1 (no data waits for it: it keeps the halves apart);
    //   the block for the vector units: softmax of this step's scores; then the loads that
    //     the wave asked for a step ago have to have landed;
    //   barrier 2: this step's values and the next step's keys are in LDS for all;
    //   the block for the matrix cores: ask for the keys of the step after the next and the
    //     values of the next step (their buffers were read for the last time before
    //     barrier 1), then probabilities times values of this step and keys times queries
    //     of the next, every LDS read asked for one run of products before its use.
    // The second half passes one barrier more before its first step and is thereby half a
    // step behind: one half's softmax runs while the other half's products do.  Left to
    // themselves the two waves of a SIMD fall into step with each other, and the vector
    // units and the matrix cores take turns.
    typedef u32x4 frag_t[HAL_WAVE];
    frag_t* const kbuf = (frag_t*)lds_raw + (size_t)half_id * 2 * (NFK + NFV);
    frag_t* const vbuf = kbuf + 2 * NFK;
    constexpr int STRIDE = KB * HALVES;
    const int n_steps = (walk_end - j_first + STRIDE - 1) / STRIDE;
    auto j_of = [&](int i) { return j_first + i * STRIDE + half_id * KB; };
    auto pages_of = [&](int j0, int (&pages)[SUBS]) {
#pragma unroll
      for (int u = 0; u < SUBS; ++u) pages[u] = page_at(j0 + 32 * u);
    };
    auto ask_keys = [&](int j0, const int (&pages)[SUBS], int b) {
#pragma unroll
      for (int i = 0; i < (NFK + WAVES - 1) / WAVES; ++i) {
        const int f = wave + WAVES * i;
        if (f < NFK)
          load_to_lds(key_frag_ptr(j0 + 32 * (f / FK), pages[f / FK], (f % FK) / KT, f % KT),
                      kbuf + b * NFK + f);
      }
    };
    auto ask_values = [&](int j0, const int (&pages)[SUBS], int b) {
#pragma unroll
      for (int i = 0; i < (NFV + WAVES - 1) / WAVES; ++i) {
        const int f = wave + WAVES * i;
        if (f < NFV)
          load_to_lds(value_frag_ptr(j0 + 32 * (f / DT), pages[f / DT], f % DT), vbuf + b * NFV + f);
      }
    };
    // the values of keys past the request's end are cleared where they landed, by the wave
    // that asked for them (after its loads have come, before the barrier that shows them)
    auto clear_tail_values = [&](int j0, int b) {
#pragma unroll
      for (int i = 0; i < (NFV + WAVES - 1) / WAVES; ++i) {
        const int f = wave + WAVES * i;
        if (f < NFV && j0 + 32 * (f / DT) + 32 > kv_len) {
          u32x4* at = &vbuf[b * NFV + f][lane];
          *at = __builtin_bit_cast(
              u32x4, clear_unwritten(j0 + 32 * (f / DT), __builtin_bit_cast(bf16x8, *at)));
        }
      }
    };
    auto loads_landed = [] { __builtin_amdgcn_s_waitcnt(0x0F70); };  // vmcnt(0)
    // barrier 1 is the instruction alone: no data waits for it (and a fence would wait for
    // the loads that are on their way)
    auto turn_barrier = [] {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    auto data_barrier = [] {
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
    };
    constexpr int FR = FK > DT ? FK : DT;
    bf16x8 fa[FR], fb[FR];  // two sets of fragment registers, filled in turn
    auto read_keys = [&](bf16x8 (&f)[FR], int b, int u) {
#pragma unroll
      for (int x = 0; x < FK; ++x) f[x] = __builtin_bit_cast(bf16x8, kbuf[b * NFK + u * FK + x][lane]);
    };
    auto read_values = [&](bf16x8 (&f)[FR], int b, int u) {
#pragma unroll
      for (int x = 0; x < DT; ++x) f[x] = __builtin_bit_cast(bf16x8, vbuf[b * NFV + u * DT + x][lane]);
    };
    f32x4 s[RT][SUBS][2];
    // consecutive products go to different sums, so none waits for the one before it
    auto keys_times_queries = [&](const bf16x8 (&f)[FR], int u) {
#pragma unroll
      for (int ks = 0; ks < KT; ++ks)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            s[rt][u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                f[t * KT + ks], bq[rt][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[rt][u][t], 0, 0, 0);
    };
    bf16x8 pb[RT][SUBS];
    auto probabilities_times_values = [&](const bf16x8 (&f)[FR], int u) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[dt], pb[rt][u], o[rt][dt], 0, 0, 0);
    };

    {  // (pages_1, pages_2: of the next step and of the one after it)
      ask_keys(j_of(0), pages_0, 0);
      ask_values(j_of(0), pages_0, 0);
      if (1 < n_steps) ask_keys(j_of(1), pages_1, 1);
      loads_landed();
      __syncthreads();
    }
    if constexpr (HALVES == 2) {
      if (half_id == 1) turn_barrier();
    }
    read_keys(fa, 0, 0);
    if constexpr (SUBS == 2) read_keys(fb, 0, 1);
    keys_times_queries(fa, 0);
    if constexpr (SUBS == 2) keys_times_queries(fb, 1);

    for (int i = 0; i < n_steps; ++i) {
      const int j0 = j_of(i), b = i & 1;
      int pages_3[SUBS];
      pages_of(j_of(i + 3), pages_3);
      turn_barrier();  // 1
      // The tiles of a wave go together: a step that concerns one of them is worked on for
      // all (the masks take care of the others); only the last steps of a walk differ.
      bool active[RT];
      bool any = false;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) any = any || tile_active(j0, rt);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) active[rt] = any;
      float alpha[RT];
      softmax_step(j0, s, active, pb, alpha);
      __builtin_amdgcn_sched_barrier(0);
      loads_landed();
      if (j0 + KB > kv_len) clear_tail_values(j0, b);
      data_barrier();  // 2
      // (a step that concerns no tile has probabilities of zero, and after the last step
      // the scores of a step that does not exist are computed from what the buffer holds
      // and never looked at: the run of products has no branch)
      __builtin_amdgcn_s_setprio(2);  // the products go first where both halves could issue
      read_values(fa, b, 0);
      if constexpr (SUBS == 2) read_values(fb, b, 1);
      __builtin_amdgcn_sched_barrier(0);
      if (i + 2 < n_steps) ask_keys(j_of(i + 2), pages_2, b);
      if (i + 1 < n_steps) ask_values(j_of(i + 1), pages_1, b ^ 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (SUBS == 2) {
        probabilities_times_values(fa, 0);
        __builtin_amdgcn_sched_barrier(0);
        read_keys(fa, b ^ 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        probabilities_times_values(fb, 1);
        __builtin_amdgcn_sched_barrier(0);
        read_keys(fb, b ^ 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        keys_times_queries(fa, 0);
        __builtin_amdgcn_sched_barrier(0);
        keys_times_queries(fb, 1);
      } else {
        read_keys(fb, b ^ 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        probabilities_times_values(fa, 0);
        __builtin_amdgcn_sched_barrier(0);
        keys_times_queries(fb, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(0);
#pragma unroll
      for (int u = 0; u < SUBS; ++u) {
        pages_1[u] = pages_2[u];
        pages_2[u] = pages_3[u];
      }
    }
    if constexpr (HALVES == 2) {
      if (half_id == 0) turn_barrier();  // as many barriers as the second half
    }
  } else {
    // Without LDS: this block's values and the next block's keys (a second buffer) are asked
    // for at the block's start; deeper or shallower schedules measured the same or worse.
    int page_0 = page_at(j_first), page_1 = page_at(j_first + 32), page_2 = page_at(j_first + 64);
    bf16x8 kcur[2][KT], knext[2][KT], vf[DT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < KT; ++ks) kcur[t][ks] = load_key_frag(j_first, page_0, t, ks);

    for (int j0 = j_first; j0 < walk_end; j0 += KB) {
      const bool tail = j0 + KB > kv_len;  // some of the keys are not written yet
      const bool more = j0 + KB < walk_end;
      const int page_3 = page_at(j0 + 96);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vf[dt] = load_value_frag(j0, page_0, dt);
      if (more) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int ks = 0; ks < KT; ++ks) knext[t][ks] = load_key_frag(j0 + 32, page_1, t, ks);
      }

      // ---- S^T = K Q^T for 32 keys (two tiles of 16), all row tiles -------------------
      f32x4 s[RT][SUBS][2];
      bool active[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        active[rt] = tile_active(j0, rt);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          s[rt][0][t] = f32x4{0.f, 0.f, 0.f, 0.f};
          if (active[rt]) {
#pragma unroll
            for (int ks = 0; ks < KT; ++ks)
              s[rt][0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kcur[t][ks], bq[rt][ks],
                                                                    s[rt][0][t], 0, 0, 0);
          }
        }
      }
      bf16x8 pb[RT][SUBS];
      float alpha[RT];
      softmax_step(j0, s, active, pb, alpha);

      // ---- O^T += V^T P^T ----------------------------------------------------------
      if (tail) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = clear_unwritten(j0, vf[dt]);
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if (!active[rt]) continue;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb[rt][0], o[rt][dt], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KT; ++ks) kcur[t][ks] = knext[t][ks];
      page_0 = page_1;
      page_1 = page_2;
      page_2 = page_3;
    }
  }
  if constexpr (HALVES == 2) {
    // The second half's sums go to the first through LDS (after a barrier that every wave
    // reaches with its last products done, so the fragment buffers are free), lane to lane:
    // wave w of both halves has the same item, so the same rows in the same lanes.  Joined
    // by the log-sum-exp rule.
    __syncthreads();
    float* xch = (float*)lds_raw + (size_t)wave * XCH_VALUES * HAL_WAVE + lane;
    if (half_id == 1) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        xch[(2 * rt) * HAL_WAVE] = m[rt];
        xch[(2 * rt + 1) * HAL_WAVE] = l[rt];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) xch[(2 * RT + (rt * DT + dt) * 4 + r) * HAL_WAVE] = o[rt][dt][r];
      }
    }
    __syncthreads();
    if (half_id == 1) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float m1 = xch[(2 * rt) * HAL_WAVE], l1 = xch[(2 * rt + 1) * HAL_WAVE];
      const float m_new = fmaxf(m[rt], m1);
      const float m_sub = m_new == -INFINITY ? 0.f : m_new;
      const float a0 = fast_exp2(m[rt] - m_sub), a1 = fast_exp2(m1 - m_sub);
      l[rt] = l[rt] * a0 + l1 * a1;
      m[rt] = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          o[rt][dt][r] = o[rt][dt][r] * a0 + xch[(2 * RT + (rt * DT + dt) * 4 + r) * HAL_WAVE] * a1;
    }
  }

  bool merged_here = false;  // the result is the tile's whole one although the item has a partial slot
  if constexpr (JOIN) {
    // lane to lane: the four waves have the same rows in the same lanes.  Joined by the
    // log-sum-exp rule, in wave order; the result is the first wave's.
    constexpr int JV = DT * 4 + 2;
    __shared__ float joined[WAVES - 1][JV][HAL_WAVE];
    __shared__ int arrived_before;
    float lt = l[0];
    lt += __shfl_xor(lt, 16, HAL_WAVE);
    lt += __shfl_xor(lt, 32, HAL_WAVE);
    auto join_waves = [&]() {
      if (wave > 0) {
        joined[wave - 1][0][lane] = m[0];
        joined[wave - 1][1][lane] = lt;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) joined[wave - 1][2 + dt * 4 + r][lane] = o[0][dt][r];
      }
      __syncthreads();
      if (wave > 0) return;
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) {
        const float m1 = joined[w][0][lane], l1 = joined[w][1][lane];
        const float m_new = fmaxf(m[0], m1);
        const float m_sub = m_new == -INFINITY ? 0.f : m_new;
        const float a0 = fast_exp2(m[0] - m_sub), a1 = fast_exp2(m1 - m_sub);
        lt = lt * a0 + l1 * a1;
        m[0] = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            o[0][dt][r] = o[0][dt][r] * a0 + joined[w][2 + dt * 4 + r][lane] * a1;
      }
    };
    join_waves();
    // A tile whose key range has several pieces (items 8, 9: its first partial slot and their
    // number): the piece's result goes to its partial slot, and the workgroup that finds all
    // the others of the tile done merges them, so that no kernel has to follow for it.  Every
    // tile has a counter, which the last one to come sets back to zero for the next launch.
    // The partial results are read back in the order of the pieces whichever workgroup reads
    // them, so the result does not depend on which came last.
    const int n_pieces = uniform(pre[9]);
    if (n_pieces > 1) {
      // What one workgroup writes and another reads in the same launch goes through loads and
      // stores of device scope (sc1), which pass the caches that are not coherent between
      // workgroups; the count is taken after the stores have completed.  A slot's sums lie in
      // the order [16 dims][lane][4], so that an instruction covers a contiguous KiB.
      auto put = [](float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
      auto get = [](const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
      constexpr int SC1 = 16;                // cache policy of a buffer access: device scope
      constexpr int RAW_BUFFER = 0x00020000;  // descriptor word 3: 32-bit elements, no swizzle
      auto slot_sums = [&](size_t slot) {
        return __builtin_amdgcn_make_buffer_rsrc(part_o + slot * 16 * D, 0, 16 * D * 4, RAW_BUFFER);
      };
      const int first_slot = uniform(pre[8]);
      int* counter = counters + (size_t)first_slot * K + g;
      if (wave == 0) {
        const size_t slot = (size_t)partial * K + g;
        const auto to = slot_sums(slot);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o[0][dt]), to,
                                                 (dt * HAL_WAVE + lane) * 16, 0, SC1);
        if (quad == 0) {
          float* pm = part_ml + (slot * 16 + col) * 2;
          put(pm, m[0]);
          put(pm + 1, lt);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the stores are done
        if (lane == 0)
          arrived_before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __syncthreads();
      if (arrived_before != n_pieces - 1) return;
      if (wave == 0 && lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      m[0] = -INFINITY;
      lt = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[0][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
      // a wave takes every fourth piece, the loads of several in flight at a time
      constexpr int U = DT <= 8 ? 4 : 2;
      for (int i0 = wave; i0 < n_pieces; i0 += WAVES * U) {
        f32x4 po[U][DT];
        float pm[U], pl[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * WAVES;
          const size_t slot = (size_t)(first_slot + (i < n_pieces ? i : i0)) * K + g;
          pm[u] = get(part_ml + (slot * 16 + col) * 2);
          pl[u] = get(part_ml + (slot * 16 + col) * 2 + 1);
          const auto from = slot_sums(slot);
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            po[u][dt] = __builtin_bit_cast(
                f32x4, __builtin_amdgcn_raw_buffer_load_b128(from, (dt * HAL_WAVE + lane) * 16, 0, SC1));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (i0 + u * WAVES >= n_pieces) break;
          const float m_new = fmaxf(m[0], pm[u]);
          const float m_sub = m_new == -INFINITY ? 0.f : m_new;
          const float a0 = fast_exp2(m[0] - m_sub), a1 = fast_exp2(pm[u] - m_sub);
          lt = lt * a0 + pl[u] * a1;
          m[0] = m_new;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[0][dt][r] = o[0][dt][r] * a0 + po[u][dt][r] * a1;
        }
      }
      join_waves();
      merged_here = true;
    }
    if (wave > 0) return;
    l[0] = lt;
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    // the denominator is spread over the four lanes that share a row (joined pieces: it is whole)
    float lt = l[rt];
    if constexpr (!JOIN) {
      lt += __shfl_xor(lt, 16, HAL_WAVE);
      lt += __shfl_xor(lt, 32, HAL_WAVE);
    }
    if (!row_ok[rt]) continue;
    if (partial < 0 || merged_here) {
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      bf16_t* op = out + (size_t)(q_start + qi[rt]) * out_row_stride + (size_t)head[rt] * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 w;
        w.x = pack2(o[rt][dt][0] * inv, o[rt][dt][1] * inv);
        w.y = pack2(o[rt][dt][2] * inv, o[rt][dt][3] * inv);
        *(uint2*)(op + dt * 16 + quad * 4) = w;
      }
    } else {
      const size_t slot = (size_t)(partial + rt) * K + g;
      float* po = part_o + (slot * 16 + col) * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(f32x4*)(po + dt * 16 + quad * 4) = o[rt][dt];
      if (quad == 0) {
        float* pm = part_ml + (slot * 16 + col) * 2;
        pm[0] = m[rt];
        pm[1] = lt;
      }
    }
  }
}

// merge item: {segment, first row (of 16), first partial slot, number of partials,
// slots from one partial to the next, the segment's first token, its number of tokens, 0}
// One block per (merge item, kv head, row of the tile).  The four waves take every
// fourth partial each, four loads in flight at a time, a lane two dimensions; their sums
// are added in wave order through LDS (deterministic).
__global__ void __launch_bounds__(256)
attention_merge_kernel(bf16_t* __restrict__ out, int out_row_stride,
                       const int* __restrict__ merges, const int* __restrict__ n_merges_ptr,
                       const float* __restrict__ part_o, const float* __restrict__ part_ml, int H,
                       int K) {
  constexpr int NC = (D + 127) / 128;  // a lane's pairs of dimensions
  constexpr int MW = 4;                // waves
  __shared__ float red_o[MW][NC * 128];
  __shared__ float red_l[MW];
  __shared__ float scratch[16];
  const int mi = blockIdx.x;
  const int g = blockIdx.y, row = blockIdx.z;
  const int G = H / K;
  // the item is asked for together with the live count (blockIdx.x is below the list's
  // capacity), and it carries what the kernel needs of its segment
  const int* mg = merges + (size_t)mi * ITEM_INTS;
  const int rho0 = mg[1], first = mg[2], n = mg[3], stride = mg[4], q_start = mg[5], q_len = mg[6];
  if (mi >= *n_merges_ptr) return;
  const int rho = rho0 + row;
  if (rho >= q_len * G) return;  // the whole block
  const int lane = threadIdx.x % HAL_WAVE, wave = threadIdx.x / HAL_WAVE;
  auto slot_row = [&](int i) { return ((size_t)(first + i * stride) * K + g) * 16 + row; };

  // A wave's partials go four at a time; the loads of the first four go out before the
  // row's largest maximum is known, which needs a pass over all maxima and a barrier.
  float2 ml[4];
  float2 v[4][NC];
  auto ask = [&](int i0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * MW;
      const size_t base = slot_row(i < n ? i : i0);
      ml[u] = *(const float2*)(part_ml + base * 2);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = c * 128 + lane * 2;
        v[u][c] = d < D ? *(const float2*)(part_o + base * D + d) : float2{0.f, 0.f};
      }
    }
  };
  if (wave < n) ask(wave);

  // the largest running maximum of the row
  float m_all = -INFINITY;
  for (int i = threadIdx.x; i < n; i += blockDim.x) m_all = fmaxf(m_all, part_ml[slot_row(i) * 2]);
  m_all = block_max(m_all, scratch);

  float acc[NC][2];
#pragma unroll
  for (int c = 0; c < NC; ++c) acc[c][0] = acc[c][1] = 0.f;
  float l_all = 0.f;
  for (int i0 = wave; i0 < n; i0 += MW * 4) {
    if (i0 != wave) ask(i0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool ok = i0 + u * MW < n;
      const float w = (!ok || ml[u].x == -INFINITY) ? 0.f : exp2f(ml[u].x - m_all);
      l_all += w * ml[u].y;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        acc[c][0] += w * v[u][c].x;
        acc[c][1] += w * v[u][c].y;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    red_o[wave][c * 128 + lane * 2] = acc[c][0];
    red_o[wave][c * 128 + lane * 2 + 1] = acc[c][1];
  }
  if (lane == 0) red_l[wave] = l_all;
  __syncthreads();
  if (wave != 0) return;
  float l_sum = 0.f;
#pragma unroll
  for (int w = 0; w < MW; ++w) l_sum += red_l[w];
  const float inv = l_sum > 0.f ? 1.0f / l_sum : 0.f;
  const int qi = rho / G, head = g * G + rho % G;
  bf16_t* op = out + (size_t)(q_start + qi) * out_row_stride + (size_t)head * D;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d = c * 128 + lane * 2;
    if (d >= D) continue;
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int w = 0; w < MW; ++w) {
      o0 += red_o[w][d];
      o1 += red_o[w][d + 1];
    }
    *(uint32_t*)(op + d) = pack2(o0 * inv, o1 * inv);
  }
}

// The same for merge items of few partials (prompt portions whose key range was cut in
// two or three): a wave per row, four rows per block, no LDS and no barrier; the
// partials are added in their order.
__global__ void __launch_bounds__(256)
attention_merge_few_kernel(bf16_t* __restrict__ out, int out_row_stride,
                           const int* __restrict__ merges, const int* __restrict__ n_merges_ptr,
                           const float* __restrict__ part_o, const float* __restrict__ part_ml,
                           int H, int K) {
  constexpr int NC = (D + 127) / 128;
  const int mi = blockIdx.x;
  const int lane = threadIdx.x % HAL_WAVE, wave = threadIdx.x / HAL_WAVE;
  const int g = blockIdx.y, row = blockIdx.z * 4 + wave;
  const int G = H / K;
  const int* mg = merges + (size_t)mi * ITEM_INTS;
  const int rho0 = mg[1], first = mg[2], n = mg[3], stride = mg[4], q_start = mg[5], q_len = mg[6];
  if (mi >= *n_merges_ptr) return;
  const int rho = rho0 + row;
  if (rho >= q_len * G) return;
  auto slot_row = [&](int i) { return ((size_t)(first + i * stride) * K + g) * 16 + row; };
  float m_all = -INFINITY;
  for (int i = 0; i < n; ++i) m_all = fmaxf(m_all, part_ml[slot_row(i) * 2]);
  float acc[NC][2];
#pragma unroll
  for (int c = 0; c < NC; ++c) acc[c][0] = acc[c][1] = 0.f;
  float l_all = 0.f;
  for (int i = 0; i < n; ++i) {
    const size_t base = slot_row(i);
    const float2 ml = *(const float2*)(part_ml + base * 2);
    const float w = ml.x == -INFINITY ? 0.f : exp2f(ml.x - m_all);
    l_all += w * ml.y;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = c * 128 + lane * 2;
      if (d >= D) continue;
      const float2 v = *(const float2*)(part_o + base * D + d);
      acc[c][0] += w * v.x;
      acc[c][1] += w * v.y;
    }
  }
  const float inv = l_all > 0.f ? 1.0f / l_all : 0.f;
  const int qi = rho / G, head = g * G + rho % G;
  bf16_t* op = out + (size_t)(q_start + qi) * out_row_stride + (size_t)head * D;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d = c * 128 + lane * 2;
    if (d >= D) continue;
    *(uint32_t*)(op + d) = pack2(acc[c][0] * inv, acc[c][1] * inv);
  }
}

extern "C" int hal_attention_mfma_head_dim() { return D; }

// How many 16-row tiles a wave takes in the kernel for long segments.
#ifndef HAL_RT_BIG
#define HAL_RT_BIG (D <= 64 ? 4 : (D <= 128 ? 2 : 1))
#endif
#define RT_BIG HAL_RT_BIG
// Keys per step of the kernel for long segments: 64 where two halves of that fit 64 KB of LDS.
#ifndef HAL_KB_BIG
#define HAL_KB_BIG (D <= 128 ? 64 : 32)
#endif
#define KB_BIG HAL_KB_BIG

// Halves of a workgroup of that kernel (see the top of the file).
#ifndef HAL_HALVES_BIG
#define HAL_HALVES_BIG 2
#endif
#define HALVES_BIG HAL_HALVES_BIG

extern "C" int hal_attention_mfma_rows_per_big_item() { return 16 * RT_BIG; }

// All arrays are device pointers.  `items` [max_items, 12] lists the work on segments of
// at most 16 query rows (one tile per wave), `big_items` [max_big, 16] the work on longer
// segments (hal_attention_mfma_rows_per_big_item() rows per wave), `merges`
// [max_merges, 8] the row tiles whose key range was cut and whose partial results the merge
// kernel joins.  counts = {items, big items, merges} holds the live numbers, so a captured
// launch can serve varying counts.  `counters` [n_counters] (or null, if no item asks the
// kernel to merge its tile's pieces itself) are zero before the call and zero after it;
// calls that overlap on one GPU must not share them.
extern "C" int hal_attention_mfma(const void* q, int q_row_stride, void* out, int out_row_stride,
                                  const int* items, int max_items, const int* big_items,
                                  int max_big, const int* merges, int max_merges,
                                  const int* counts, const int* seg_q_start,
                                  const int* seg_q_len, const int* seg_kv_len,
                                  const int* block_table, int bt_stride, const void* k_pages,
                                  const void* v_pages, float* part_o, float* part_ml,
                                  int* counters, int n_counters, int H, int K, int head_dim,
                                  int page_size, int tiled, float scale, int window,
                                  int merge_parts, hipStream_t stream) {
  HAL_REQUIRE(head_dim == D, "hal_attention_mfma: built for head size %d, called with %d", D,
              head_dim);
  HAL_REQUIRE(H > 0 && K > 0 && H % K == 0, "hal_attention_mfma: %d heads, %d kv heads", H, K);
  HAL_REQUIRE(K <= 65535, "hal_attention_mfma: %d kv heads exceed the grid limit", K);
  HAL_REQUIRE(page_size > 0 && page_size % 8 == 0,
              "hal_attention_mfma: page size %d must be a multiple of 8", page_size);
  HAL_REQUIRE(q_row_stride % 8 == 0 && out_row_stride % 4 == 0 && ((uintptr_t)q % 16) == 0 &&
                  ((uintptr_t)out % 8) == 0,
              "hal_attention_mfma: q and out rows must be 16-byte aligned");
  HAL_REQUIRE(window >= 0 && max_items >= 0 && max_big >= 0 && max_merges >= 0,
              "hal_attention_mfma: bad counts");
  HAL_REQUIRE(max_merges == 0 || (part_o && part_ml), "hal_attention_mfma: no partial buffers");
  HAL_REQUIRE(!tiled || (D % 32 == 0 && page_size >= 32 && (page_size & (page_size - 1)) == 0),
              "hal_attention_mfma: the tiled page layout needs a head size of a multiple of 32 "
              "and pages of a power of two of at least 32 tokens (head %d, page %d)", D, page_size);
  const float scale_log2e = scale * 1.4426950408889634f;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0)
    for (page_shift = 0; (1 << page_shift) < page_size; ++page_shift) {}
  const int waves = WAVES;
#define LAUNCH_ATTENTION(RT_, SHARED_, KB_, HV_, LIST, MAX, COUNT)                                 \
  {                                                                                               \
    dim3 grid(((MAX) + waves - 1) / waves, K);                                                    \
    auto kernel = attention_mfma_kernel<RT_, false, false, SHARED_, false, KB_, HV_>;             \
    if (tiled) kernel = attention_mfma_kernel<RT_, true, true, SHARED_, D % 32 == 0, KB_, HV_>;   \
    else if (page_shift >= 5) kernel = attention_mfma_kernel<RT_, true, true, SHARED_, false, KB_, HV_>; \
    else if (page_shift >= 0) kernel = attention_mfma_kernel<RT_, true, false, SHARED_, false, KB_, HV_>; \
    hipLaunchKernelGGL(kernel, grid, dim3(waves * HAL_WAVE * HV_), 0, stream, (const bf16_t*)q,   \
                       q_row_stride, (bf16_t*)out, out_row_stride, LIST, COUNT, seg_q_start,      \
                       seg_q_len, seg_kv_len, block_table, bt_stride, (const bf16_t*)k_pages,     \
                       (const bf16_t*)v_pages, part_o, part_ml, counters, H, K, page_size,        \
                       page_shift, scale_log2e, window, MAX);                                     \
    HAL_LAUNCH_CHECK();                                                                           \
  }
  HAL_REQUIRE(max_items % WAVES == 0 && max_big % WAVES == 0,
              "hal_attention_mfma: items come in runs of %d, a workgroup's waves", WAVES);
  HAL_REQUIRE(!counters || (part_o && part_ml && (long long)(max_items / WAVES) * K <= n_counters),
              "hal_attention_mfma: %d counters and the partial buffers do not serve %d items of %d "
              "kv heads", n_counters, max_items, K);
  if (max_items > 0) LAUNCH_ATTENTION(1, false, 32, 1, items, max_items, counts)
  if (max_big > 0) LAUNCH_ATTENTION(RT_BIG, true, KB_BIG, HALVES_BIG, big_items, max_big, counts + 1)
#undef LAUNCH_ATTENTION
  if (max_merges > 0) {
    if (merge_parts > 0 && merge_parts <= MERGE_FEW_PARTS)
      hipLaunchKernelGGL(attention_merge_few_kernel, dim3(max_merges, K, 4), dim3(256), 0, stream,
                         (bf16_t*)out, out_row_stride, merges, counts + 2, part_o, part_ml, H, K);
    else
      hipLaunchKernelGGL(attention_merge_kernel, dim3(max_merges, K, 16), dim3(256), 0, stream,
                         (bf16_t*)out, out_row_stride, merges, counts + 2, part_o, part_ml, H, K);
    HAL_LAUNCH_CHECK();
  }
  return 0;
}
