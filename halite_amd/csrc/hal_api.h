// The C interface of the kernel library.  Every function launches on the given
// stream, returns 0 on success and otherwise leaves a message for
// hal_last_error().  Pointers are device pointers unless a comment says otherwise;
// dtype codes are HAL_F32 = 0 and HAL_BF16 = 1.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* hal_last_error();
int hal_version();

int hal_embedding(const int* ids, const void* table, int table_dtype, float* out, int n_tokens,
                  int d, int vocab, hipStream_t stream);

int hal_take_tokens(const int* src, int n_src, int* tokens, int n, hipStream_t stream);

int hal_rmsnorm(float* h, const void* delta, const int* rows, const void* w, int w_dtype,
                float eps, void* out, int dtype, int n_rows, int d, int update_h,
                hipStream_t stream);

int hal_residual_add(float* h, const void* delta, int dtype, long long n, hipStream_t stream);

int hal_silu_mul(const void* gu, void* out, int dtype, int n_tokens, int F, hipStream_t stream);

// out [m, d] = bf16(x * rsqrt(sum_p ss[p][row] / d + eps)): the rows of an RMSNorm whose
// scaling was left to the reader (x = bf16(w * bf16(h)), ss [n_parts, row_width] partial
// sums of h^2), for a reader that does not scale by itself.
int hal_scale_normed_rows(const void* x, int ldx, const float* ss, int n_parts, int row_width,
                          float eps, void* out, int m, int d, hipStream_t stream);

int hal_rope_append(void* qkv, int dtype, int row_stride, const int* positions,
                    const int* token_seg, const int* block_table, int bt_stride,
                    const float* cos_t, const float* sin_t, int table_len, void* k_pages,
                    void* v_pages, int n_tokens, int H, int K, int D, int rot, int interleaved,
                    int page_size, int n_pages, int tiled, hipStream_t stream);

// `max_kv_len`: no request of the step has more keys (an upper bound will do); `min_q_len`:
// none has fewer tokens in the step (a lower bound will do, 1 if not known).  They decide how
// the step is cut, never a result.  `hal_attention_simple_plan` says how; if `split`, `part`
// must bring `part_floats` floats for the pieces' partial sums.
int hal_attention_simple_plan(int n_tokens, int H, int K, int D, int max_kv_len, int min_q_len, int* tq,
                              int* split, int* rows_per_wave, int* max_pieces, long long* part_floats);
int hal_attention_simple(const void* q, int q_row_stride, void* out, int out_row_stride,
                         int dtype, const int* positions, const int* token_seg,
                         const int* block_table, int bt_stride, const void* k_pages,
                         const void* v_pages, float* part, int n_tokens, int H, int K, int D,
                         int page_size, int n_pages, float scale, int window, int max_kv_len,
                         int min_q_len, hipStream_t stream);

int hal_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M,
                 int N, int K, hipStream_t stream);

// X [M <= 64, K] bf16, W [N, K] bf16, optional W2 [N, K] (gated: up * silu(gate), W the gate).
// out_mode: 0 bf16, 1 float32, 2 add into float32.
int hal_gemm_bf16_skinny(const void* X, int ldx, const void* W, const void* W2, int ldw, void* C,
                         int ldc, int out_mode, int M, int N, int K, hipStream_t stream);

// The packed q, k, v projection of M <= 32 tokens with the rotation of q and k (pairs
// (j, j + D/2), whole head) and the append of k and v to the pages in its epilogue.  W:
// the weight's rows reordered per head to [8j .. 8j+7, D/2 + 8j .. D/2 + 8j+7] for
// j = 0 .. D/16 - 1, then tiled as for ldw == 0 above.  q_out [M, H * D] bf16.  ss_in (or
// null), n_parts, eps: the norm before the projection, as for hal_gemm_bf16_skinny_norm.
int hal_qkv_rope_append(const void* X, int ldx, const void* W, void* q_out, int M, int K_in,
                        const int* positions, const int* token_seg, const int* block_table,
                        int bt_stride, const float* cos_t, const float* sin_t, int table_len,
                        void* k_pages, void* v_pages, int H, int K, int D, int page_size,
                        int n_pages, int tiled, const float* ss_in, int n_parts, float eps,
                        hipStream_t stream);

// The product for M <= 32 rows with the RMSNorm before it (ss_in: partial sums of squares
// [n_parts, 16] (32 for more than 16 rows) left by the product before; X holds
// bf16(w * bf16(h))) or after it (norm_w: C is the float32 stream h, added into; xw_out [M, N]
// and ss_out [ceil(N/16), 16 or 32] are left for the product after) folded in.
int hal_gemm_bf16_skinny_norm(const void* X, int ldx, const void* W, const void* W2, int ldw,
                              void* C, int ldc, int M, int N, int K, const float* ss_in,
                              int n_parts, float eps, const void* norm_w, int norm_w_dtype,
                              void* xw_out, float* ss_out, hipStream_t stream);

int hal_sample(const float* logits, int ld, int n_rows, int V, const float* temperature,
               const int* top_k, const float* top_p, const float* min_p, const uint64_t* seeds,
               const int* draw_index, int* out_token, float* out_logprob, uint32_t* key_rows,
               hipStream_t stream);

// Greedy decoding of every row, each row spread over 32 blocks.  `parts`: n_rows * 32 * 4 floats.
int hal_sample_greedy(const float* logits, int ld, int n_rows, int V, float* parts,
                      int* out_token, float* out_logprob, hipStream_t stream);

// hal_sample_greedy without any allocation.  This entry point has no counterpart in the
// reference.  It is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  The partial results go
// to an array that the library holds on every GPU it runs on (512 KiB, there until the
// process ends) instead of to `parts`; at most hal_sample_greedy_static_max_rows() (1024)
// rows, more are refused.  It calls no hipMalloc, hipFree or allocating routine.  All calls
// on one GPU share that array: calls that may overlap there (other streams, other host
// threads) race; calls on one stream do not.
int hal_sample_greedy_static_max_rows();
int hal_sample_greedy_static(const float* logits, int ld, int n_rows, int V, int* out_token,
                             float* out_logprob, hipStream_t stream);

// Rows without filters, greedy or drawn from the whole temperature-scaled distribution; each
// row is spread over 32 blocks.  `parts`: room for n_rows * 32 * 4 floats.
int hal_sample_unfiltered(const float* logits, int ld, int n_rows, int V, const float* temperature,
                          const int* top_k, const uint64_t* seeds, const int* draw_index,
                          float* parts, int* out_token, float* out_logprob, hipStream_t stream);

// Rows with filters spread over 32 blocks a pass.  any_late: some row has top-k, top-p and
// min-p all at once (searched twice).  parts: n_rows * 32 * 4 floats; kept: n_rows * 32
// floats; state: n_rows * 20 words; hist: n_rows * 2 * 2048 64-bit words.
int hal_sample_spread(const float* logits, int ld, int n_rows, int V, const float* temperature,
                      const int* top_k, const float* top_p, const float* min_p,
                      const uint64_t* seeds, const int* draw_index, float* parts, float* kept,
                      void* state, void* hist, int any_late, int* out_token, float* out_logprob,
                      hipStream_t stream);

// ---- the head-size-specific library (attention_mfma.hip) ---------------------------------
int hal_attention_mfma_head_dim();
int hal_attention_mfma_rows_per_big_item();
// merge_parts: the most partial results that any merge item joins, or 0 if not known (the
// kernel for many partials is taken then).  Items of both lists come in runs of four, a
// workgroup's waves (max_items and max_big are multiples of four): the one-tile items of a
// run are four pieces of one piece of a tile's key range (the last may be empty), whose sums
// the kernel joins itself, into the output or the run's partial slot.  counters: zeroed
// ints (left zeroed), one per (partial slot, kv head), for the one-tile items that ask the
// kernel to merge their tile's partial results itself; null if none does.
int hal_attention_mfma(const void* q, int q_row_stride, void* out, int out_row_stride,
                       const int* items, int max_items, const int* big_items, int max_big,
                       const int* merges, int max_merges, const int* counts,
                       const int* seg_q_start, const int* seg_q_len, const int* seg_kv_len,
                       const int* block_table, int bt_stride, const void* k_pages,
                       const void* v_pages, float* part_o, float* part_ml, int* counters,
                       int n_counters, int H, int K, int head_dim, int page_size, int tiled,
                       float scale, int window, int merge_parts, hipStream_t stream);

}  // extern "C"
