// The C interface of libholon_hip: one function per device operation, raw device pointers, a HIP stream.
// dtype: 0 = float32, 1 = bfloat16 (activations, weights and cache share it). Index arrays are int32.
// Every function returns 0 on success; otherwise holon_last_error() describes what was refused.
#pragma once
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* holon_last_error(void);
int holon_abi_version(void);

// out[t] = table[ids[t]]; with take_slot and last_token (both or neither), token t is last_token[take_slot[t]] where
// take_slot[t] >= 0: a token the previous step drew and left on the device.
// stats_out (nullable, tokens <= 16): [16] float32, the sum of squares of every row written.
int holon_embedding(const int32_t* ids, const int32_t* take_slot, const int32_t* last_token, const void* table, void* out,
                    int tokens, int hidden, int vocab, int dtype, float* stats_out, void* stream);
// stats[m] = sum of squares of row m of x [rows, dim], rows <= 16.
int holon_row_sumsq(const void* x, float* stats, int rows, int dim, int dtype, void* stream);
// y = rmsnorm(x) over rows of `dim`; with `residual`: residual += x (rounded), y = rmsnorm(residual).
int holon_rmsnorm(const void* x, void* residual, const void* weight, void* y, int64_t rows, int dim, float eps,
                  int dtype, void* stream);
// The same with what is added given as float32 sums over shares of K, parts [splits, rows, dim]: residual +=
// round(parts[0] + parts[1] + ...), y = rmsnorm(residual); residual, weight and y bfloat16.
int holon_rmsnorm_parts(const float* parts, int splits, void* residual, const void* weight, void* y, int64_t rows,
                        int dim, float eps, void* stream);
int holon_silu_mul(const void* gate_up, void* out, int64_t tokens, int inter, int dtype, void* stream);
// Per (token, head): optional rmsnorm over head_dim, optional half-split rotation with table[pos] = cos|sin, then
// q -> q_out [T, heads, D]; k, v -> the paged cache (pages == NULL: only q heads are processed).
int holon_qk_norm_rope_write(const void* qkv, int64_t qkv_stride, void* q_out, int tokens, int heads, int kv_heads,
                             int head_dim, const void* q_weight, const void* k_weight, float eps, const float* table,
                             int rotary_dim, int max_positions, const int32_t* positions, void* pages,
                             const int32_t* write_page, const int32_t* write_off, int page_size, int num_pages,
                             int dtype, void* stream);
int holon_kv_write(const void* k, const void* v, void* pages, const int32_t* write_page, const int32_t* write_off,
                   int tokens, int kv_heads, int head_dim, int page_size, int num_pages, int dtype, void* stream);
// Attention of every query token over its row's cached keys (any dtype, page size and head_dim % 8 == 0).
int holon_attention_generic(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                            const int32_t* slots, const int32_t* lens, const int32_t* query_start, int rows,
                            int tokens, int heads, int kv_heads, int head_dim, int page_size, int num_pages,
                            float scale, int window, int dtype, void* stream);
// Matrix-core attention (bfloat16, head_dim 64/128/256, page_size % 16 == 0). `row_ids` lists the rows served.
int holon_attention_mfma_supported(int head_dim, int page_size, int dtype);
int holon_attention_prefill_bf16(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                                 const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                 const int32_t* row_ids, int n_rows, int max_query, int max_len, int heads,
                                 int kv_heads, int head_dim, int page_size, float scale, int window, void* stream);
// Which kernel long prompt portions of groups of up to 32 heads take: 0 one tile of 32 rows a wave, 2 two tiles a wave,
// 1 (the default) two from 12,288 keys on. Returns the setting before; a negative argument changes nothing.
int holon_attention_prefill_form(int form);
// 1 (default): long portions at head_dim 128 copy their stages into LDS without passing registers; 0: through registers.
// Returns the setting before; a negative argument only asks.
int holon_attention_prefill_copies(int direct);
// One query token per row; the keys are split over `splits` waves of `keys_per_split` keys (a multiple of 32) whose
// partial results (part_o [n_rows, heads, splits, head_dim], part_ml [n_rows, heads, splits, 2], float32) are merged
// in split order.
int holon_attention_decode_bf16(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                                const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                const int32_t* row_ids, int n_rows, int max_len, int heads, int kv_heads, int head_dim,
                                int page_size, float scale, int window, float* part_o, float* part_ml, int splits,
                                int keys_per_split, void* stream);
// The same with `waves` waves a block (1 to 8, a divisor of `splits`), whose partials are combined through LDS: a
// (row, head) leaves splits / waves partials (the workspace's third dimension), and when that is one the block writes
// the result itself (the workspace may then be NULL, and no merge runs). rows_in_order: every row of the step is a
// decode row with row_ids[i] = i and query_start[i] = i (neither array is then read).
int holon_attention_decode_waves_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                      int table_stride, const int32_t* slots, const int32_t* lens,
                                      const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                      int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                      float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                      int rows_in_order, void* stream);
// The same from the step's raw q/k/v projection `qkv` [T, (heads + 2 kv_heads) head_dim]: per-head RMSNorm (q_weight
// and k_weight, both or neither), rotation (rope_table [max_positions, head_dim] = cos | sin, or NULL) and the cache
// write of every row's new token (write_page, write_off by token; its position is the row's len - 1) happen inside
// the attention kernel.
int holon_attention_decode_fused_bf16(const void* qkv, void* out, void* pages, const int32_t* table, int table_stride,
                                      const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                      const int32_t* row_ids, int n_rows, int max_len, int heads, int kv_heads,
                                      int head_dim, int page_size, float scale, int window, const void* q_weight,
                                      const void* k_weight, float eps, const float* rope_table,
                                      int max_positions, const int32_t* write_page, const int32_t* write_off,
                                      float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                      int rows_in_order, void* stream);
// The same decode attention for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The split partials that
// holon_attention_decode_bf16 takes as a workspace live in a device array inside the library instead, of
// HOLON_DECODE_SCRATCH_BYTES on every GPU the library runs on, held until the process ends; no call allocates or frees.
// n_rows * heads * splits * (head_dim + 2) floats (the first part rounded up to 256 bytes) must fit, or the call is
// refused. All calls on one GPU share that GPU's array: calls that overlap on one GPU (other streams, other threads)
// race; calls in one stream's order do not. holon_decode_scratch_init() looks the array's address up for the current
// device ahead of time (the entry point does it at its first call on a device otherwise).
#define HOLON_DECODE_SCRATCH_BYTES (16 << 20)
int holon_decode_scratch_init(void);
int64_t holon_decode_scratch_bytes(void);
int holon_attention_decode_bf16_static(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, const int32_t* slots, const int32_t* lens,
                                       const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                       int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                       int splits, int keys_per_split, void* stream);
// y[M, N] = x[M, K] w[N, K]^T for M <= 16 rows, bfloat16 in, float32 accumulation; out_f32: 0 bfloat16 out, 1 float32
// out, 2 float32 out of values rounded to bfloat16 first;
// tiled says that `w` is holon_tile_weight_bf16's copy ([N/16, K/32, 64, 8]: lane-major 16-byte pieces).
int holon_gemm_skinny_supported(int M, int N, int K);
int holon_gemm_skinny_bf16(const void* x, const void* w, void* y, int M, int N, int K, int out_f32, int tiled,
                           void* stream);
// residual[M, N] = round(residual + round(x w^T)) in place, tiled weights: the product and the residual add that
// follows it in one kernel.
// With stats_out ([N / 16, 16] float32): per block of 16 columns, the sums of squares of the residual values written.
int holon_gemm_skinny_add_bf16(const void* x, const void* w_tiled, void* residual, int M, int N, int K, float* stats_out,
                               void* stream);
// A norm folded into the product: w_tiled holds W * diag(g) (holon_tile_weight_bf16 with `scale`), x the un-normed rows,
// stats [parts, 16] partial sums of squares of x's rows (row m in column m); row m of the result is scaled by
// rsqrt(sum(stats[:, m]) / K + eps) before rounding.
int holon_gemm_skinny_scaled_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K, int out_f32,
                                  const float* stats, int parts, float eps, void* stream);
// y[M, I] = round(silu(round(x gate^T))) * round(x up^T) with w = [gate; up] ([2I, K]), M <= 16.
// stats (nullable): as in holon_gemm_skinny_scaled_bf16 (tiled weights with the norm's weight folded in).
int holon_gemm_skinny_glu_bf16(const void* x, const void* w, void* y, int M, int I, int K, int tiled, const float* stats,
                               int parts, float eps, void* stream);
// The same products for 17 <= M <= 64 rows over tiled weights with many tiles (N / 16 a multiple of 8 and at least
// 1,024; K a multiple of 256): the rows of activations go through LDS, shared by a block's waves, and every wave sums
// its tile over all of K in order. `gated`: N is I and the weight has 2 I rows.
int holon_gemm_rows_supported(int M, int N, int K, int gated);
int holon_gemm_rows_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K, int out_f32, void* stream);
int holon_gemm_rows_glu_bf16(const void* x, const void* w_tiled, void* y, int M, int I, int K, void* stream);
// The same for narrow weights (a few hundred tiles) and up to 128 rows, with K cut into `splits` shares over the grid as well: blocks of
// four waves, N / 16 a multiple of 4, K a multiple of 128 * splits, splits <= 16. parts [splits, M, N]
// float32 holds each share's sums; the product is their sum in order (holon_sum_parts rounds it to bfloat16;
// holon_rmsnorm_parts, the residual add + norm, reads them itself). holon_gemm_rows_splits: the number of shares that
// serves this shape best (0: none does).
int holon_gemm_rows_splits(int M, int N, int K);
int holon_gemm_rows_parts_supported(int M, int N, int K, int splits);
int holon_gemm_rows_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K, int splits,
                               void* stream);
// The same for 129 to 1,024 rows over a weight whose K is at least twice its N (a feed-forward's second product;
// up to 768 rows: one and a half times):
// blocks of 128 rows against 256 columns. holon_gemm_tiles_splits: the shares to take, 0 where the shape is not served
// or not this kernel's to take.
int holon_gemm_tiles_splits(int M, int N, int K);
int holon_gemm_tiles_parts_supported(int M, int N, int K, int splits);
int holon_gemm_tiles_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K, int splits,
                                void* stream);
int holon_sum_parts(const void* parts, void* y, int splits, int64_t count, void* stream);
// y[M, N] = x[M, K] w[N, K]^T, all float32, true 32-bit products and sums in an order that depends on K alone: a row's
// result is bit for bit the same whatever other rows are in the call.
int holon_gemm_f32(const void* x, const void* w, void* y, int M, int N, int K, void* stream);
// scale (nullable, [K] bfloat16): tiled holds round(w[n][k] * scale[k]).
int holon_tile_weight_bf16(const void* w, void* tiled, int N, int K, const void* scale, void* stream);
// `pieces`: room for rows x holon_argmax_pieces(vocab) pairs (float32, int32) when that is not 0 (a wide row is then
// searched by many blocks and a second kernel picks among them), or NULL (one block a row).
int holon_argmax_pieces(int vocab);
int holon_argmax(const float* logits, int32_t* out, int rows, int vocab, void* pieces, void* stream);
// last_token[slots[r]] = tokens[r] for r < rows (slots are distinct; last_token has n_slots entries).
int holon_store_tokens(int32_t* last_token, const int32_t* slots, const int32_t* tokens, int rows, int n_slots,
                       void* stream);
// One token per row. Without `slots`, row r's parameters are temperature[r], top_k[r], ...; with `slots` ([rows]) they
// are tables by slot and row r reads entry slots[r]. `positions` ([rows]: the position of the token being drawn) is
// int32 when positions_i32 is set, int64 otherwise.
int holon_sample(const float* logits, int32_t* out, int rows, int vocab, const float* temperature,
                 const int32_t* top_k, const float* top_p, const float* min_p, const int64_t* seeds,
                 const void* positions, const int32_t* slots, int positions_i32, void* stream);
// dst[idx[r], :] = src[r, :], rows of `width` int32 values; idx outside [0, dst_rows) is skipped.
int holon_scatter_rows(int32_t* dst, const int32_t* idx, const int32_t* src, int rows, int width, int dst_rows,
                       void* stream);

// log_softmax of the raw logits: token_lp[r] for tokens[r], and the k (<= 32) largest with their ids, [rows, k].
int holon_logprobs(const float* logits, const int32_t* tokens, int rows, int vocab, int k, float* token_lp,
                   int32_t* top_ids, float* top_lp, void* stream);

#ifdef __cplusplus
}
#endif
