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

int holon_embedding(const int32_t* ids, const void* table, void* out, int tokens, int hidden, int vocab, int dtype,
                    void* stream);
// y = rmsnorm(x) over rows of `dim`; with `residual`: residual += x (rounded), y = rmsnorm(residual).
int holon_rmsnorm(const void* x, void* residual, const void* weight, void* y, int64_t rows, int dim, float eps,
                  int dtype, void* stream);
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
int holon_argmax(const float* logits, int32_t* out, int rows, int vocab, void* stream);
int holon_sample(const float* logits, int32_t* out, int rows, int vocab, const float* temperature,
                 const int32_t* top_k, const float* top_p, const float* min_p, const int64_t* seeds,
                 const int64_t* positions, void* stream);

#ifdef __cplusplus
}
#endif
