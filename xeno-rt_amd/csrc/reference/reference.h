// Plain C++ references of the kernel library's operations (reference.cpp): float32, host memory, no HIP.
// Arguments as in xrt_hip.h, without element type codes, workspaces and streams.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

int xrt_ref_block_tokens(void);
// element offset of (token, dim) of a key, and of (dim, token) of a value, within the cache block of one key/value head
int xrt_ref_cache_key_offset(int token, int dim, int head_dim);
int xrt_ref_cache_value_offset(int dim, int token, int head_dim);
void xrt_ref_embed(const float* table, const int* ids, float* out, int tokens, int hidden);
void xrt_ref_add(float* residual, const float* delta, long count);
void xrt_ref_rmsnorm(const float* x, const float* weight, float eps, float* out, const int* rows, int n_rows, int hidden);
void xrt_ref_linear(const float* a, const float* w, float* out, int M, int N, int K, int mode);
void xrt_ref_qkv_prepare(float* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const int* positions,
                         const int* slots, const float* q_norm, const float* k_norm, float norm_eps,
                         const float* rope_theta, int rope_dim, float rope_scale, float* k_cache, float* v_cache,
                         const int* block_table, int table_stride, int n_blocks);
void xrt_ref_attention(const float* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const float* k_cache,
                       const float* v_cache, const int* block_table, int table_stride, const int* positions,
                       const int* slots, float* out, float scale, int window, const float* distance_slopes);
void xrt_ref_sample(const float* logits, int rows, int vocab, int* out, const float* temperature, const int* top_k,
                    const float* top_p, const float* penalty, int* history, const int* history_spans,
                    const int* append_at, const float* uniforms);
void xrt_ref_random_normal(float* out, long count, unsigned long long key, float scale, float offset);
void xrt_ref_pack_weight(const float* w, float* packed, int rows, int K, int kind, int gated_n, int head_dim, int rotated_heads);

#ifdef __cplusplus
}
#endif
