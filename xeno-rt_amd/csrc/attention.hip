// Entry point of attention: checks the operands and picks the kernel.
//   bfloat16, head size 64 or 128, no window: the matrix-core kernels: decode (every sequence
//   brings one token) or prefill (any token counts);
//   everything else (float32, any other head size up to 512, windows, scores biased by distance): the general kernel.
#include "common.h"
#include "xrt_hip.h"

int xrt_attention_generic(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                          const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                          int n_blocks, const int* positions, const int* slots, void* out, float scale,
                          int window, const float* distance_slopes, hipStream_t s);
bool xrt_attention_decode_accepts(int head_dim);
long xrt_attention_decode_workspace(int tokens, int n_heads, int n_kv_heads, int head_dim, int max_context);
int xrt_attention_decode(const void* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const void* k_cache,
                         const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                         const int* positions, const int* slots, void* out, float scale, int max_context,
                         float* workspace, long workspace_floats, const xrt_qkv_finish* finish, hipStream_t s);
bool xrt_attention_prefill_accepts(int head_dim);
int xrt_attention_prefill(const void* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const void* k_cache,
                          const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                          const int* seq_offsets, const int* seq_slots, const int* seq_starts, int n_seqs, void* out,
                          float scale, hipStream_t s);

static bool takes_decode_kernel(int dtype, int n_heads, int n_kv_heads, int head_dim, int window, int max_count, int max_context) {
    return dtype == XRT_BF16 && window == 0 && max_count == 1 && max_context > 0 && n_heads > 0 && n_kv_heads > 0 &&
           n_heads % n_kv_heads == 0 && xrt_attention_decode_accepts(head_dim);
}

extern "C" long xrt_attention_workspace(int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim, int window,
                                        int max_count, int max_context) {
    if (tokens <= 0 || !takes_decode_kernel(dtype, n_heads, n_kv_heads, head_dim, window, max_count, max_context)) return 0;
    return xrt_attention_decode_workspace(tokens, n_heads, n_kv_heads, head_dim, max_context);
}

extern "C" int xrt_attention(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                             const void* k_cache, const void* v_cache, const int* block_table,
                             int table_stride, int n_blocks, const int* positions, const int* slots, void* out,
                             float scale, int window, const float* distance_slopes, const int* seq_offsets, const int* seq_slots,
                             const int* seq_starts, int n_seqs, int max_count, int max_context,
                             float* workspace, long workspace_floats, void* stream) {
    XRT_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention: head counts %d/%d: the first must be a multiple of the second", n_heads, n_kv_heads);
    XRT_REQUIRE(head_dim > 0, "attention: head_dim %d must be positive", head_dim);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "attention: unknown dtype %d", dtype);
    XRT_REQUIRE(qkv && k_cache && v_cache && block_table && positions && slots && out, "attention: null operand");
    XRT_REQUIRE(table_stride > 0 && n_blocks > 0, "attention: empty cache");
    XRT_REQUIRE(window >= 0, "attention: negative window");
    if (tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool described = seq_offsets && seq_slots && seq_starts && n_seqs > 0 && max_count > 0 && max_context > 0;
    if (dtype == XRT_BF16 && window == 0 && distance_slopes == nullptr && described) {
        const long need = xrt_attention_workspace(dtype, tokens, n_heads, n_kv_heads, head_dim, window, max_count, max_context);
        if (takes_decode_kernel(dtype, n_heads, n_kv_heads, head_dim, window, max_count, max_context) &&
            (need == 0 || (workspace != nullptr && workspace_floats >= need)))
            return xrt_attention_decode(qkv, tokens, n_heads, n_kv_heads, head_dim, k_cache, v_cache, block_table,
                                        table_stride, n_blocks, positions, slots, out, scale, max_context, workspace,
                                        workspace_floats, nullptr, s);
        if (max_count > 1 && xrt_attention_prefill_accepts(head_dim)) {
            // tokens beyond the sequences (padding) get zeros
            // (their rows are read by nothing, but must not hold what a later product could choke on)
            XRT_REQUIRE(n_seqs <= tokens, "attention: more sequences than tokens");
            return xrt_attention_prefill(qkv, tokens, n_heads, n_kv_heads, head_dim, k_cache, v_cache, block_table,
                                         table_stride, n_blocks, seq_offsets, seq_slots, seq_starts, n_seqs, out,
                                         scale, s);
        }
    }
    return xrt_attention_generic(qkv, dtype, tokens, n_heads, n_kv_heads, head_dim, k_cache, v_cache, block_table,
                                 table_stride, n_blocks, positions, slots, out, scale, window, distance_slopes, s);
}

// ---- a decode step whose attention also finishes q, k and v (xrt_hip.h)

extern "C" int xrt_attention_finishes_qkv(int dtype, int n_heads, int n_kv_heads, int head_dim, int window, int max_count, int rope_dim,
                                          int table_positions, int max_context) {
    return max_context > 0 && takes_decode_kernel(dtype, n_heads, n_kv_heads, head_dim, window, max_count, max_context) &&
           (rope_dim == 0 || (rope_dim == head_dim && table_positions >= max_context));
}

extern "C" int xrt_attention_finishing(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                                       void* k_cache, void* v_cache, const int* block_table, int table_stride,
                                       int n_blocks, const int* positions, const int* slots, void* out, float scale,
                                       const xrt_qkv_finish* finish, int max_context, float* workspace, long workspace_floats, void* stream) {
    XRT_REQUIRE(finish != nullptr, "attention (finishing q/k/v): nothing to finish");
    XRT_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention: head counts %d/%d: the first must be a multiple of the second", n_heads, n_kv_heads);
    XRT_REQUIRE(xrt_attention_finishes_qkv(dtype, n_heads, n_kv_heads, head_dim, 0, 1, finish->rope_table ? finish->rope_dim : 0,
                                           finish->table_positions, max_context),
                "attention (finishing q/k/v): only a bfloat16 decode step with heads of 64 or 128 dims, rotated whole (with a table "
                "of the rotation's turns that covers the step's positions) or not at all");
    XRT_REQUIRE(qkv && k_cache && v_cache && block_table && positions && slots && out, "attention: null operand");
    XRT_REQUIRE(table_stride > 0 && n_blocks > 0, "attention: empty cache");
    if (tokens == 0) return 0;
    const long need = xrt_attention_decode_workspace(tokens, n_heads, n_kv_heads, head_dim, max_context);
    XRT_REQUIRE(need == 0 || (workspace != nullptr && workspace_floats >= need), "attention (finishing q/k/v): the workspace needs %ld floats", need);
    return xrt_attention_decode(qkv, tokens, n_heads, n_kv_heads, head_dim, k_cache, v_cache, block_table, table_stride, n_blocks,
                                positions, slots, out, scale, max_context, workspace, workspace_floats, finish, (hipStream_t)stream);
}
