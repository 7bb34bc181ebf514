// Entry point of attention: checks the operands and picks the kernel.
#include "common.h"
#include "xrt_hip.h"

int xrt_attention_generic(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                          const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                          int n_blocks, const int* positions, const int* slots, void* out, float scale,
                          int window, hipStream_t s);

extern "C" int xrt_attention(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                             const void* k_cache, const void* v_cache, const int* block_table,
                             int table_stride, int n_blocks, const int* positions, const int* slots, void* out,
                             float scale, int window, void* stream) {
    XRT_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention: head counts %d/%d: the first must be a multiple of the second", n_heads, n_kv_heads);
    XRT_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "attention: head_dim %d must be a multiple of 16", head_dim);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "attention: unknown dtype %d", dtype);
    XRT_REQUIRE(qkv && k_cache && v_cache && block_table && positions && slots && out, "attention: null operand");
    XRT_REQUIRE(table_stride > 0 && n_blocks > 0, "attention: empty cache");
    XRT_REQUIRE(window >= 0, "attention: negative window");
    if (tokens == 0) return 0;
    return xrt_attention_generic(qkv, dtype, tokens, n_heads, n_kv_heads, head_dim, k_cache, v_cache, block_table,
                                 table_stride, n_blocks, positions, slots, out, scale, window, (hipStream_t)stream);
}
