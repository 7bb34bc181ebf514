// The product for few rows (gemm_skinny.hip), as the entry points of the products see it.
#pragma once
#include "cache_layout.h"
#include "xrt_hip.h"

// What follows the q/k/v projection of a decode step, done by the product's own epilogue: rotation
// of q and k by the token's position and the write of k and v into the cache (no head norms).
struct QkvAfter {
    const int* positions; const int* slots;
    const float* rope_theta; int rope_dim; float rope_scale;      // rope_theta null: no rotation
    int n_heads, n_kv_heads, head_dim;
    bf16* k_cache; bf16* v_cache; const int* block_table; int table_stride, n_blocks;     // k_cache null: no write
    int kv_rows = 16;                                              // rows of a key or value head's tile: set by the kernel's launcher
};

bool xrt_linear_skinny_accepts(const void* a, const void* w, int M, int K);
bool xrt_linear_skinny_takes_norm(int M);
int xrt_linear_skinny_norm_tiles(int N);
bool xrt_linear_skinny_takes_qkv(int M, int N, const QkvAfter& after);
// norm and after may be null; with `after`, out is the bfloat16 q/k/v buffer and mode is 0
// activation: the XRT_ACT_* code of a gated product (mode 2), unused otherwise
int xrt_linear_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                      const xrt_linear_norm* norm, const QkvAfter* after, hipStream_t s);
