// Entry point of all matrix products: checks the operands and picks the kernel.
#include "packing.h"
#include "gemm_skinny.h"
#include "activation.h"

int xrt_linear_plain(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
                     int mode, int activation, hipStream_t s);
bool xrt_linear_mfma_accepts(const void* a, const void* w, int M, int N, int K, int mode);
int xrt_linear_mfma(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                    const Packing& packing, hipStream_t s);

bool xrt_linear_split_takes(const void* a, const void* w, int M, int N, int K, int mode, long* workspace_floats);
bool xrt_linear_split_takes_norm(const void* a, const void* w, int M, int N, int K, int mode);
bool xrt_linear_split_takes_whole_norm(const void* a, const void* w, int M, int N, int K, int mode, long* workspace_floats);
bool xrt_linear_split_takes_qkv(const void* a, const void* w, int M, int N, int K, const QkvAfter& after, long* workspace_floats);
int xrt_linear_split_qkv(const void* a, const void* w, void* qkv, int M, int N, int K, const Packing& packing, float* workspace,
                         const xrt_linear_norm* norm, const QkvAfter& after, hipStream_t s);
int xrt_linear_split(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                     const Packing& packing, float* workspace, const xrt_linear_norm* norm, hipStream_t s);

bool xrt_linear_packed_accepts(const void* a, const void* w, int M, int K, int mode, const Packing* packing);
bool xrt_linear_packed_takes_norm(int M);
bool xrt_linear_packed_takes_qkv(int M, int N, const Packing& packing, const QkvAfter& after);
int xrt_linear_packed(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                      const Packing* packing, const xrt_linear_norm* norm, const QkvAfter* after, hipStream_t s);

static const Packing ROWS_ALONG_K = {XRT_PACK_NONE, 0, 0, 0};
static const Packing& packing_of(const xrt_packing* packing) { return packing ? *packing : ROWS_ALONG_K; }

// A packed w must fit its product: bfloat16, K in whole tiles, gate/up pairs for exactly the gated product.
static int check_packing(const xrt_packing* packing, int dtype, int N, int K, int mode) {
    if (!packing || packing->kind == XRT_PACK_NONE) return 0;
    XRT_REQUIRE(packing->kind == XRT_PACK_TILES || packing->kind == XRT_PACK_GATED || packing->kind == XRT_PACK_ROTARY,
                "linear: unknown packing %d", packing->kind);
    XRT_REQUIRE(dtype == XRT_BF16 && K % 32 == 0, "linear: a packed w is bfloat16 with K a multiple of 32 (dtype %d, K=%d)", dtype, K);
    XRT_REQUIRE((mode == 2) == (packing->kind == XRT_PACK_GATED), "linear: gate/up pairs are packed for the gated product and nothing else");
    XRT_REQUIRE(packing->kind != XRT_PACK_GATED || packing->gated_n == N, "linear: w was packed for %d gated outputs, not %d", packing->gated_n, N);
    XRT_REQUIRE(packing->kind != XRT_PACK_ROTARY || (packing->head_dim > 0 && N % packing->head_dim == 0),
                "linear: w was packed for heads of %d, which do not divide %d rows", packing->head_dim, N);
    return 0;
}

extern "C" long xrt_linear_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode) {
    long need = 0;
    if (dtype != XRT_BF16 || M <= 0 || N <= 0 || K <= 0 || mode < 0 || mode > 2) return 0;
    xrt_linear_split_takes(a, w, M, N, K, mode, &need);
    return need;
}

extern "C" int xrt_linear(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N,
                          int K, int mode, float* workspace, long workspace_floats, void* stream) {
    return xrt_linear_with(a, w, nullptr, dtype, out, out_dtype, M, N, K, mode, workspace, workspace_floats, stream);
}

extern "C" int xrt_linear_with(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype,
                               int M, int N, int K, int mode, float* workspace, long workspace_floats, void* stream) {
    // a gated product carries its activation's code above the mode's low byte
    const int activation = mode >= 0 ? activation_of(mode) : 0;
    XRT_REQUIRE(activation >= 0 && activation < XRT_ACT_COUNT && (activation == 0 || mode_of(mode) == 2),
                "linear: unknown activation %d in mode %d", activation, mode);
    if (mode >= 0) mode = mode_of(mode);
    XRT_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
    XRT_REQUIRE(mode >= 0 && mode <= 2, "linear: unknown mode %d", mode);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "linear: unknown dtype %d", dtype);
    XRT_REQUIRE(out_dtype == XRT_F32 || out_dtype == XRT_BF16, "linear: unknown output dtype %d", out_dtype);
    XRT_REQUIRE(!(dtype == XRT_F32 && out_dtype == XRT_BF16), "linear: float32 operands need a float32 output");
    XRT_REQUIRE(mode != 1 || out_dtype == XRT_F32, "linear: accumulation needs a float32 output");
    XRT_REQUIRE(a && w && out, "linear: null operand");
    if (check_packing(packing, dtype, N, K, mode) != 0) return 1;
    const Packing& layout = packing_of(packing);
    if (M == 0) return 0;
    // The matrix-core kernels address their operands with 32-bit offsets. A step of so many tokens that x
    // exceeds them (a batch of long prompts) goes in runs of rows; an output element's sum is the same.
    if (dtype == XRT_BF16 && (long)M * K >= (1L << 31) && K <= (1 << 22)) {
        const int run = (int)(((1L << 31) - 1) / K / 256 * 256);
        const long out_row = (long)N * (out_dtype == XRT_F32 ? 4 : 2);
        for (int m0 = 0; m0 < M; m0 += run) {
            const int status = xrt_linear_with((const char*)a + (long)m0 * K * 2, w, packing, dtype, (char*)out + m0 * out_row, out_dtype,
                                               M - m0 < run ? M - m0 : run, N, K, mode | (activation << 8), workspace, workspace_floats, stream);
            if (status != 0) return status;
        }
        return 0;
    }
    // bfloat16: the matrix-core kernels; float32, and shapes they refuse: the plain kernel
    if (dtype == XRT_BF16) {
        long need = 0;
        if (xrt_linear_split_takes(a, w, M, N, K, mode, &need) && (need == 0 || (workspace != nullptr && workspace_floats >= need)))
            return xrt_linear_split(a, w, out, out_dtype, M, N, K, mode, activation, layout, workspace, nullptr, (hipStream_t)stream);
    }
    if (xrt_linear_packed_accepts(a, w, M, K, mode, packing))
        return xrt_linear_packed(a, w, out, out_dtype, M, N, K, mode, activation, packing, nullptr, nullptr, (hipStream_t)stream);
    if (dtype == XRT_BF16 && !is_packed(layout) && xrt_linear_skinny_accepts(a, w, M, K))
        return xrt_linear_skinny(a, w, out, out_dtype, M, N, K, mode, activation, nullptr, nullptr, (hipStream_t)stream);
    if (dtype == XRT_BF16 && xrt_linear_mfma_accepts(a, w, M, N, K, mode))
        return xrt_linear_mfma(a, w, out, out_dtype, M, N, K, mode, activation, layout, (hipStream_t)stream);
    XRT_REQUIRE(!is_packed(layout), "linear: M=%d N=%d K=%d is beyond what the kernels for a packed w take", M, N, K);
    return xrt_linear_plain(a, w, dtype, out, out_dtype, M, N, K, mode, activation, (hipStream_t)stream);
}

extern "C" int xrt_linear_takes_norm(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K, int mode) {
    if (dtype != XRT_BF16 || M < 1 || N <= 0 || K <= 0 || mode < 0 || mode > 2) return 0;
    if (packing && is_packed(*packing)) {
        if (xrt_linear_packed_accepts(a, w, M, K, mode, packing) && xrt_linear_packed_takes_norm(M))
            return mode != 1 || (packing->kind == XRT_PACK_TILES && N % 16 == 0);      // an accumulating product writes per tile of 16 columns
    } else if (xrt_linear_skinny_accepts(a, w, M, K) && xrt_linear_skinny_takes_norm(M)) {
        return 1;
    }
    if (xrt_linear_split_takes_norm(a, w, M, N, K, mode)) return 1;
    long unused = 0;
    return xrt_linear_split_takes_whole_norm(a, w, M, N, K, mode, &unused) ? 2 : 0;
}

// Floats of workspace for xrt_linear_normed where xrt_linear_takes_norm says 2 (the product's second kernel does the whole norm).
extern "C" long xrt_linear_whole_norm_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode) {
    long need = 0;
    if (dtype == XRT_BF16) xrt_linear_split_takes_whole_norm(a, w, M, N, K, mode, &need);
    return need;
}

// Tiles of columns for which an accumulating product that xrt_linear_takes_norm accepts writes sums of
// squares: the rows of the table that the caller provides (and hands to the product after the norm).
extern "C" int xrt_linear_norm_tiles(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K) {
    const bool packed = packing && is_packed(*packing);
    if (dtype == XRT_BF16 && !packed && xrt_linear_skinny_accepts(a, w, M, K) && xrt_linear_skinny_takes_norm(M))
        return xrt_linear_skinny_norm_tiles(N);
    return (N + 15) / 16;
}

extern "C" int xrt_linear_normed(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype,
                                 int M, int N, int K, int mode, const xrt_linear_norm* norm, float* workspace,
                                 long workspace_floats, void* stream) {
    XRT_REQUIRE(a && w && out && norm, "linear with norm: null operand");
    const int activation = mode >= 0 ? activation_of(mode) : 0;
    XRT_REQUIRE(activation >= 0 && activation < XRT_ACT_COUNT && (activation == 0 || mode_of(mode) == 2),
                "linear with norm: unknown activation %d in mode %d", activation, mode);
    if (mode >= 0) mode = mode_of(mode);
    if (check_packing(packing, dtype, N, K, mode) != 0) return 1;
    const Packing& layout = packing_of(packing);
    XRT_REQUIRE(dtype == XRT_BF16 && M >= 1 && N > 0 && K > 0 && mode >= 0 && mode <= 2,
                "linear with norm: M=%d N=%d K=%d mode %d of dtype %d is not a product that takes it", M, N, K, mode, dtype);
    XRT_REQUIRE(out_dtype == XRT_F32 || out_dtype == XRT_BF16, "linear with norm: unknown output dtype %d", out_dtype);
    XRT_REQUIRE(mode != 1 || out_dtype == XRT_F32, "linear with norm: accumulation needs a float32 output");
    if (norm->squares_in)
        XRT_REQUIRE(norm->width_in == K && norm->tiles_in >= (K + 15) / 16 && norm->tiles_in <= (K + 7) / 8,     // tiles of 8 to 16 columns
                    "linear with norm: sums of squares of %d tiles over %d columns for a of %d columns",
                    norm->tiles_in, norm->width_in, K);
    const bool whole_norm = norm->scaled_out && norm->gain && !norm->squares_out && !norm->squares_in;
    if (whole_norm) {
        // many rows: the product's second kernel adds the parts, and writes the rows' RMSNorm (gain, eps) to scaled_out
        long need = 0;
        XRT_REQUIRE(norm->gain_dtype == XRT_F32 || norm->gain_dtype == XRT_BF16, "linear with norm: unknown gain dtype %d", norm->gain_dtype);
        XRT_REQUIRE(xrt_linear_split_takes_whole_norm(a, w, M, N, K, mode, &need) && out_dtype == XRT_F32,
                    "linear with norm: M=%d N=%d K=%d mode %d is not a product that does the whole norm after it", M, N, K, mode);
        XRT_REQUIRE(workspace != nullptr && workspace_floats >= need, "linear with norm: the workspace needs %ld floats", need);
        return xrt_linear_split(a, w, out, out_dtype, M, N, K, mode, activation, layout, workspace, norm, (hipStream_t)stream);
    }
    const bool emits = norm->squares_out || norm->scaled_out || norm->gain;
    if (emits) {
        XRT_REQUIRE(mode == 1, "linear with norm: only an accumulating product writes what the norm after it needs");
        XRT_REQUIRE(norm->squares_out && norm->scaled_out && norm->gain, "linear with norm: scaled_out, gain and squares_out come together");
        XRT_REQUIRE(norm->gain_dtype == XRT_F32 || norm->gain_dtype == XRT_BF16, "linear with norm: unknown gain dtype %d", norm->gain_dtype);
        XRT_REQUIRE(xrt_linear_takes_norm(a, w, packing, dtype, M, N, K, mode), "linear with norm: M=%d N=%d K=%d cannot write what the norm after it needs", M, N, K);
    }
    if (is_packed(layout) && xrt_linear_packed_accepts(a, w, M, K, mode, packing) && xrt_linear_packed_takes_norm(M)) {
        XRT_REQUIRE(mode != 1 || layout.kind == XRT_PACK_TILES, "linear with norm: an accumulating product takes a w packed in plain tiles");
        return xrt_linear_packed(a, w, out, out_dtype, M, N, K, mode, activation, packing, norm, nullptr, (hipStream_t)stream);
    }
    if (!is_packed(layout) && xrt_linear_skinny_accepts(a, w, M, K) && xrt_linear_skinny_takes_norm(M))
        return xrt_linear_skinny(a, w, out, out_dtype, M, N, K, mode, activation, norm, nullptr, (hipStream_t)stream);
    long need = 0;
    XRT_REQUIRE(M <= 64 && xrt_linear_split_takes(a, w, M, N, K, mode, &need),
                "linear with norm: M=%d N=%d K=%d is not a product that takes it", M, N, K);
    XRT_REQUIRE(need == 0 || (workspace != nullptr && workspace_floats >= need), "linear with norm: the workspace needs %ld floats", need);
    return xrt_linear_split(a, w, out, out_dtype, M, N, K, mode, activation, layout, workspace, norm, (hipStream_t)stream);
}

extern "C" int xrt_linear_qkv(const void* a, const void* w, const xrt_packing* packing, int dtype, void* qkv, int M, int K,
                              const xrt_linear_norm* norm, int n_heads, int n_kv_heads, int head_dim,
                              const int* positions, const int* slots, const void* q_norm, const void* k_norm,
                              int norm_dtype, float norm_eps, const float* rope_theta, int rope_dim,
                              float rope_scale, void* k_cache, void* v_cache, const int* block_table,
                              int table_stride, int n_blocks, int longest_run, float* workspace,
                              long workspace_floats, void* stream) {
    XRT_REQUIRE(n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "linear_qkv: bad head sizes %d/%d x %d", n_heads, n_kv_heads, head_dim);
    const int N = (n_heads + 2 * n_kv_heads) * head_dim;
    if (check_packing(packing, dtype, N, K, 0) != 0) return 1;
    const Packing& layout = packing_of(packing);
    if (M == 0) return 0;
    // a decode step without head norms: one kernel does the product, the rotation and the cache write
    QkvAfter after = {positions, slots, rope_theta, rope_dim, rope_scale, n_heads, n_kv_heads, head_dim,
                      (bf16*)k_cache, (bf16*)v_cache, block_table, table_stride, n_blocks};
    const bool one_kernel = dtype == XRT_BF16 && a && w && qkv && M > 0 && K > 0 && !q_norm && !k_norm && positions &&
        (uintptr_t)qkv % 8 == 0 && (uintptr_t)k_cache % 8 == 0 && (k_cache == nullptr) == (v_cache == nullptr) &&
        (k_cache == nullptr || (block_table && slots && table_stride > 0 && n_blocks > 0)) &&
        (rope_theta == nullptr || rope_dim > 0);
    if (one_kernel && is_packed(layout) && xrt_linear_packed_accepts(a, w, M, K, 0, packing) && xrt_linear_packed_takes_qkv(M, N, layout, after))
        return xrt_linear_packed(a, w, qkv, XRT_BF16, M, N, K, 0, XRT_ACT_SILU, packing, norm, &after, (hipStream_t)stream);
    if (one_kernel && !is_packed(layout) && xrt_linear_skinny_accepts(a, w, M, K) && xrt_linear_skinny_takes_qkv(M, N, after))
        return xrt_linear_skinny(a, w, qkv, XRT_BF16, M, N, K, 0, XRT_ACT_SILU, norm, &after, (hipStream_t)stream);
    // 17 to 64 tokens, the product split along k: the kernel that adds the partial sums does the rest
    long need = 0;
    if (dtype == XRT_BF16 && a && w && qkv && M > 0 && K > 0 && !q_norm && !k_norm && positions &&
        (k_cache == nullptr) == (v_cache == nullptr) &&
        (k_cache == nullptr || (block_table && slots && table_stride > 0 && n_blocks > 0)) &&
        (!norm || (norm->squares_in && !norm->squares_out && xrt_linear_split_takes_norm(a, w, M, N, K, 0))) &&
        xrt_linear_split_takes_qkv(a, w, M, N, K, after, &need) && workspace != nullptr && workspace_floats >= need)
        return xrt_linear_split_qkv(a, w, qkv, M, N, K, layout, workspace, norm, after, (hipStream_t)stream);
    const int status = norm ? xrt_linear_normed(a, w, packing, dtype, qkv, dtype, M, N, K, 0, norm, workspace, workspace_floats, stream)
                            : xrt_linear_with(a, w, packing, dtype, qkv, dtype, M, N, K, 0, workspace, workspace_floats, stream);
    if (status != 0) return status;
    return xrt_qkv_prepare(qkv, dtype, M, n_heads, n_kv_heads, head_dim, positions, slots, q_norm, k_norm, norm_dtype,
                           norm_eps, rope_theta, rope_dim, rope_scale, k_cache, v_cache, block_table, table_stride,
                           n_blocks, longest_run, stream);
}
