// C interface of the kernel library. Every function returns 0 on success; otherwise
// xrt_last_error() describes what was refused. Pointers are device pointers unless
// said otherwise; `stream` is a hipStream_t. Element type codes: 0 = float32, 1 = bfloat16.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

const char* xrt_last_error(void);

// tokens in one block of the cache. A cache is [blocks][kv_heads][xrt_block_tokens() * head_dim elements], keys and
// values apart. Whoever keeps the block tables must count in the same blocks.
int xrt_block_tokens(void);
// Where the elements lie inside the part of a block that belongs to one key/value head: the element offset of dim
// `dim` of the key (of the value) of the block's token `token`. Heads whose size is a multiple of 32 lie in the order
// in which the matrix cores take them in a decode step (csrc/cache_layout.h); others as keys [token][dim], values
// [dim][token]. Host functions, for whoever wants to fill or read a cache outside the kernels.
int xrt_cache_key_offset(int token, int dim, int head_dim);
int xrt_cache_value_offset(int dim, int token, int head_dim);

// How a bfloat16 weight matrix w[rows][K] is laid out. XRT_PACK_NONE (or a null pointer wherever a packing
// is passed): rows contiguous along k. Otherwise tiles of 16 rows x 32 columns in the order in which the matrix
// cores take them, rows padded to a multiple of 16 with zeros, K a multiple of 32; the rows may also be
// regrouped so that outputs which an epilogue combines share a tile (csrc/packing.h says how):
// XRT_PACK_GATED for [gate rows | up rows] (gated_n outputs, a multiple of 8), XRT_PACK_ROTARY for rows
// [heads][head_dim] whose first rotated_heads heads are rotated over the whole head.
// Products that are bound by reading w (few rows of a) stream a packed w faster; all others take either form.
enum { XRT_PACK_NONE = 0, XRT_PACK_TILES = 1, XRT_PACK_GATED = 2, XRT_PACK_ROTARY = 3 };
typedef struct xrt_packing { int kind; int gated_n; int head_dim; int rotated_heads; } xrt_packing;
// packed[...] = w in the layout `packing` (rows padded to a multiple of 16: the packed matrix has
// (rows + 15) / 16 * 16 * K elements); XRT_PACK_GATED needs rows = 2 * gated_n, XRT_PACK_ROTARY rows a
// multiple of head_dim
int xrt_pack_weight(const void* w, void* packed, int rows, int K, const xrt_packing* packing, void* stream);
// whether packing pays for a matrix of these sizes (its tiles divide evenly among the compute units)
int xrt_packing_suits(int rows, int K);

// out[t, :] = table[ids[t], :] as float32
int xrt_embed(const void* table, int table_dtype, const xrt_packing* packing, const int* ids, float* out, int tokens,
              int hidden, int vocab, void* stream);

// out[i] = element i of the random-weights stream `key`: float(2 * (sum of twelve 10-bit fields of two
// splitmix64 words) - 12 * 1023) * scale + offset, the same values as the host-side generator gives
int xrt_random_normal(void* out, int dtype, long count, unsigned long long key, float scale, float offset,
                      void* stream);

// Probes for the benchmark's measured ceilings; nothing of the model runs through them.
// xrt_probe_read reads xrt_probe_read_bytes(bytes) bytes of `buffer` once (plain or non-temporal loads) and
// writes nothing (sink: 4 bytes that stay as they are). xrt_probe_mfma runs `iterations` rounds of four
// 32x32x16 bfloat16 matrix-core products per wavefront on tiles held in registers, in XRT_PROBE_MFMA_GROUPS
// workgroups of four wavefronts: XRT_PROBE_MFMA_GROUPS * 4 * iterations * 4 * 2 * 32 * 32 * 16 flops. Its operands
// are small whole numbers, or with random_operands numbers of either sign with random mantissas, on which
// the chip holds a lower clock.
#define XRT_PROBE_MFMA_GROUPS 512
int xrt_probe_read(const void* buffer, long bytes, int nontemporal, void* sink, void* stream);
long xrt_probe_read_bytes(long bytes);
int xrt_probe_mfma(long iterations, int random_operands, void* sink, void* stream);

// residual[i] += delta[i]
int xrt_add(float* residual, const void* delta, int delta_dtype, long count, void* stream);

// out[r, :] = rmsnorm(x[rows ? rows[r] : r, :]) * weight ; x float32, out of out_dtype
int xrt_rmsnorm(const float* x, const void* weight, int weight_dtype, float eps, void* out, int out_dtype,
                const int* rows, int n_rows, int hidden, void* stream);

// out[m, n] (+)= sum_k a[m, k] * w[n, k]   (mode 0 store, 1 accumulate into float32 out,
// 2 gated: out[m, n] = act(a.w[n]) * (a.w[n + N]) with w of 2N rows; the activation's code rides above the
// mode's low byte, XRT_GATED(XRT_ACT_SILU) == 2: silu(z) = z / (1 + exp(-z)) is the one that exists)
#define XRT_ACT_SILU 0
#define XRT_GATED(activation) (2 | ((activation) << 8))
// Some products (17 to 64 rows of a, or more rows and a narrow w) run faster split along k, through a workspace of float32
// sums: xrt_linear_workspace says how many floats that takes (0: none); without it the product
// takes another kernel.
int xrt_linear(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
               int mode, float* workspace, long workspace_floats, void* stream);
long xrt_linear_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode);
// the same with w in the layout `packing` (null: rows contiguous along k)
int xrt_linear_with(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype, int M, int N,
                    int K, int mode, float* workspace, long workspace_floats, void* stream);

// xrt_linear for callers that cannot allocate device memory: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The partial sums of a
// product split along k go to a fixed array of XRT_LINEAR_STATIC_FLOATS floats (16 MiB) that the library
// holds in device memory on every GPU it is used on; the call allocates nothing and refuses a product
// whose partial sums do not fit (xrt_linear_workspace says how many floats a product needs). Calls on one
// GPU share that array: calls that overlap there (different streams) race.
#define XRT_LINEAR_STATIC_FLOATS (4L << 20)
long xrt_linear_static_floats(void);       // XRT_LINEAR_STATIC_FLOATS, for callers that do not read this header
int xrt_linear_static(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
                      int mode, void* stream);

// An RMSNorm between two products, x += a w^T; y = rmsnorm(x) * gain; z = y v^T, without a kernel of
// its own. The first product (mode 1) also writes scaled_out[m, n] = bfloat16(x[m, n] * gain[n]) and
// squares_out[t * XRT_SQUARES_STRIDE + m], the sum of x[m, n]^2 over the columns n of tile t (xrt_linear_norm_tiles of them, 16 columns or fewer each). The
// second takes scaled_out as its a, squares_in (tiles_in = ceil(width_in / 16) tiles) and multiplies its
// rows by 1 / sqrt(sum of squares / width_in + eps) before its epilogue. A half left all zero is not done.
// xrt_linear_takes_norm says whether an accumulating product can write these (bfloat16 operands, up to 64 rows,
// and with more than 16 rows: split along k, N a multiple of 64); then the product after it (same rows) can
// take them, and xrt_linear_normed refuses what cannot. workspace: as for xrt_linear.
// xrt_linear_takes_norm returns 2 for an accumulating product of many rows that runs as large tiles splitting k: its second
// kernel then does the whole norm. For that, scaled_out, gain, gain_dtype and eps are set and the other fields left zero:
// scaled_out[m, n] = bfloat16((x[m, n] / rms(x[m, :])) * gain[n]), the norm kernel's result to the bit, which the product after
// it takes like any rows. Its workspace has xrt_linear_whole_norm_workspace(...) floats.
#define XRT_SQUARES_STRIDE 64
typedef struct xrt_linear_norm {
    const float* squares_in; int tiles_in; int width_in; float eps;
    void* scaled_out; const void* gain; int gain_dtype; float* squares_out;
} xrt_linear_norm;
int xrt_linear_takes_norm(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K, int mode);
int xrt_linear_norm_tiles(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K);   // rows of the table at squares_out
long xrt_linear_whole_norm_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode);
int xrt_linear_normed(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype, int M, int N,
                      int K, int mode, const xrt_linear_norm* norm, float* workspace, long workspace_floats, void* stream);

// per-head RMSNorm of q and k (optional), rotation of q and k (optional), write of k and v
// into the cache (optional); qkv rows are [q heads | k heads | v heads]. longest_run: the most
// consecutive tokens that one sequence brings (0 if unknown); it only picks the faster way to
// write the values
int xrt_qkv_prepare(void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                    const int* positions, const int* slots,
                    const void* q_norm, const void* k_norm, int norm_dtype, float norm_eps,
                    const float* rope_theta, int rope_dim, float rope_scale,
                    void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks,
                    int longest_run, void* stream);

// The q/k/v projection qkv = a w^T followed by xrt_qkv_prepare (same arguments), in one kernel where a
// decode step allows it (bfloat16, at most 16 rows, no head norms), else in two. norm: null, or the
// squares_in half of an RMSNorm before the projection (then a is what xrt_linear_normed would take).
// workspace as for xrt_linear.
int xrt_linear_qkv(const void* a, const void* w, const xrt_packing* packing, int dtype, void* qkv, int M, int K, const xrt_linear_norm* norm,
                   int n_heads, int n_kv_heads, int head_dim, const int* positions, const int* slots,
                   const void* q_norm, const void* k_norm, int norm_dtype, float norm_eps,
                   const float* rope_theta, int rope_dim, float rope_scale,
                   void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks,
                   int longest_run, float* workspace, long workspace_floats, void* stream);

// causal attention of every token of a step over its sequence's cache. The sequences of the
// step may be described (seq_* arrays, n_seqs, the largest token count of a sequence and the
// longest sequence after the step): then the matrix-core kernels can be used; a decode step (max_count 1)
// then needs a workspace of xrt_attention_workspace(...) floats for the partial results of the parts that
// its keys are cut into (0: none), and takes the general kernel without it. distance_slopes (null: none): one
// float per query head; a key at position j then adds slope * (j - P) to the scaled score of the query at
// position P, for position encodings that act on the scores (the general kernel serves them).
long xrt_attention_workspace(int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim, int window,
                             int max_count, int max_context);
// A decode step (every sequence brings one token) of bfloat16 heads of 64 or 128 dims can leave to the attention what
// xrt_qkv_prepare would do between the projection and it: qkv then holds the projection as it came, and the attention
// kernel norms the heads of q and k (q_norm null: no head norms), rotates them over the whole head (rope_table null: no
// rotation; rope_dim must be head_dim), uses the new key and value and writes them into the cache, which must be
// writable. The cosines and sines of the rotation are read from rope_table, which xrt_rope_table has made and which
// must cover the step's positions (table_positions >= the longest sequence after the step).
// xrt_attention_finishes_qkv says whether a step is one that xrt_attention_finishing takes.
typedef struct xrt_qkv_finish {
    const void* q_norm; const void* k_norm; int norm_dtype; float norm_eps;
    int rope_dim; const float* rope_table; int table_positions;
} xrt_qkv_finish;
// table[p][i] = (cos, sin) of the angle p * rope_scale / rope_theta[i] for p < positions, i < rope_dim / 2, float32:
// the values that the kernels which rotate work out for themselves
int xrt_rope_table(const float* rope_theta, int rope_dim, float rope_scale, int positions, float* table, void* stream);
int xrt_attention_finishes_qkv(int dtype, int n_heads, int n_kv_heads, int head_dim, int window, int max_count, int rope_dim,
                               int table_positions, int max_context);
int xrt_attention_finishing(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                            void* k_cache, void* v_cache, const int* block_table, int table_stride,
                            int n_blocks, const int* positions, const int* slots, void* out, float scale,
                            const xrt_qkv_finish* finish, int max_context, float* workspace, long workspace_floats, void* stream);
int xrt_attention(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                  const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                  int n_blocks, const int* positions, const int* slots, void* out, float scale, int window,
                  const float* distance_slopes, const int* seq_offsets, const int* seq_slots, const int* seq_starts, int n_seqs,
                  int max_count, int max_context, float* workspace, long workspace_floats, void* stream);

// one token per row of float32 logits. With a workspace of xrt_sample_workspace(rows, vocab) bytes (0: this
// vocabulary gains nothing from it) rows with a top-k of 1 to 64 are sampled from candidates that
// workgroups find slice by slice, instead of in eight passes over the row; without, all rows take the passes.
// The penalty of row r reads history[history_spans[2r] .. history_spans[2r + 1]); with append_at (may be
// null) the row's token is also written to history[append_at[r]] (nowhere if that is negative), so that a
// caller can keep the sequences' tokens on the device.
int xrt_sample(const float* logits, int rows, int vocab, int* out, const float* temperature,
               const int* top_k, const float* top_p, const float* penalty, int* history,
               const int* history_spans, const int* append_at, const float* uniforms, void* workspace,
               long workspace_bytes, void* stream);
long xrt_sample_workspace(int rows, int vocab);

#ifdef __cplusplus
}
#endif
