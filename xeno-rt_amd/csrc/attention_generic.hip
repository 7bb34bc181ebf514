// Causal attention of every token of a step over its own sequence's cache, float32 math,
// for any element type, head size (up to 512), head grouping and window.
// It is the attention of the 32-bit path and the fallback of the bfloat16 path.
//
// Reference: crates/xrt-models/src/llama.rs:504-574 (online softmax: running maximum m and
// sum l, rescaled by exp(m_old - m_new)) and :727-770 (a token at position P sees keys
// 0..P; query head h reads key/value head h / group; score = (q.k) * scale).
//
// One wavefront per (token, head). Keys are visited block by block (64 keys, lane j takes
// key j) in the order of their positions, whatever the step looks like, so the result of a
// token does not depend on how its request was cut into steps or batched.
//
// A position encoding that acts on the scores instead of on q and k is served here too: with
// distance_slopes (one float per query head) a key at position j adds slope * (j - P) to the
// score of the query at position P, after the scale. Not in the reference's model.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

constexpr int MAX_HEAD_DIM = 512;
constexpr int MAX_OWNED = MAX_HEAD_DIM / XRT_WAVE;

// eight elements from p (aligned to eight elements: a piece of a cache block), as floats, in one or two loads
template <typename T>
__device__ __forceinline__ void load_piece(const T* __restrict__ p, float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        struct alignas(16) Eight { T e[8]; };
        const Eight q = *reinterpret_cast<const Eight*>(p);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = to_float(q.e[e]);
    }
}

template <typename T>
__global__ void __launch_bounds__(XRT_WAVE) attention_generic_kernel(
    const T* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads, int head_dim,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ positions, const int* __restrict__ slots,
    T* __restrict__ out, float scale, int window, const float* __restrict__ distance_slopes) {
    __shared__ float qs[MAX_HEAD_DIM];
    __shared__ float ps[XRT_WAVE];
    const int lane = threadIdx.x;
    const int token = blockIdx.x / n_heads, head = blockIdx.x % n_heads;
    const int kv_head = head / (n_heads / n_kv_heads);
    T* dst = out + ((long)token * n_heads + head) * head_dim;
    const int slot = slots[token];
    if (slot < 0) {
        for (int e = lane; e < head_dim; e += XRT_WAVE) dst[e] = from_float<T>(0.f);
        return;
    }
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const float slope = distance_slopes ? distance_slopes[head] : 0.f;
    // pieces of eight elements can be loaded whole if they are aligned: head sizes that are multiples of 8, caches aligned to 32 bytes
    const bool whole_pieces = head_dim % 8 == 0 && (uintptr_t)k_cache % 32 == 0 && (uintptr_t)v_cache % 32 == 0;
    const T* q = qkv + (long)token * row_width + (long)head * head_dim;
    for (int e = lane; e < head_dim; e += XRT_WAVE) qs[e] = to_float(q[e]);
    wave_sync();

    float m = -INFINITY, l = 0.f, acc[MAX_OWNED];
#pragma unroll
    for (int i = 0; i < MAX_OWNED; ++i) acc[i] = 0.f;

    for (int b = first / XRT_BLOCK_TOKENS; b <= pos / XRT_BLOCK_TOKENS; ++b) {
        const int block = block_table[(long)slot * table_stride + b];
        if (block < 0 || block >= n_blocks) continue;          // the host never lets this happen
        const int j = b * XRT_BLOCK_TOKENS + lane;
        const bool valid = j >= first && j <= pos;
        const long head_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
        float s = -INFINITY;
        if (valid) {
            // the key's dims in order, piece by piece of the cache's order: a piece's products are added up, then
            // the pieces' sums (less rounding than one running sum)
            float dot = 0.f;
            if (whole_pieces) {
#pragma unroll 4
                for (int d0 = 0; d0 < head_dim; d0 += 8) {
                    float key[8], of_piece = 0.f;
                    load_piece(k_cache + head_base + cache_key_offset(lane, d0, head_dim), key);
#pragma unroll
                    for (int e = 0; e < 8; ++e) of_piece = fmaf(qs[d0 + e], key[e], of_piece);
                    dot += of_piece;
                }
            } else {
                for (int d0 = 0; d0 < head_dim; d0 += 8) {
                    const T* piece = k_cache + head_base + cache_key_offset(lane, d0, head_dim);
                    const int dims = min(8, head_dim - d0);
                    float of_piece = 0.f;
                    for (int e = 0; e < dims; ++e) of_piece = fmaf(qs[d0 + e], to_float(piece[e]), of_piece);
                    dot += of_piece;
                }
            }
            s = dot * scale;
            if (distance_slopes) s += slope * (float)(j - pos);
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float correction = expf(m - m_new);              // 0 for the first block (m = -inf)
        l = l * correction + wave_sum(p);
        m = m_new;
        ps[lane] = p;
        wave_sync();
        const int j_begin = max(0, first - b * XRT_BLOCK_TOKENS);
        const int j_end = min(XRT_BLOCK_TOKENS - 1, pos - b * XRT_BLOCK_TOKENS);
#pragma unroll
        for (int i = 0; i < MAX_OWNED; ++i) {
            const int d = lane + i * XRT_WAVE;
            if (d < head_dim) {
                float sum = 0.f;
#pragma unroll 4
                for (int j0 = j_begin / 8 * 8; j0 <= j_end; j0 += 8) {   // the dim's values in the order of their tokens
                    const T* piece = v_cache + head_base + cache_value_offset(d, j0, head_dim);
                    if (whole_pieces) {
                        float value[8];                         // (what lies beyond the sequence's end is loaded and not used)
                        load_piece(piece, value);
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (j0 + e >= j_begin && j0 + e <= j_end) sum = fmaf(ps[j0 + e], value[e], sum);
                    } else {
                        for (int jj = max(j0, j_begin); jj <= min(j0 + 7, j_end); ++jj) sum = fmaf(ps[jj], to_float(piece[jj - j0]), sum);
                    }
                }
                acc[i] = acc[i] * correction + sum;
            }
        }
        wave_sync();
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;                // llama.rs:566-571
#pragma unroll
    for (int i = 0; i < MAX_OWNED; ++i) {
        const int d = lane + i * XRT_WAVE;
        if (d < head_dim) dst[d] = from_float<T>(acc[i] * inv);
    }
}

}  // namespace

int xrt_attention_generic(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                          const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                          int n_blocks, const int* positions, const int* slots, void* out, float scale,
                          int window, const float* distance_slopes, hipStream_t s) {
    XRT_REQUIRE(head_dim <= MAX_HEAD_DIM, "attention: head_dim %d exceeds %d", head_dim, MAX_HEAD_DIM);
    const long items = (long)tokens * n_heads;
    XRT_REQUIRE(items < (1L << 31), "attention: too many (token, head) pairs");
    const int row_width = (n_heads + 2 * n_kv_heads) * head_dim;
    if (dtype == XRT_F32)
        attention_generic_kernel<float><<<(unsigned)items, XRT_WAVE, 0, s>>>(
            (const float*)qkv, row_width, n_heads, n_kv_heads, head_dim, (const float*)k_cache,
            (const float*)v_cache, block_table, table_stride, n_blocks, positions, slots, (float*)out, scale, window, distance_slopes);
    else
        attention_generic_kernel<bf16><<<(unsigned)items, XRT_WAVE, 0, s>>>(
            (const bf16*)qkv, row_width, n_heads, n_kv_heads, head_dim, (const bf16*)k_cache,
            (const bf16*)v_cache, block_table, table_stride, n_blocks, positions, slots, (bf16*)out, scale, window, distance_slopes);
    XRT_LAUNCH_CHECK("attention (generic)");
    return 0;
}
