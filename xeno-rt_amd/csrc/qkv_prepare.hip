// After the q/k/v projection, in one pass over a token's heads: RMSNorm of every head of
// q and k (one weight [head_dim] each), rotation of q and k by the token's position, and
// the write of k (rotated) and v (raw) into the sequence's cache block.
//
// Reference formulas: head norm crates/xrt-models/src/llama.rs:1025-1040 (val * inv_rms * w);
// rotation crates/xrt-kernels/src/cpu/rope.rs:59-89: angle = pos * scale / theta_i, pairs
// (i, i + rope_dim/2), d[i] = a cos - b sin, d[i + half] = a sin + b cos; elements beyond
// rope_dim stay. Norm, angle, sine, cosine and rotation are float32.
//
// One wavefront per (token, head). A token with a negative slot is padding and is not cached.
#include "common.h"
#include "xrt_hip.h"

namespace {

constexpr int MAX_HEAD_DIM = 512;
constexpr int WAVES = 4;

template <typename T, typename TW>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) qkv_prepare_kernel(
    T* __restrict__ qkv, int items, int n_heads, int n_kv_heads, int head_dim,
    const int* __restrict__ positions, const int* __restrict__ slots,
    const TW* __restrict__ q_norm, const TW* __restrict__ k_norm, float norm_eps,
    const float* __restrict__ rope_theta, int rope_dim, float rope_scale,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks) {
    __shared__ float buffer[WAVES][MAX_HEAD_DIM];
    const int wave = threadIdx.x / XRT_WAVE, lane = threadIdx.x % XRT_WAVE;
    const long item = (long)blockIdx.x * WAVES + wave;
    if (item >= items) return;                      // whole wave leaves together; no block barrier below
    const int heads_total = n_heads + 2 * n_kv_heads;
    const int token = (int)(item / heads_total), head = (int)(item % heads_total);
    const bool is_q = head < n_heads, is_k = !is_q && head < n_heads + n_kv_heads, is_v = !is_q && !is_k;
    T* row = qkv + (long)token * heads_total * head_dim + (long)head * head_dim;
    float* x = buffer[wave];
    const int pos = positions[token];

    long cache_base = -1;                           // element offset of this head's block in the cache
    if ((is_k || is_v) && k_cache != nullptr) {
        const int slot = slots[token];
        if (slot >= 0) {
            const int block = block_table[(long)slot * table_stride + pos / XRT_BLOCK_TOKENS];
            if (block >= 0 && block < n_blocks) {
                const int kv_head = head - n_heads - (is_v ? n_kv_heads : 0);
                cache_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
            }
        }
    }
    const int within = pos % XRT_BLOCK_TOKENS;

    if (is_v) {
        if (cache_base >= 0)
            for (int e = lane; e < head_dim; e += XRT_WAVE)
                v_cache[cache_base + (long)e * XRT_BLOCK_TOKENS + within] = row[e];
        return;
    }

    float sum_sq = 0.f;
    for (int e = lane; e < head_dim; e += XRT_WAVE) {
        const float v = to_float(row[e]);
        x[e] = v;
        sum_sq = fmaf(v, v, sum_sq);
    }
    const TW* norm = is_q ? q_norm : k_norm;
    if (norm != nullptr) {
        sum_sq = wave_sum(sum_sq);
        const float inv_rms = 1.0f / sqrtf(sum_sq / (float)head_dim + norm_eps);
        for (int e = lane; e < head_dim; e += XRT_WAVE) x[e] = x[e] * inv_rms * to_float(norm[e]);
    }
    wave_sync();
    if (rope_theta != nullptr) {
        const int half = rope_dim / 2;
        for (int i = lane; i < half; i += XRT_WAVE) {
            const float angle = (float)pos * rope_scale / rope_theta[i];
            float sine, cosine;
            sincosf(angle, &sine, &cosine);
            const float a = x[i], b = x[i + half];
            x[i] = a * cosine - b * sine;
            x[i + half] = a * sine + b * cosine;
        }
    }
    wave_sync();
    for (int e = lane; e < head_dim; e += XRT_WAVE) {
        const T value = from_float<T>(x[e]);
        row[e] = value;
        if (is_k && cache_base >= 0) k_cache[cache_base + (long)within * head_dim + e] = value;
    }
}

}  // namespace

extern "C" int xrt_qkv_prepare(void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                               const int* positions, const int* slots, const void* q_norm, const void* k_norm,
                               int norm_dtype, float norm_eps, const float* rope_theta, int rope_dim,
                               float rope_scale, void* k_cache, void* v_cache, const int* block_table,
                               int table_stride, int n_blocks, void* stream) {
    XRT_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0, "qkv_prepare: bad head counts %d/%d", n_heads, n_kv_heads);
    XRT_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= MAX_HEAD_DIM,
                "qkv_prepare: head_dim %d must be even and at most %d", head_dim, MAX_HEAD_DIM);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "qkv_prepare: unknown dtype %d", dtype);
    XRT_REQUIRE(norm_dtype == XRT_F32 || norm_dtype == XRT_BF16, "qkv_prepare: unknown norm dtype %d", norm_dtype);
    XRT_REQUIRE(rope_theta == nullptr || (rope_dim > 0 && rope_dim % 2 == 0 && rope_dim <= head_dim),
                "qkv_prepare: rope_dim %d must be even and at most head_dim %d", rope_dim, head_dim);
    XRT_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "qkv_prepare: key and value cache come together");
    XRT_REQUIRE(k_cache == nullptr || (block_table != nullptr && table_stride > 0 && n_blocks > 0 && slots != nullptr),
                "qkv_prepare: a cache write needs slots and a block table");
    XRT_REQUIRE(positions != nullptr, "qkv_prepare: positions missing");
    if (tokens == 0) return 0;
    const long items = (long)tokens * (n_heads + 2 * n_kv_heads);
    const unsigned grid = (unsigned)((items + WAVES - 1) / WAVES);
    hipStream_t s = (hipStream_t)stream;
#define XRT_PREP(T, TW)                                                                                   \
    qkv_prepare_kernel<T, TW><<<grid, WAVES * XRT_WAVE, 0, s>>>(                                          \
        (T*)qkv, (int)items, n_heads, n_kv_heads, head_dim, positions, slots, (const TW*)q_norm,          \
        (const TW*)k_norm, norm_eps, rope_theta, rope_dim, rope_scale, (T*)k_cache, (T*)v_cache,          \
        block_table, table_stride, n_blocks)
    if (dtype == XRT_F32 && norm_dtype == XRT_F32) XRT_PREP(float, float);
    else if (dtype == XRT_F32) XRT_PREP(float, bf16);
    else if (norm_dtype == XRT_F32) XRT_PREP(bf16, float);
    else XRT_PREP(bf16, bf16);
#undef XRT_PREP
    XRT_LAUNCH_CHECK("qkv_prepare");
    return 0;
}
