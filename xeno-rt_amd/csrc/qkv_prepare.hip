// After the q/k/v projection, in one pass over a token's heads: RMSNorm of every head of
// q and k (one weight [head_dim] each), rotation of q and k by the token's position, and
// the write of k (rotated) and v (raw) into the sequence's cache block.
//
// Reference formulas: head norm crates/xrt-models/src/llama.rs:1025-1040 (val * inv_rms * w);
// rotation crates/xrt-kernels/src/cpu/rope.rs:59-89: angle = pos * scale / theta_i, pairs
// (i, i + rope_dim/2), d[i] = a cos - b sin, d[i + half] = a sin + b cos; elements beyond
// rope_dim stay. Norm, angle, sine, cosine and rotation are float32.
//
// Three kernels. The vector kernel takes the usual case (the rotation spans the whole head, and
// the head size is 16 bytes times a power of two, twice): the lanes of a head each hold 16 bytes
// of its lower and of its upper half, which are each other's partners in the rotation, so a
// head is read and written in 16-byte pieces and the norm's sum is a few lane exchanges. When a
// step brings many tokens, the values go to their transposed cache blocks through a kernel of
// their own, which turns tiles of 64 tokens in LDS so that writes to the cache are whole lines.
// Where a key or a value lies inside its block: cache_layout.h.
// The general kernel (one wavefront per (token, head), any even head size and rotation width)
// takes the rest. A token with a negative slot is padding and is not cached. Per head, all
// kernels use the same formulas in the same order; only the order of the norm's sum differs,
// and which kernel a model takes depends on its sizes alone, never on the step.
#include "cache_layout.h"
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
                v_cache[cache_base + cache_value_offset(e, within, head_dim)] = row[e];
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
        if (is_k && cache_base >= 0) k_cache[cache_base + cache_key_offset(within, e, head_dim)] = value;
    }
}


template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T e[N]; };

// One workgroup per token. LANES lanes per head; head_dim = 2 * LANES * VEC with VEC elements in
// 16 bytes. Sine and cosine of the token's angles are worked out once, into LDS, and serve all
// its heads.
template <typename T, typename TW, int LANES>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) qkv_prepare_vector_kernel(
    T* __restrict__ qkv, int n_heads, int n_kv_heads,
    const int* __restrict__ positions, const int* __restrict__ slots,
    const TW* __restrict__ q_norm, const TW* __restrict__ k_norm, float norm_eps,
    const float* __restrict__ rope_theta, float rope_scale,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, int write_values) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int HALF = LANES * VEC, HEAD = 2 * HALF;
    constexpr int HEADS_PER_WAVE = XRT_WAVE / LANES;
    __shared__ float cosines[HALF], sines[HALF];
    const int wave = threadIdx.x / XRT_WAVE, lane = threadIdx.x % XRT_WAVE;
    const int token = blockIdx.x;
    const int pos = positions[token];
    const int slot = slots[token];
    if (rope_theta != nullptr) {
        for (int i = threadIdx.x; i < HALF; i += WAVES * XRT_WAVE) {
            const float angle = (float)pos * rope_scale / rope_theta[i];
            sincosf(angle, &sines[i], &cosines[i]);
        }
    }
    __syncthreads();
    const int at = (lane % LANES) * VEC;           // this lane's elements: at.. in the lower half, HALF + at.. in the upper
    const int heads_total = n_heads + 2 * n_kv_heads;
    const int within = pos % XRT_BLOCK_TOKENS;
    const int heads_here = write_values ? heads_total : n_heads + n_kv_heads;     // value heads come last
    for (int head = wave * HEADS_PER_WAVE + lane / LANES; head < heads_here; head += WAVES * HEADS_PER_WAVE) {
        // lanes of one head stay together: the exchanges below are within a head
        const bool is_q = head < n_heads, is_v = head >= n_heads + n_kv_heads, is_k = !is_q && !is_v;
        T* row = qkv + (long)token * heads_total * HEAD + (long)head * HEAD;
        const Pack<T, VEC> lower = *reinterpret_cast<const Pack<T, VEC>*>(row + at);
        const Pack<T, VEC> upper = *reinterpret_cast<const Pack<T, VEC>*>(row + HALF + at);
        long cache_base = -1;
        if (!is_q && k_cache != nullptr)
            cache_base = cache_block_base(block_table, table_stride, n_blocks, slot, pos, n_kv_heads,
                                          head - n_heads - (is_v ? n_kv_heads : 0), HEAD);
        if (is_v) {
            if (cache_base >= 0) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v_cache[cache_base + cache_value_offset(at + e, within, HEAD)] = lower.e[e];
                    v_cache[cache_base + cache_value_offset(HALF + at + e, within, HEAD)] = upper.e[e];
                }
            }
            continue;
        }
        float a[VEC], b[VEC];
        float sum_sq = 0.f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) { a[e] = to_float(lower.e[e]); sum_sq = fmaf(a[e], a[e], sum_sq); }
#pragma unroll
        for (int e = 0; e < VEC; ++e) { b[e] = to_float(upper.e[e]); sum_sq = fmaf(b[e], b[e], sum_sq); }
        const TW* norm = is_q ? q_norm : k_norm;
        if (norm != nullptr) {
#pragma unroll
            for (int offset = LANES / 2; offset > 0; offset >>= 1) sum_sq += __shfl_xor(sum_sq, offset, XRT_WAVE);
            const float inv_rms = 1.0f / sqrtf(sum_sq / (float)HEAD + norm_eps);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                a[e] = a[e] * inv_rms * to_float(norm[at + e]);
                b[e] = b[e] * inv_rms * to_float(norm[HALF + at + e]);
            }
        }
        if (rope_theta != nullptr) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float sine = sines[at + e], cosine = cosines[at + e];
                const float lo = a[e], hi = b[e];
                a[e] = lo * cosine - hi * sine;
                b[e] = lo * sine + hi * cosine;
            }
        }
        Pack<T, VEC> out_lower, out_upper;
#pragma unroll
        for (int e = 0; e < VEC; ++e) { out_lower.e[e] = from_float<T>(a[e]); out_upper.e[e] = from_float<T>(b[e]); }
        *reinterpret_cast<Pack<T, VEC>*>(row + at) = out_lower;
        *reinterpret_cast<Pack<T, VEC>*>(row + HALF + at) = out_upper;
        if (is_k && cache_base >= 0) {
            T* dst = k_cache + cache_base;                  // (16 bytes from a multiple of 16 bytes stay together in the cache's order)
            *reinterpret_cast<Pack<T, VEC>*>(dst + cache_key_offset(within, at, HEAD)) = out_lower;
            *reinterpret_cast<Pack<T, VEC>*>(dst + cache_key_offset(within, HALF + at, HEAD)) = out_upper;
        }
    }
}

// Values of 64 consecutive tokens of a step and one key/value head: read row by row, turned in
// LDS, and written so that a store instruction of a wavefront takes 8 tokens of 8 dims: where the
// tokens follow each other in a sequence these are the eight pieces of one line of the cache block
// (cache_layout.h). Tokens of different sequences or blocks may share a tile: every token has its
// own block.
constexpr int TILE_DIMS = 128;
template <typename T>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) value_cache_write_kernel(
    const T* __restrict__ qkv, int tokens, int n_heads, int n_kv_heads, int head_dim,
    const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_stride, int n_blocks) {
    // A store step reads 8 tokens (rows) x 8 dims: with rows 8 elements longer than a multiple of 256 bytes the 8 rows
    // start 4 (bfloat16) or 8 (float32) banks apart, and the step's 32 or 64 words lie in as many banks.
    __shared__ __attribute__((aligned(16))) T tile[XRT_WAVE][TILE_DIMS + 8];
    __shared__ long bases[XRT_WAVE];                                  // of the tile's tokens: their block (-1: none) ...
    __shared__ int withins[XRT_WAVE];                                 // ... and their place in it
    const int wave = threadIdx.x / XRT_WAVE, lane = threadIdx.x % XRT_WAVE;
    const int first = blockIdx.x * XRT_WAVE, kv_head = blockIdx.y;
    const int heads_total = n_heads + 2 * n_kv_heads;
    if (wave == 0) {
        const int token = first + lane;
        long cache_base = -1;
        int within = 0;
        if (token < tokens) {
            const int pos = positions[token];
            cache_base = cache_block_base(block_table, table_stride, n_blocks, slots[token], pos, n_kv_heads, kv_head, head_dim);
            within = pos % XRT_BLOCK_TOKENS;
        }
        bases[lane] = cache_base;
        withins[lane] = within;
    }
    const T* source = qkv + (long)(n_heads + n_kv_heads + kv_head) * head_dim;
    constexpr int VEC = 16 / (int)sizeof(T);                  // the launcher sends only head sizes that are multiples of this
    for (int d0 = 0; d0 < head_dim; d0 += TILE_DIMS) {
        const int dims = min(TILE_DIMS, head_dim - d0);
        const int pieces = dims / VEC;                        // 16-byte pieces per row
        for (int i = threadIdx.x; i < XRT_WAVE * pieces; i += WAVES * XRT_WAVE) {
            const int r = i / pieces, d = (i % pieces) * VEC;
            const long from = min(first + r, tokens - 1);     // rows past the end repeat the last one; nobody writes them
            *reinterpret_cast<Pack<T, VEC>*>(&tile[r][d]) = *reinterpret_cast<const Pack<T, VEC>*>(source + from * heads_total * head_dim + d0 + d);
        }
        __syncthreads();
        // a store of a wavefront: tokens 8 g .. 8 g + 7 of the tile (lane % 8), dims 8 h .. 8 h + 7 (lane / 8);
        // a wavefront keeps its tokens while it walks the dims
        for (int g = wave; g < XRT_WAVE / 8; g += WAVES) {
            const int token = g * 8 + lane % 8;
            const long cache_base = bases[token];
            const int within = withins[token];
            if (cache_base < 0) continue;
#pragma unroll 4
            for (int d = lane / 8; d < dims; d += 8)
                v_cache[cache_base + cache_value_offset(d0 + d, within, head_dim)] = tile[token][d];
        }
        __syncthreads();
    }
}

__global__ void __launch_bounds__(256) rope_table_kernel(const float* __restrict__ rope_theta, int half, float rope_scale,
                                                         long entries, float2* __restrict__ table) {
    const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= entries) return;
    const int pos = (int)(index / half), i = (int)(index % half);
    const float angle = (float)pos * rope_scale / rope_theta[i];       // as in the kernels above
    float sine, cosine;
    sincosf(angle, &sine, &cosine);
    table[index] = make_float2(cosine, sine);
}

}  // namespace

extern "C" int xrt_rope_table(const float* rope_theta, int rope_dim, float rope_scale, int positions, float* table, void* stream) {
    XRT_REQUIRE(rope_theta && table && rope_dim > 0 && rope_dim % 2 == 0 && positions > 0 && (uintptr_t)table % 8 == 0,
                "rope_table: a rotation over an even number of dims, at least one position, a table aligned to 8 bytes");
    const long entries = (long)positions * (rope_dim / 2);
    rope_table_kernel<<<(unsigned)((entries + 255) / 256), 256, 0, (hipStream_t)stream>>>(rope_theta, rope_dim / 2, rope_scale, entries, (float2*)table);
    XRT_LAUNCH_CHECK("rope_table");
    return 0;
}

extern "C" int xrt_qkv_prepare(void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                               const int* positions, const int* slots, const void* q_norm, const void* k_norm,
                               int norm_dtype, float norm_eps, const float* rope_theta, int rope_dim,
                               float rope_scale, void* k_cache, void* v_cache, const int* block_table,
                               int table_stride, int n_blocks, int longest_run, void* stream) {
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
    hipStream_t s = (hipStream_t)stream;
    // the vector kernel: rotation over the whole head (or none), 16-byte pieces, a power of two of lanes per head
    const int vec = dtype == XRT_F32 ? 4 : 8;
    const int lanes = head_dim % (2 * vec) == 0 ? head_dim / (2 * vec) : 0;
    const bool vector = lanes >= 1 && lanes <= XRT_WAVE && (lanes & (lanes - 1)) == 0 &&
                        (rope_theta == nullptr || rope_dim == head_dim) && (uintptr_t)qkv % 16 == 0 &&
                        (k_cache == nullptr || ((uintptr_t)k_cache % 16 == 0));
    if (vector) {
        // sequences that bring many tokens: their values go through the transposing kernel;
        // otherwise element by element from this one
        const bool values_apart = v_cache != nullptr && longest_run >= XRT_WAVE / 2;
        const unsigned grid = (unsigned)tokens;
#define XRT_VEC(T, TW, L)                                                                                  \
    qkv_prepare_vector_kernel<T, TW, L><<<grid, WAVES * XRT_WAVE, 0, s>>>(                                 \
        (T*)qkv, n_heads, n_kv_heads, positions, slots, (const TW*)q_norm, (const TW*)k_norm,              \
        norm_eps, rope_theta, rope_scale, (T*)k_cache, (T*)v_cache, block_table, table_stride, n_blocks,   \
        values_apart ? 0 : 1)
#define XRT_VEC_LANES(T, TW)                                                                               \
    switch (lanes) {                                                                                       \
        case 1: XRT_VEC(T, TW, 1); break;                                                                  \
        case 2: XRT_VEC(T, TW, 2); break;                                                                  \
        case 4: XRT_VEC(T, TW, 4); break;                                                                  \
        case 8: XRT_VEC(T, TW, 8); break;                                                                  \
        case 16: XRT_VEC(T, TW, 16); break;                                                                \
        case 32: XRT_VEC(T, TW, 32); break;                                                                \
        default: XRT_VEC(T, TW, 64); break;                                                                \
    }
        if (dtype == XRT_F32 && norm_dtype == XRT_F32) { XRT_VEC_LANES(float, float) }
        else if (dtype == XRT_F32) { XRT_VEC_LANES(float, bf16) }
        else if (norm_dtype == XRT_F32) { XRT_VEC_LANES(bf16, float) }
        else { XRT_VEC_LANES(bf16, bf16) }
#undef XRT_VEC_LANES
#undef XRT_VEC
        XRT_LAUNCH_CHECK("qkv_prepare");
        if (values_apart) {
            const dim3 tiles((unsigned)((tokens + XRT_WAVE - 1) / XRT_WAVE), (unsigned)n_kv_heads);
            if (dtype == XRT_F32)
                value_cache_write_kernel<float><<<tiles, WAVES * XRT_WAVE, 0, s>>>(
                    (const float*)qkv, tokens, n_heads, n_kv_heads, head_dim, positions, slots, (float*)v_cache,
                    block_table, table_stride, n_blocks);
            else
                value_cache_write_kernel<bf16><<<tiles, WAVES * XRT_WAVE, 0, s>>>(
                    (const bf16*)qkv, tokens, n_heads, n_kv_heads, head_dim, positions, slots, (bf16*)v_cache,
                    block_table, table_stride, n_blocks);
            XRT_LAUNCH_CHECK("qkv_prepare (values)");
        }
        return 0;
    }
    const unsigned grid = (unsigned)((items + WAVES - 1) / WAVES);
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
