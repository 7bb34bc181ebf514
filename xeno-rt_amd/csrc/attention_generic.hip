// Causal attention of every token of a step over its own sequence's cache, float32 math,
// for any element type, head size (up to 512), head grouping and window.
// It is the attention of the 32-bit path and the fallback of the bfloat16 path.
//
// Reference: crates/xrt-models/src/llama.rs:504-574 (online softmax: running maximum m and
// sum l, rescaled by exp(m_old - m_new)) and :727-770 (a token at position P sees keys
// 0..P; query head h reads key/value head h / group; score = (q.k) * scale).
//
// One wavefront per (token, head), or a workgroup of eight where a step brings few tokens. Keys are visited block by
// block (64 keys, lane j takes key j) in chunks of eight blocks that are cut at absolute positions and merged in
// their order, whatever the step looks like, so the result of a token does not depend on how its request was cut
// into steps or batched, nor on which of the two launches a step takes.
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

// What one wavefront keeps of the keys it has seen for one (token, head): the largest score, the sum of the
// probabilities relative to it, and the weighted values of the dims this lane owns (lane, lane + 64, ...).
struct Seen {
    float m, l, acc[MAX_OWNED];
    __device__ __forceinline__ void clear() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int i = 0; i < MAX_OWNED; ++i) acc[i] = 0.f;
    }
};

// The keys of a sequence are taken in chunks of CHUNK_BLOCKS cache blocks, cut at absolute positions (chunk c holds the
// keys from 512 c on). A chunk is worked off from empty hands (its own maximum, sum and weighted values) and then
// merged into what the chunks before it left, in the order of the chunks. So it makes no difference to the result
// whether one wavefront takes all chunks of a (token, head) one after the other (many tokens in a step) or the
// wavefronts of a workgroup take them side by side (few tokens: a decode step, where one wavefront per (token, head)
// would leave most of the chip idle): the same sums in the same order, to the bit.
constexpr int CHUNK_BLOCKS = 8;

// `from` merged into `into` (both relative to their own maximum). The products are rounded before they are added
// (explicit fmaf: what the compiler may contract elsewhere it must not contract differently in two kernels).
__device__ __forceinline__ void merge(Seen& into, const Seen& from) {
    const float m_new = fmaxf(into.m, from.m);
    const float keep = expf(into.m - m_new), take = expf(from.m - m_new);     // keep is 0 for empty hands (m = -inf)
    const float taken = from.l * take;
    into.l = fmaf(into.l, keep, taken);
#pragma unroll
    for (int i = 0; i < MAX_OWNED; ++i) {
        const float part = from.acc[i] * take;
        into.acc[i] = fmaf(into.acc[i], keep, part);
    }
    into.m = m_new;
}

// The blocks b_begin .. b_end of the sequence in `slot`, for the query whose dims lie in qs: online softmax as in
// llama.rs:514-574, block by block (64 keys, lane j takes key j). ps: 64 floats of LDS of this wavefront.
template <typename T>
__device__ __forceinline__ void attend_blocks(Seen& seen, int b_begin, int b_end, int first, int pos, const float* qs, float* ps,
                                              const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                              const int* __restrict__ table, int n_blocks, int n_kv_heads, int kv_head, int head_dim,
                                              float scale, bool biased, float slope, bool whole_pieces) {
    const int lane = threadIdx.x % XRT_WAVE;
    for (int b = b_begin; b <= b_end; ++b) {
        const int block = table[b];
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
            if (biased) s += slope * (float)(j - pos);
        }
        const float m_new = fmaxf(seen.m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float correction = expf(seen.m - m_new);         // 0 for the first block (m = -inf)
        seen.l = seen.l * correction + wave_sum(p);
        seen.m = m_new;
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
                seen.acc[i] = seen.acc[i] * correction + sum;
            }
        }
        wave_sync();
    }
}

// WAVES wavefronts per (token, head): 1 where a step brings tokens enough to fill the chip, CHUNK_WAVES where it brings few.
constexpr int CHUNK_WAVES = 8;

template <typename T, int WAVES>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) attention_generic_kernel(
    const T* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads, int head_dim,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ positions, const int* __restrict__ slots,
    T* __restrict__ out, float scale, int window, const float* __restrict__ distance_slopes) {
    __shared__ float qs[MAX_HEAD_DIM];
    __shared__ float ps[WAVES][XRT_WAVE];
    // what the wavefronts found in the chunks of a round, for the merge: two sets, used in turn (WAVES > 1)
    __shared__ float round_ml[WAVES > 1 ? 2 : 1][WAVES][2];
    extern __shared__ float round_acc[];                       // [2][WAVES][head_dim] where WAVES > 1
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int token = blockIdx.x / n_heads, head = blockIdx.x % n_heads;
    const int kv_head = head / (n_heads / n_kv_heads);
    T* dst = out + ((long)token * n_heads + head) * head_dim;
    const int slot = slots[token];
    if (slot < 0) {                                            // the whole workgroup leaves
        for (int e = threadIdx.x; e < head_dim; e += WAVES * XRT_WAVE) dst[e] = from_float<T>(0.f);
        return;
    }
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const bool biased = distance_slopes != nullptr;
    const float slope = biased ? distance_slopes[head] : 0.f;
    // pieces of eight elements can be loaded whole if they are aligned: head sizes that are multiples of 8, caches aligned to 32 bytes
    const bool whole_pieces = head_dim % 8 == 0 && (uintptr_t)k_cache % 32 == 0 && (uintptr_t)v_cache % 32 == 0;
    const T* q = qkv + (long)token * row_width + (long)head * head_dim;
    for (int e = threadIdx.x; e < head_dim; e += WAVES * XRT_WAVE) qs[e] = to_float(q[e]);
    if constexpr (WAVES > 1) __syncthreads(); else wave_sync();
    const int* table = block_table + (long)slot * table_stride;
    const int first_block = first / XRT_BLOCK_TOKENS, last_block = pos / XRT_BLOCK_TOKENS;
    const int first_chunk = first_block / CHUNK_BLOCKS, last_chunk = last_block / CHUNK_BLOCKS;

    Seen all;
    all.clear();
    if constexpr (WAVES == 1) {
        for (int chunk = first_chunk; chunk <= last_chunk; ++chunk) {
            Seen here;
            here.clear();
            attend_blocks(here, max(first_block, chunk * CHUNK_BLOCKS), min(last_block, chunk * CHUNK_BLOCKS + CHUNK_BLOCKS - 1), first, pos,
                          qs, ps[0], k_cache, v_cache, table, n_blocks, n_kv_heads, kv_head, head_dim, scale, biased, slope, whole_pieces);
            merge(all, here);
        }
    } else {
        // rounds of WAVES chunks: every wavefront takes one, leaves what it found in LDS, and all wavefronts merge the
        // round's chunks in order (each for itself: they all hold the same sums, and the first writes them in the end)
        int set = 0;
        for (int round = first_chunk; round <= last_chunk; round += WAVES, set ^= 1) {
            const int chunk = round + wave;
            float* mine = round_acc + ((long)set * WAVES + wave) * head_dim;
            if (chunk <= last_chunk) {
                Seen here;
                here.clear();
                attend_blocks(here, max(first_block, chunk * CHUNK_BLOCKS), min(last_block, chunk * CHUNK_BLOCKS + CHUNK_BLOCKS - 1), first, pos,
                              qs, ps[wave], k_cache, v_cache, table, n_blocks, n_kv_heads, kv_head, head_dim, scale, biased, slope, whole_pieces);
#pragma unroll
                for (int i = 0; i < MAX_OWNED; ++i)
                    if (lane + i * XRT_WAVE < head_dim) mine[lane + i * XRT_WAVE] = here.acc[i];
                if (lane == 0) { round_ml[set][wave][0] = here.m; round_ml[set][wave][1] = here.l; }
            }
            __syncthreads();                                   // (a set is written again two rounds on, after the next barrier)
            for (int w = 0; w < WAVES && round + w <= last_chunk; ++w) {
                Seen from;
                from.m = round_ml[set][w][0];
                from.l = round_ml[set][w][1];
                const float* theirs = round_acc + ((long)set * WAVES + w) * head_dim;
#pragma unroll
                for (int i = 0; i < MAX_OWNED; ++i) from.acc[i] = lane + i * XRT_WAVE < head_dim ? theirs[lane + i * XRT_WAVE] : 0.f;
                merge(all, from);
            }
        }
        if (wave != 0) return;
    }
    const float inv = all.l > 0.f ? 1.0f / all.l : 0.f;        // llama.rs:566-571
#pragma unroll
    for (int i = 0; i < MAX_OWNED; ++i) {
        const int d = lane + i * XRT_WAVE;
        if (d < head_dim) dst[d] = from_float<T>(all.acc[i] * inv);
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
    // few (token, head) pairs (a decode step): a workgroup of wavefronts each, which take the chunks of keys side by side
    const bool side_by_side = items <= 8L * XRT_COMPUTE_UNITS;
    const size_t round_bytes = (size_t)2 * CHUNK_WAVES * head_dim * sizeof(float);
#define XRT_GENERIC(T, WAVES_)                                                                                            \
    attention_generic_kernel<T, WAVES_><<<(unsigned)items, WAVES_ * XRT_WAVE, WAVES_ > 1 ? round_bytes : 0, s>>>(           \
        (const T*)qkv, row_width, n_heads, n_kv_heads, head_dim, (const T*)k_cache, (const T*)v_cache, block_table,       \
        table_stride, n_blocks, positions, slots, (T*)out, scale, window, distance_slopes)
    if (dtype == XRT_F32) { if (side_by_side) XRT_GENERIC(float, CHUNK_WAVES); else XRT_GENERIC(float, 1); }
    else { if (side_by_side) XRT_GENERIC(bf16, CHUNK_WAVES); else XRT_GENERIC(bf16, 1); }
#undef XRT_GENERIC
    XRT_LAUNCH_CHECK("attention (generic)");
    return 0;
}
