// Causal attention of every token of a step over its own sequence's cache, float32 math,
// for any element type, head size (up to 512), head grouping and window.
// It is the attention of the 32-bit path and the fallback of the bfloat16 path.
//
// Reference: crates/xrt-models/src/llama.rs:504-574 (online softmax: running maximum m and
// sum l, rescaled by exp(m_old - m_new)) and :727-770 (a token at position P sees keys
// 0..P; query head h reads key/value head h / group; score = (q.k) * scale).
//
// One wavefront per (token, head), or a workgroup of eight where a step brings few tokens; with grouped heads and a head
// size of up to 128 a wavefront takes two or four query heads of one key/value head together: a piece of a key or a
// value is loaded once for all of them, and their chains of dependent steps (score, maximum, sum) run side by side,
// each with the arithmetic and the order it has alone (so the bits do not depend on it). Keys are visited block by
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
template <int OWNED>
struct Seen {
    float m, l, acc[OWNED];
    __device__ __forceinline__ void clear() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int i = 0; i < OWNED; ++i) acc[i] = 0.f;
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
template <int OWNED>
__device__ __forceinline__ void merge(Seen<OWNED>& into, const Seen<OWNED>& from) {
    const float m_new = fmaxf(into.m, from.m);
    const float keep = expf(into.m - m_new), take = expf(from.m - m_new);     // keep is 0 for empty hands (m = -inf)
    const float taken = from.l * take;
    into.l = fmaf(into.l, keep, taken);
#pragma unroll
    for (int i = 0; i < OWNED; ++i) {
        const float part = from.acc[i] * take;
        into.acc[i] = fmaf(into.acc[i], keep, part);
    }
    into.m = m_new;
}

// The blocks b_begin .. b_end of the sequence in `slot`, for the G queries (heads of one key/value head) whose dims lie in
// qs[g * head_dim ..]: online softmax as in llama.rs:514-574, block by block (64 keys, lane j takes key j).
// ps: G x 64 floats of LDS of this wavefront. slopes: of the G heads (biased).
template <typename T, int G, int OWNED>
__device__ __forceinline__ void attend_blocks(Seen<OWNED> (&seen)[G], int b_begin, int b_end, int first, int pos, const float* qs, float* ps,
                                              const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                              const int* __restrict__ table, int n_blocks, int n_kv_heads, int kv_head, int head_dim,
                                              float scale, bool biased, const float (&slopes)[G], bool whole_pieces) {
    const int lane = threadIdx.x % XRT_WAVE;
    for (int b = b_begin; b <= b_end; ++b) {
        const int block = table[b];
        if (block < 0 || block >= n_blocks) continue;          // the host never lets this happen
        const int j = b * XRT_BLOCK_TOKENS + lane;
        const bool valid = j >= first && j <= pos;
        const long head_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
        float s[G];
#pragma unroll
        for (int g = 0; g < G; ++g) s[g] = -INFINITY;
        if (valid) {
            // the key's dims in order, piece by piece of the cache's order: a piece's products are added up, then
            // the pieces' sums (less rounding than one running sum)
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; ++g) dot[g] = 0.f;
            if (whole_pieces) {
#pragma unroll 4
                for (int d0 = 0; d0 < head_dim; d0 += 8) {
                    float key[8];
                    load_piece(k_cache + head_base + cache_key_offset(lane, d0, head_dim), key);
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        float of_piece = 0.f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) of_piece = fmaf(qs[g * head_dim + d0 + e], key[e], of_piece);
                        dot[g] += of_piece;
                    }
                }
            } else {
                for (int d0 = 0; d0 < head_dim; d0 += 8) {
                    const T* piece = k_cache + head_base + cache_key_offset(lane, d0, head_dim);
                    const int dims = min(8, head_dim - d0);
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        float of_piece = 0.f;
                        for (int e = 0; e < dims; ++e) of_piece = fmaf(qs[g * head_dim + d0 + e], to_float(piece[e]), of_piece);
                        dot[g] += of_piece;
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                s[g] = dot[g] * scale;
                if (biased) s[g] = fmaf(slopes[g], (float)(j - pos), s[g]);
            }
        }
        float correction[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float m_new = fmaxf(seen[g].m, wave_max(s[g]));
            const float p = valid ? expf(s[g] - m_new) : 0.f;
            correction[g] = expf(seen[g].m - m_new);           // 0 for the first block (m = -inf)
            seen[g].l = fmaf(seen[g].l, correction[g], wave_sum(p));    // (explicit, like all sums of a product here: the kernel's variants must agree to the bit)
            seen[g].m = m_new;
            ps[g * XRT_WAVE + lane] = p;
        }
        wave_sync();
        const int j_begin = max(0, first - b * XRT_BLOCK_TOKENS);
        const int j_end = min(XRT_BLOCK_TOKENS - 1, pos - b * XRT_BLOCK_TOKENS);
#pragma unroll
        for (int i = 0; i < OWNED; ++i) {
            const int d = lane + i * XRT_WAVE;
            if (d < head_dim) {
                float sum[G];
#pragma unroll
                for (int g = 0; g < G; ++g) sum[g] = 0.f;
#pragma unroll 4
                for (int j0 = j_begin / 8 * 8; j0 <= j_end; j0 += 8) {   // the dim's values in the order of their tokens
                    const T* piece = v_cache + head_base + cache_value_offset(d, j0, head_dim);
                    if (whole_pieces) {
                        float value[8];                         // (what lies beyond the sequence's end is loaded and not used)
                        load_piece(piece, value);
#pragma unroll
                        for (int g = 0; g < G; ++g)
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (j0 + e >= j_begin && j0 + e <= j_end) sum[g] = fmaf(ps[g * XRT_WAVE + j0 + e], value[e], sum[g]);
                    } else {
                        for (int jj = max(j0, j_begin); jj <= min(j0 + 7, j_end); ++jj) {
                            const float value = to_float(piece[jj - j0]);
#pragma unroll
                            for (int g = 0; g < G; ++g) sum[g] = fmaf(ps[g * XRT_WAVE + jj], value, sum[g]);
                        }
                    }
                }
#pragma unroll
                for (int g = 0; g < G; ++g) seen[g].acc[i] = fmaf(seen[g].acc[i], correction[g], sum[g]);
            }
        }
        wave_sync();
    }
}

// WAVES wavefronts per (token, G heads): 1 where a step brings tokens enough to fill the chip, CHUNK_WAVES where it brings few.
// G: query heads of one key/value head that a wavefront takes together (1, or 2 or 4 with OWNED = 2: head sizes up to 128).
constexpr int CHUNK_WAVES = 8;

template <typename T, int WAVES, int G, int OWNED>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) attention_generic_kernel(
    const T* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads, int head_dim,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ positions, const int* __restrict__ slots,
    T* __restrict__ out, float scale, int window, const float* __restrict__ distance_slopes) {
    __shared__ float qs[G * OWNED * XRT_WAVE];                 // [G][head_dim]
    __shared__ float ps[WAVES][G * XRT_WAVE];
    // what the wavefronts found in the chunks of a round, for the merge: two sets, used in turn (WAVES > 1)
    __shared__ float round_ml[WAVES > 1 ? 2 : 1][WAVES][G][2];
    extern __shared__ float round_acc[];                       // [2][WAVES][G][head_dim] where WAVES > 1
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int sets = n_heads / G;                              // sets of G heads per token
    const int token = blockIdx.x / sets, head0 = blockIdx.x % sets * G;
    const int kv_head = head0 / (n_heads / n_kv_heads);        // (G divides the group: the set shares its key/value head)
    T* dst = out + ((long)token * n_heads + head0) * head_dim;
    const int slot = slots[token];
    if (slot < 0) {                                            // the whole workgroup leaves
        for (int e = threadIdx.x; e < G * head_dim; e += WAVES * XRT_WAVE) dst[e] = from_float<T>(0.f);
        return;
    }
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const bool biased = distance_slopes != nullptr;
    float slopes[G];
#pragma unroll
    for (int g = 0; g < G; ++g) slopes[g] = biased ? distance_slopes[head0 + g] : 0.f;
    // pieces of eight elements can be loaded whole if they are aligned: head sizes that are multiples of 8, caches aligned to 32 bytes
    const bool whole_pieces = head_dim % 8 == 0 && (uintptr_t)k_cache % 32 == 0 && (uintptr_t)v_cache % 32 == 0;
    const T* q = qkv + (long)token * row_width + (long)head0 * head_dim;      // the set's heads lie side by side
    for (int e = threadIdx.x; e < G * head_dim; e += WAVES * XRT_WAVE) qs[e] = to_float(q[e]);
    if constexpr (WAVES > 1) __syncthreads(); else wave_sync();
    const int* table = block_table + (long)slot * table_stride;
    const int first_block = first / XRT_BLOCK_TOKENS, last_block = pos / XRT_BLOCK_TOKENS;
    const int first_chunk = first_block / CHUNK_BLOCKS, last_chunk = last_block / CHUNK_BLOCKS;

    Seen<OWNED> all[G];
#pragma unroll
    for (int g = 0; g < G; ++g) all[g].clear();
    if constexpr (WAVES == 1) {
        for (int chunk = first_chunk; chunk <= last_chunk; ++chunk) {
            Seen<OWNED> here[G];
#pragma unroll
            for (int g = 0; g < G; ++g) here[g].clear();
            attend_blocks<T, G, OWNED>(here, max(first_block, chunk * CHUNK_BLOCKS), min(last_block, chunk * CHUNK_BLOCKS + CHUNK_BLOCKS - 1),
                                       first, pos, qs, ps[0], k_cache, v_cache, table, n_blocks, n_kv_heads, kv_head, head_dim, scale,
                                       biased, slopes, whole_pieces);
#pragma unroll
            for (int g = 0; g < G; ++g) merge(all[g], here[g]);
        }
    } else {
        // rounds of WAVES chunks: every wavefront takes one, leaves what it found in LDS, and all wavefronts merge the
        // round's chunks in order (each for itself: they all hold the same sums, and the first writes them in the end)
        int set = 0;
        for (int round = first_chunk; round <= last_chunk; round += WAVES, set ^= 1) {
            const int chunk = round + wave;
            float* mine = round_acc + ((long)set * WAVES + wave) * G * head_dim;
            if (chunk <= last_chunk) {
                Seen<OWNED> here[G];
#pragma unroll
                for (int g = 0; g < G; ++g) here[g].clear();
                attend_blocks<T, G, OWNED>(here, max(first_block, chunk * CHUNK_BLOCKS), min(last_block, chunk * CHUNK_BLOCKS + CHUNK_BLOCKS - 1),
                                           first, pos, qs, ps[wave], k_cache, v_cache, table, n_blocks, n_kv_heads, kv_head, head_dim, scale,
                                           biased, slopes, whole_pieces);
#pragma unroll
                for (int g = 0; g < G; ++g) {
#pragma unroll
                    for (int i = 0; i < OWNED; ++i)
                        if (lane + i * XRT_WAVE < head_dim) mine[g * head_dim + lane + i * XRT_WAVE] = here[g].acc[i];
                    if (lane == 0) { round_ml[set][wave][g][0] = here[g].m; round_ml[set][wave][g][1] = here[g].l; }
                }
            }
            __syncthreads();                                   // (a set is written again two rounds on, after the next barrier)
            for (int w = 0; w < WAVES && round + w <= last_chunk; ++w) {
                const float* theirs = round_acc + ((long)set * WAVES + w) * G * head_dim;
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    Seen<OWNED> from;
                    from.m = round_ml[set][w][g][0];
                    from.l = round_ml[set][w][g][1];
#pragma unroll
                    for (int i = 0; i < OWNED; ++i) from.acc[i] = lane + i * XRT_WAVE < head_dim ? theirs[g * head_dim + lane + i * XRT_WAVE] : 0.f;
                    merge(all[g], from);
                }
            }
        }
        if (wave != 0) return;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float inv = all[g].l > 0.f ? 1.0f / all[g].l : 0.f;        // llama.rs:566-571
#pragma unroll
        for (int i = 0; i < OWNED; ++i) {
            const int d = lane + i * XRT_WAVE;
            if (d < head_dim) dst[g * head_dim + d] = from_float<T>(all[g].acc[i] * inv);
        }
    }
}

}  // namespace

int xrt_attention_generic(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                          const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                          int n_blocks, const int* positions, const int* slots, void* out, float scale,
                          int window, const float* distance_slopes, hipStream_t s) {
    XRT_REQUIRE(head_dim <= MAX_HEAD_DIM, "attention: head_dim %d exceeds %d", head_dim, MAX_HEAD_DIM);
    // Query heads of a key/value head that a wavefront takes together: as many of the group as 4, for head sizes up to 128
    // (what a lane then owns of a head fits two registers a head), where that still leaves two workgroups to a compute
    // unit (a decode step of few sequences would rather have the workgroups). Either way a head's arithmetic is the same.
    const int group = n_heads / n_kv_heads;
    int together = head_dim > 2 * XRT_WAVE ? 1 : group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    if ((long)tokens * (n_heads / together) < 2L * XRT_COMPUTE_UNITS) together = 1;
    const long items = (long)tokens * (n_heads / together);
    XRT_REQUIRE((long)tokens * n_heads < (1L << 31), "attention: too many (token, head) pairs");
    const int row_width = (n_heads + 2 * n_kv_heads) * head_dim;
    // few (token, head) pairs (a decode step): a workgroup of wavefronts each, which take the chunks of keys side by side
    const bool side_by_side = (long)tokens * n_heads <= 8L * XRT_COMPUTE_UNITS;
    const size_t round_bytes = (size_t)2 * CHUNK_WAVES * together * head_dim * sizeof(float);
#define XRT_GENERIC(T, WAVES_, G_, OWNED_)                                                                                \
    attention_generic_kernel<T, WAVES_, G_, OWNED_><<<(unsigned)items, WAVES_ * XRT_WAVE, WAVES_ > 1 ? round_bytes : 0, s>>>( \
        (const T*)qkv, row_width, n_heads, n_kv_heads, head_dim, (const T*)k_cache, (const T*)v_cache, block_table,       \
        table_stride, n_blocks, positions, slots, (T*)out, scale, window, distance_slopes)
#define XRT_GENERIC_WAVES(T, G_, OWNED_) do { if (side_by_side) XRT_GENERIC(T, CHUNK_WAVES, G_, OWNED_); else XRT_GENERIC(T, 1, G_, OWNED_); } while (0)
#define XRT_GENERIC_SETS(T)                                                                                               \
    do {                                                                                                                  \
        if (together == 4) XRT_GENERIC_WAVES(T, 4, 2);                                                                    \
        else if (together == 2) XRT_GENERIC_WAVES(T, 2, 2);                                                               \
        else XRT_GENERIC_WAVES(T, 1, MAX_OWNED);                                                                          \
    } while (0)
    if (dtype == XRT_F32) XRT_GENERIC_SETS(float); else XRT_GENERIC_SETS(bf16);
#undef XRT_GENERIC_SETS
#undef XRT_GENERIC_WAVES
#undef XRT_GENERIC
    XRT_LAUNCH_CHECK("attention (generic)");
    return 0;
}
