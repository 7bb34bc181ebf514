// One token for every row of float32 logits: greedy, or temperature sampling with top-k,
// top-p and a repetition penalty. One workgroup per row; nothing leaves the device but the ids.
//
// Meaning of the options: crates/xrt-runtime/src/sampler.rs of the reference.
//   penalty > 1: logits of tokens in the row's history are divided (if > 0) or multiplied (:77-91)
//   temperature <= 1e-5: first index of the maximum, strict >, so NaN never wins (:62-65, :83-98)
//   top_k > 0: only the k largest logits stay (:116-145)
//   weights exp((logit - max) / temperature) (:147-164)
//   top_p < 1: the shortest descending prefix whose share reaches top_p stays (:166-183)
//   inverse CDF with one uniform number (:185-195)
// Where the reference sorts, this kernel finds thresholds by a search on the bit patterns, four
// bits a pass (eight passes over the row instead of thirty-two), so tokens that tie with the
// last kept one stay too; the CDF runs in the order of token ids. With a top-k, what survives it
// is gathered into LDS (if it fits) and top-p and the CDF work on that short list; only without
// a top-k do they pass over the whole row. A workgroup is one compute unit, so a pass is bound by
// how many loads it keeps in flight: sixteen per thread.
//
// A small top-k (up to 64, the usual case) does not pass over the row eight times: the row is cut
// into slices of 4096 tokens, a workgroup per slice holds its slice in registers and finds the
// slice's own k largest (ties included), and the row's workgroup then works on those few
// candidates only: the row's k largest are among them. Slices whose ties overflow their list send the
// row back to the path above. A temperature alone (no top-k, no top-p) goes through the slices too: each
// hands on its mass, the row's workgroup finds the slice in which the drawn number falls and walks it.
#include "common.h"
#include "xrt_hip.h"

namespace {

constexpr int THREADS = 1024;
constexpr int BLOCK_WAVES = THREADS / XRT_WAVE;
constexpr int IN_FLIGHT = 16;          // loads of a thread that a pass keeps in flight
constexpr int MAX_VOCAB = 255 * THREADS;   // the largest vocabulary that goes through slices (one lane per slice below)
constexpr int LARGEST_VOCAB = 1 << 19;     // the largest vocabulary at all: its seen-bitmap, vocab / 8 bytes, fits the LDS of a compute unit beside the rest
constexpr int COUNTED_AT_ONCE = 240;       // keys that a thread counts in 8-bit counters before it empties them
constexpr int SEGMENT = 128;           // survivors of top-k that one wavefront's run of ids may hold in LDS
constexpr int CANDIDATES = 15;         // thresholds tried per pass: the non-zero values of four bits

// monotone map float -> unsigned: a > b  <=>  key(a) > key(b)
__device__ __forceinline__ unsigned order_key(float v) {
    const unsigned bits = __float_as_uint(v);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

struct Row {
    const float* logits;
    const unsigned* seen;
    float penalty;
    bool penalised;
    int vocab;
    // without branches: a pass makes this choice a hundred times per thread
    __device__ __forceinline__ float adjusted(int i, float v) const {
        const unsigned word = penalised ? seen[i >> 5] : 0u;
        const float changed = v > 0.f ? v / penalty : v * penalty;
        return (word >> (i & 31)) & 1u ? changed : v;
    }
    // f(i, value) for this thread's tokens i = tid, tid + THREADS, ..., in ascending order
    template <typename F>
    __device__ __forceinline__ void each(F&& f) const {
        for (int base = threadIdx.x; base < vocab; base += IN_FLIGHT * THREADS) {
            float v[IN_FLIGHT];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) v[u] = logits[min(base + u * THREADS, vocab - 1)];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) {
                const int i = base + u * THREADS;
                if (i < vocab) f(i, adjusted(i, v[u]));
            }
        }
    }
};

constexpr int SUMS = 17;               // most values that block_sums adds at once

// Sums over the block of N values per thread; every thread gets the sums. The order of the
// additions is fixed: lanes in a tree, then wavefronts in order. `scratch` holds
// (BLOCK_WAVES + 1) * SUMS values.
template <typename T, int N, int WAVES_ = BLOCK_WAVES>
__device__ __forceinline__ void block_sums(T (&v)[N], T* scratch) {
    constexpr int BLOCK_WAVES = WAVES_;
    static_assert(N <= SUMS, "scratch too small");
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
#pragma unroll
    for (int j = 0; j < N; ++j)
#pragma unroll
        for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) v[j] += __shfl_xor(v[j], offset, XRT_WAVE);
    __syncthreads();                                   // whoever still reads the scratch of the pass before is done
    if (lane == 0)
#pragma unroll
        for (int j = 0; j < N; ++j) scratch[wave * N + j] = v[j];
    __syncthreads();
    if (threadIdx.x < N) {
        T total = 0;
        for (int w = 0; w < BLOCK_WAVES; ++w) total += scratch[w * N + threadIdx.x];
        scratch[BLOCK_WAVES * N + threadIdx.x] = total;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < N; ++j) v[j] = scratch[BLOCK_WAVES * N + j];
}

// Where a row's token goes: out[r], and, for a caller that keeps the sequences' tokens on the device (what
// the penalty reads), the place behind the row's span of them.
struct Chosen {
    int* out;
    int* history;
    const int* append_at;
    __device__ __forceinline__ void put(int r, int token) const {
        out[r] = token;
        if (append_at != nullptr && append_at[r] >= 0) history[append_at[r]] = token;
    }
};

// The whole of it for row r, by one workgroup of THREADS threads; `seen` holds vocab bits of LDS.
__device__ void sample_row(
    const int r, unsigned* seen,
    const float* __restrict__ logits, int vocab, const Chosen out, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ history, const int* __restrict__ history_spans, const float* __restrict__ uniforms) {
    __shared__ float scratch_f[(BLOCK_WAVES + 1) * SUMS];
    __shared__ unsigned scratch_u[(BLOCK_WAVES + 1) * SUMS];
    __shared__ int survivor_id[BLOCK_WAVES * SEGMENT];      // what top-k leaves, by wavefront run, in the order of ids
    __shared__ float survivor_weight[BLOCK_WAVES * SEGMENT];
    __shared__ int survivors_of[BLOCK_WAVES];
    __shared__ int scratch_i[BLOCK_WAVES];
    __shared__ float wave_mass[BLOCK_WAVES];
    __shared__ float target_in_wave;
    __shared__ int chosen_wave, chosen;

    const int tid = threadIdx.x;
    const int lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    Row row;
    row.logits = logits + (long)r * vocab;
    row.seen = seen;
    row.penalty = penalty[r];
    row.vocab = vocab;
    const int h_begin = history_spans[2 * r], h_end = history_spans[2 * r + 1];
    row.penalised = row.penalty > 1.0f && h_end > h_begin;
    if (row.penalised) {
        const int words = (vocab + 31) / 32;
        for (int i = tid; i < words; i += THREADS) seen[i] = 0u;
        __syncthreads();
        for (int i = h_begin + tid; i < h_end; i += THREADS) {
            const int token = history[i];
            if (token >= 0 && token < vocab) atomicOr(&seen[token >> 5], 1u << (token & 31));
        }
        __syncthreads();
    }

    // ---- maximum and its first index -----------------------------------------
    float best = -INFINITY;
    int best_index = 0x7fffffff;
    row.each([&](int i, float v) { if (v > best) { best = v; best_index = i; } });
#pragma unroll
    for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) {
        const float other = __shfl_xor(best, offset, XRT_WAVE);
        const int other_index = __shfl_xor(best_index, offset, XRT_WAVE);
        if (other > best || (other == best && other_index < best_index)) { best = other; best_index = other_index; }
    }
    if (lane == 0) { scratch_f[wave] = best; scratch_i[wave] = best_index; }
    __syncthreads();
    best = scratch_f[0];
    best_index = scratch_i[0];
    for (int w = 1; w < BLOCK_WAVES; ++w) {
        const float other = scratch_f[w];
        const int other_index = scratch_i[w];
        if (other > best || (other == best && other_index < best_index)) { best = other; best_index = other_index; }
    }
    if (best_index == 0x7fffffff) best_index = 0;       // nothing compared greater (all NaN or -inf): index 0
    __syncthreads();

    const float temp = temperature[r];
    if (temp <= 1e-5f) {
        if (tid == 0) out.put(r, best_index);
        return;
    }
    const float inv_temp = 1.0f / temp;

    // ---- top-k: the largest key T with count(key >= T) >= k ---------------------
    // Found four bits at a time from the top. With the bits above already fixed in `low`, a pass
    // counts, among the keys that share those bits, how many have each value of the next four
    // (sixteen 8-bit counters packed into two registers, emptied before any of them can reach 256), and
    // how many keys lie above altogether. The largest value whose keys, with everything above
    // them, number at least k fixes the next four bits.
    unsigned k_threshold = 0u;
    const int k = top_k[r];
    if (k > 0 && k < vocab) {
        unsigned low = 0u;
        for (int shift = 28; shift >= 0; shift -= 4) {
            unsigned long long packed_low = 0ull, packed_high = 0ull;
            unsigned above = 0u;
            const unsigned fixed_bits = shift == 28 ? 0u : low >> (shift + 4);
            unsigned count[SUMS] = {};
            auto empty_counters = [&]() {
#pragma unroll
                for (int d = 0; d < 8; ++d) {
                    count[d] += (unsigned)(packed_low >> (d * 8)) & 255u;
                    count[8 + d] += (unsigned)(packed_high >> (d * 8)) & 255u;
                }
                packed_low = packed_high = 0ull;
            };
            int counted = 0;
            row.each([&](int, float v) {
                const unsigned key = order_key(v);
                const unsigned upper = shift == 28 ? 0u : key >> (shift + 4);
                const unsigned digit = (key >> shift) & 15u;
                const unsigned long long one = 1ull << ((digit & 7u) * 8u);
                if (upper == fixed_bits) {
                    if (digit & 8u) packed_high += one; else packed_low += one;
                } else if (upper > fixed_bits) {
                    above += 1u;
                }
                if (++counted == COUNTED_AT_ONCE) {             // (only vocabularies beyond 245 760 get here)
                    empty_counters();
                    counted = 0;
                }
            });
            empty_counters();
            count[16] = above;
            block_sums(count, scratch_u);
            unsigned at_or_above = count[16], digit = 0u;
            bool found = false;
#pragma unroll
            for (int d = 15; d >= 0; --d) {
                at_or_above += count[d];
                if (!found && at_or_above >= (unsigned)k) { digit = (unsigned)d; found = true; }
            }
            low |= digit << shift;                      // found always: the keys at or above low number at least k
        }
        k_threshold = low;
    }
    auto weight = [&](float v) -> float {
        return order_key(v) >= k_threshold ? expf((v - best) * inv_temp) : 0.f;
    };

    const float p = top_p[r];
    // ---- with a top-k: its survivors go to LDS, in the order of ids ------------------
    // Every wavefront owns a run of consecutive ids, reads it 64 ids at a time and appends what
    // survives to its own segment of the list. If a segment overflows (ties by the thousand), the
    // general path below takes over.
    const int span = ((vocab + BLOCK_WAVES - 1) / BLOCK_WAVES + XRT_WAVE - 1) / XRT_WAVE * XRT_WAVE;
    const int begin = min(vocab, wave * span), end = min(vocab, begin + span);
    if (k > 0 && k < vocab) {
        int held = 0;                                   // uniform in the wavefront
        for (int base = begin; base < end; base += IN_FLIGHT * XRT_WAVE) {
            float v[IN_FLIGHT];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) v[u] = row.logits[min(base + u * XRT_WAVE + lane, vocab - 1)];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) {
                const int i = base + u * XRT_WAVE + lane;
                const float w = i < end ? weight(row.adjusted(min(i, vocab - 1), v[u])) : 0.f;
                const bool survives = i < end && order_key(row.adjusted(min(i, vocab - 1), v[u])) >= k_threshold;
                const unsigned long long mask = __ballot(survives);
                const int place = held + __popcll(mask & ((1ull << lane) - 1ull));
                if (survives && place < SEGMENT) {
                    survivor_id[wave * SEGMENT + place] = i;
                    survivor_weight[wave * SEGMENT + place] = w;
                }
                held += __popcll(mask);
            }
        }
        if (lane == 0) survivors_of[wave] = held;
        __syncthreads();
        bool fits = true;
        for (int w = 0; w < BLOCK_WAVES; ++w) fits = fits && survivors_of[w] <= SEGMENT;
        if (fits) {
            // this thread's two places in the list
            float mine[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int place = tid + h * THREADS;
                mine[h] = place % SEGMENT < survivors_of[place / SEGMENT] ? survivor_weight[place] : 0.f;
            }
            float w_threshold = 0.f;
            if (p < 1.0f) {
                float all[1] = {mine[0] + mine[1]};
                block_sums(all, scratch_f);
                const float need = p * all[0];
                unsigned low = 0u;
                for (int shift = 28; shift >= 0; shift -= 4) {
                    float mass[CANDIDATES];
#pragma unroll
                    for (int j = 0; j < CANDIDATES; ++j) {
                        const unsigned threshold = low | ((unsigned)(j + 1) << shift);
                        mass[j] = (__float_as_uint(mine[0]) >= threshold ? mine[0] : 0.f) +
                                  (__float_as_uint(mine[1]) >= threshold ? mine[1] : 0.f);
                    }
                    block_sums(mass, scratch_f);
                    unsigned digit = 0u;
#pragma unroll
                    for (int j = 0; j < CANDIDATES; ++j) if (mass[j] >= need) digit = (unsigned)(j + 1);
                    low |= digit << shift;
                }
                w_threshold = __uint_as_float(min(low, __float_as_uint(1.0f)));
            }
            if (tid == 0) {
                // the list is short: one thread adds it up, in the order of ids, and walks it to the target
                float total = 0.f;
                for (int w = 0; w < BLOCK_WAVES; ++w)
                    for (int j = 0; j < survivors_of[w]; ++j) {
                        const float x = survivor_weight[w * SEGMENT + j];
                        total += x >= w_threshold ? x : 0.f;
                    }
                const float target = uniforms[r] * total;
                float running = 0.f;
                int pick = -1, last_kept = -1;
                for (int w = 0; w < BLOCK_WAVES && pick < 0; ++w)
                    for (int j = 0; j < survivors_of[w] && pick < 0; ++j) {
                        const float x = survivor_weight[w * SEGMENT + j];
                        if (x >= w_threshold && x > 0.f) {
                            last_kept = survivor_id[w * SEGMENT + j];
                            running += x;
                            if (running > target) pick = last_kept;
                        }
                    }
                if (pick < 0) pick = last_kept;         // rounding at the end: the last kept token
                out.put(r, pick >= 0 ? pick : best_index); // sampler.rs:195: fall back to the top candidate
            }
            return;
        }
    }

    // ---- top-p: the largest weight threshold whose kept mass reaches p * total ------
    // Weights lie in [0, 1] and non-negative floats order like their bits: the same search, on
    // the weights' bits, with masses in place of counts. A mass over a smaller set is summed in
    // the same order over fewer terms, so the masses of the fifteen thresholds never rise.
    float w_threshold = 0.f;
    if (p < 1.0f) {
        float all[1] = {0.f};
        row.each([&](int, float v) { all[0] += weight(v); });
        block_sums(all, scratch_f);
        const float need = p * all[0];
        unsigned low = 0u;
        for (int shift = 28; shift >= 0; shift -= 4) {
            float mass[CANDIDATES];
#pragma unroll
            for (int j = 0; j < CANDIDATES; ++j) mass[j] = 0.f;
            row.each([&](int, float v) {
                const float w = weight(v);
                const unsigned bits = __float_as_uint(w);
#pragma unroll
                for (int j = 0; j < CANDIDATES; ++j) mass[j] += bits >= (low | ((unsigned)(j + 1) << shift)) ? w : 0.f;
            });
            block_sums(mass, scratch_f);
            unsigned digit = 0u;
#pragma unroll
            for (int j = 0; j < CANDIDATES; ++j) if (mass[j] >= need) digit = (unsigned)(j + 1);
            low |= digit << shift;
        }
        w_threshold = __uint_as_float(min(low, __float_as_uint(1.0f)));      // top_p 0 asks for nothing: the top weight alone
    }
    auto kept = [&](int i, float raw) -> float {
        const float w = weight(row.adjusted(i, raw));
        return w >= w_threshold ? w : 0.f;
    };

    // ---- inverse CDF over token ids ----------------------------------------------
    // Every wavefront owns a run of consecutive ids and reads it 64 ids at a time. First the mass
    // of every run; then the run in which the target falls is walked again with a running sum.
    float mine = 0.f;
    for (int base = begin; base < end; base += IN_FLIGHT * XRT_WAVE) {
        float v[IN_FLIGHT];
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; ++u) v[u] = row.logits[min(base + u * XRT_WAVE + lane, vocab - 1)];
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; ++u) {
            const int i = base + u * XRT_WAVE + lane;
            if (i < end) mine += kept(i, v[u]);
        }
    }
    mine = wave_sum(mine);
    if (lane == 0) wave_mass[wave] = mine;
    if (tid == 0) chosen = -1;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int w = 0; w < BLOCK_WAVES; ++w) total += wave_mass[w];
        const float target = uniforms[r] * total;
        float before = 0.f;
        int pick = -1, last = -1;
        for (int w = 0; w < BLOCK_WAVES && pick < 0; ++w) {
            if (wave_mass[w] > 0.f) {
                last = w;
                if (target < before + wave_mass[w]) { pick = w; break; }
                before += wave_mass[w];
            }
        }
        if (pick < 0) { pick = last; before -= last >= 0 ? wave_mass[last] : 0.f; }     // rounding at the very end: the last run with mass
        chosen_wave = pick;
        target_in_wave = target - before;
    }
    __syncthreads();
    if (wave == chosen_wave) {
        const float target = target_in_wave;
        float running = 0.f;                            // mass of the ids before the current 64
        int pick = -1, last_kept = -1;
        for (int outer = begin; outer < end && pick < 0; outer += IN_FLIGHT * XRT_WAVE) {
            float v[IN_FLIGHT];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) v[u] = row.logits[min(outer + u * XRT_WAVE + lane, vocab - 1)];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; ++u) {
                const int base = outer + u * XRT_WAVE;
                if (base >= end || pick >= 0) continue;     // uniform in the wavefront
                const int i = base + lane;
                const float w = i < end ? kept(i, v[u]) : 0.f;
                float through = w;                      // inclusive sum over the lanes, in lane order
#pragma unroll
                for (int offset = 1; offset < XRT_WAVE; offset <<= 1) {
                    const float below = __shfl_up(through, offset, XRT_WAVE);
                    if (lane >= offset) through += below;
                }
                const bool hit = w > 0.f && running + through > target;
                const unsigned long long hits = __ballot(hit);
                const unsigned long long kepts = __ballot(w > 0.f);
                if (hits != 0ull) pick = base + __builtin_ctzll(hits);
                if (kepts != 0ull) last_kept = base + 63 - __builtin_clzll(kepts);
                running += __shfl(through, XRT_WAVE - 1, XRT_WAVE);
            }
        }
        if (pick < 0) pick = last_kept;                 // rounding at the run's end: its last kept token
        if (lane == 0) chosen = pick;
    }
    __syncthreads();
    if (tid == 0) out.put(r, chosen >= 0 ? chosen : best_index);   // sampler.rs:195: fall back to the top candidate
}

__global__ void __launch_bounds__(THREADS) sample_kernel(
    const float* __restrict__ logits, int vocab, const Chosen out, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ history, const int* __restrict__ history_spans, const float* __restrict__ uniforms) {
    extern __shared__ unsigned seen[];                 // vocab bits
    sample_row(blockIdx.x, seen, logits, vocab, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms);
}

// ---- a small top-k: candidates by slice, then the row ---------------------------------------------
constexpr int SLICE = 4096;            // tokens of a slice
constexpr int SLICE_THREADS = 256;
constexpr int SLICE_WAVES = SLICE_THREADS / XRT_WAVE;
constexpr int SLICE_EACH = SLICE / SLICE_THREADS;
constexpr int SLICE_HOLDS = 128;       // candidates that a slice can hand on
constexpr int FAST_TOP_K = 64;         // the largest top-k that goes this way
constexpr int MOST_SLICES = (MAX_VOCAB + SLICE - 1) / SLICE;
constexpr int ROW_HOLDS = THREADS;     // survivors of the row's top-k that the row's workgroup can hold: one per thread

constexpr int SLICE_TOPS = 8;          // of a slice's largest values, one per thread that holds them, what it hands on apart
constexpr int LEAST_SLICES = 8;        // with fewer slices their tops are too few to bound a top-k of FAST_TOP_K

struct SliceCandidates {
    int count;                         // -1: this row does not go this way; more than SLICE_HOLDS: they did not fit;
                                       // -2: a row that takes the largest logit: `largest` is the slice's, `unused` its first index (0x7fffffff: none);
                                       // -3: a row that draws from all tokens (no top-k, no top-p): `largest` and `mass` only
    float largest, mass;               // for a row without top-k: the slice's largest value, and the sum of exp((value - largest) / temperature)
    int unused;
    unsigned top[SLICE_TOPS];          // keys of SLICE_TOPS different tokens of the slice, the largest first (0: none)
    int id[SLICE_HOLDS];
    float value[SLICE_HOLDS];          // after the penalty
};

// The top-k that a row takes through the slices; 0: it does not go this way. A row with a top-p but
// no top-k goes as if it had the largest top-k: when those candidates hold top-p's share of the whole
// row's mass (usual with a model's logits), top-p's threshold lies among them and the answer is exact;
// when they do not, the row's workgroup turns to the passes over the row.
__device__ __forceinline__ int top_k_by_slices(float temperature, int k, float p, int vocab) {
    if (!(temperature > 1e-5f) || vocab <= FAST_TOP_K) return 0;
    if (k > 0) return k <= FAST_TOP_K ? k : 0;
    return p < 1.0f ? FAST_TOP_K : 0;
}

// How many of the block's threads hold a larger maximum than this one (ties: lower thread first): the
// place of the thread's maximum among all. The thread in place k - 1 holds a lower bound of the k-th
// largest of all keys of the block (there are k keys at or above it, one in each of k threads); what
// lies at or above the bound is a short list, in which the exact place can then be looked for.
// `mine` is the thread's largest key (0: it holds none).
template <int THREADS_>
__device__ __forceinline__ int place_of_maximum(unsigned mine, unsigned* maxima) {
    maxima[threadIdx.x] = mine;
    __syncthreads();
    int larger = 0;
    for (int j = 0; j < THREADS_; j += 4) {
        const uint4 other = *reinterpret_cast<const uint4*>(&maxima[j]);
        larger += other.x > mine || (other.x == mine && j + 0 < (int)threadIdx.x) ? 1 : 0;
        larger += other.y > mine || (other.y == mine && j + 1 < (int)threadIdx.x) ? 1 : 0;
        larger += other.z > mine || (other.z == mine && j + 2 < (int)threadIdx.x) ? 1 : 0;
        larger += other.w > mine || (other.w == mine && j + 3 < (int)threadIdx.x) ? 1 : 0;
    }
    return larger;
}

__global__ void __launch_bounds__(SLICE_THREADS) sample_slices_kernel(
    const float* __restrict__ logits, int vocab, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ penalty, const int* __restrict__ history,
    const int* __restrict__ history_spans, SliceCandidates* __restrict__ candidates, int slices) {
    __shared__ unsigned seen[SLICE / 32];
    __shared__ __attribute__((aligned(16))) unsigned maxima[SLICE_THREADS];
    __shared__ unsigned bound;
    __shared__ float slice_largest, wave_mass[SLICE_WAVES];
    __shared__ int held;
    const int r = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
    SliceCandidates& mine = candidates[(long)r * slices + slice];
    const bool greedy = temperature[r] <= 1e-5f;                // the largest logit, first index: the slices' largest, then the first of those
    const int k = top_k_by_slices(temperature[r], top_k[r], top_p[r], vocab);
    // a temperature alone: the draw runs over all tokens; a slice hands on its mass and largest value, the row's
    // workgroup finds the slice in which the drawn number falls and walks that slice alone
    const bool whole = !greedy && top_k[r] == 0 && !(top_p[r] < 1.0f);
    if (k == 0 && !greedy && !whole) {
        if (tid == 0) mine.count = -1;
        return;
    }
    const int first = slice * SLICE;
    const float factor = penalty[r];
    const int h_begin = history_spans[2 * r], h_end = history_spans[2 * r + 1];
    const bool penalised = factor > 1.0f && h_end > h_begin;
    if (tid < SLICE / 32) seen[tid] = 0u;
    if (tid == 0) held = 0;
    __syncthreads();
    if (penalised) {
        for (int i = h_begin + tid; i < h_end; i += SLICE_THREADS) {
            const int token = history[i] - first;
            if (token >= 0 && token < SLICE && token + first < vocab) atomicOr(&seen[token >> 5], 1u << (token & 31));
        }
        __syncthreads();
    }
    // thread t holds tokens first + e * 256 + t
    float value[SLICE_EACH];
    unsigned key[SLICE_EACH];
    const float* row = logits + (long)r * vocab;
#pragma unroll
    for (int e = 0; e < SLICE_EACH; ++e) value[e] = row[min(first + e * SLICE_THREADS + tid, vocab - 1)];
#pragma unroll
    for (int e = 0; e < SLICE_EACH; ++e) {
        const int local = e * SLICE_THREADS + tid;
        const float v = value[e];
        const float changed = v > 0.f ? v / factor : v * factor;
        value[e] = (seen[local >> 5] >> (local & 31)) & 1u ? changed : v;
        // key 0 stands for "no token"; no float maps to it but a NaN with all bits set, which can go without loss
        key[e] = first + local < vocab ? order_key(value[e]) : 0u;
    }
    if (greedy) {
        // strict >, so NaN never wins (sampler.rs:83-98); a thread's tokens come in the order of their indices
        float best = -INFINITY;
        int best_index = 0x7fffffff;
#pragma unroll
        for (int e = 0; e < SLICE_EACH; ++e)
            if (key[e] != 0u && value[e] > best) { best = value[e]; best_index = first + e * SLICE_THREADS + tid; }
#pragma unroll
        for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) {
            const float other = __shfl_xor(best, offset, XRT_WAVE);
            const int other_index = __shfl_xor(best_index, offset, XRT_WAVE);
            if (other > best || (other == best && other_index < best_index)) { best = other; best_index = other_index; }
        }
        if (tid % XRT_WAVE == 0) { wave_mass[tid / XRT_WAVE] = best; maxima[tid / XRT_WAVE] = (unsigned)best_index; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < SLICE_WAVES; ++w) {
                const float other = wave_mass[w];
                const int other_index = (int)maxima[w];
                if (other > best || (other == best && other_index < best_index)) { best = other; best_index = other_index; }
            }
            mine.count = -2;
            mine.largest = best;
            mine.unused = best_index;
        }
        return;
    }
    unsigned largest = 0u;
    float largest_value = -INFINITY;
#pragma unroll
    for (int e = 0; e < SLICE_EACH; ++e) {
        if (key[e] > largest) { largest = key[e]; largest_value = value[e]; }
    }
    const int place = place_of_maximum<SLICE_THREADS>(largest, maxima);
    if (place == k - 1) bound = largest;                // 0 if fewer than k threads hold a token
    if (place < SLICE_TOPS) mine.top[place] = largest;
    if (place == 0) slice_largest = largest_value;
    __syncthreads();
    const unsigned threshold = bound;
    if (top_k[r] == 0) {
        // the slice's share of the row's mass, relative to its own largest value: threads add their tokens in
        // order, lanes in a tree, wavefronts in order
        const float inv_temp = 1.0f / temperature[r], top = slice_largest;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < SLICE_EACH; ++e) sum += key[e] != 0u && top > -INFINITY ? expf((value[e] - top) * inv_temp) : 0.f;   // (a slice of -inf alone has no mass)
        sum = wave_sum(sum);
        if (tid % XRT_WAVE == 0) wave_mass[tid / XRT_WAVE] = sum;
        __syncthreads();
        if (tid == 0) {
            float total = 0.f;
            for (int w = 0; w < SLICE_WAVES; ++w) total += wave_mass[w];
            mine.mass = total;
            mine.largest = top;
            if (whole) mine.count = -3;
        }
    }
    if (whole) return;
#pragma unroll
    for (int e = 0; e < SLICE_EACH; ++e) {
        if (key[e] != 0u && key[e] >= threshold) {
            const int at = atomicAdd(&held, 1);
            if (at < SLICE_HOLDS) {
                mine.id[at] = first + e * SLICE_THREADS + tid;
                mine.value[at] = value[e];
            }
        }
    }
    __syncthreads();
    if (tid == 0) mine.count = held;
}

__global__ void __launch_bounds__(THREADS) sample_candidates_kernel(
    const float* __restrict__ logits, int vocab, const Chosen out, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ history, const int* __restrict__ history_spans, const float* __restrict__ uniforms,
    const SliceCandidates* __restrict__ candidates, int slices) {
    extern __shared__ unsigned seen[];                 // vocab bits, for the rows that take the whole-row path
    __shared__ float scratch_f[(BLOCK_WAVES + 1) * SUMS];
    __shared__ int first_place[MOST_SLICES + 1];
    __shared__ unsigned bound, exact;
    __shared__ int kept_id[ROW_HOLDS];
    __shared__ float kept_value[ROW_HOLDS];
    __shared__ int sorted_id[ROW_HOLDS];
    __shared__ float sorted_weight[ROW_HOLDS];
    __shared__ int kept, survivors;
    __shared__ float row_mass;
    static_assert(MOST_SLICES <= XRT_WAVE, "one lane per slice");
    const int r = blockIdx.x, tid = threadIdx.x;
    const SliceCandidates* mine = candidates + (long)r * slices;
    // where every slice's candidates start in the row's list (one lane per slice; an inclusive sum over the
    // lanes); a slice that says "not this way" or "they did not fit" sends the row to the whole-row path
    if (temperature[r] <= 1e-5f) {                              // the largest logit: the largest of the slices', the first among equals
        if (tid < XRT_WAVE) {
            float best = tid < slices ? mine[tid].largest : -INFINITY;
            int best_index = tid < slices ? mine[tid].unused : 0x7fffffff;
#pragma unroll
            for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) {
                const float other = __shfl_xor(best, offset, XRT_WAVE);
                const int other_index = __shfl_xor(best_index, offset, XRT_WAVE);
                if (other > best || (other == best && other_index < best_index)) { best = other; best_index = other_index; }
            }
            if (tid == 0) out.put(r, best_index == 0x7fffffff ? 0 : best_index);   // nothing compared greater (all NaN or -inf): index 0
        }
        return;
    }
    if (mine[0].count == -3) {
        // A temperature alone: the inverse CDF over all tokens, in the order of ids (sampler.rs:147-164, :185-195). The
        // slices' masses say in which slice the drawn number falls; that slice's weights are worked out again, relative
        // to the row's largest value, and one wavefront walks them.
        __shared__ float whole_weight[SLICE];
        __shared__ unsigned whole_seen[SLICE / 32];
        __shared__ int whole_slice;
        __shared__ float whole_target, whole_best;
        const float inv_temp = 1.0f / temperature[r];
        if (tid < XRT_WAVE) {
            float best = tid < slices ? mine[tid].largest : -INFINITY;
#pragma unroll
            for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) best = fmaxf(best, __shfl_xor(best, offset, XRT_WAVE));
            const float share = tid < slices ? mine[tid].mass * expf((mine[tid].largest - best) * inv_temp) : 0.f;
            float total = 0.f;
            for (int j = 0; j < slices; ++j) total += __shfl(share, j, XRT_WAVE);
            const float target = uniforms[r] * total;
            float before = 0.f;
            int pick = -1, last = -1;
            for (int j = 0; j < slices && pick < 0; ++j) {      // every lane walks the same list
                const float x = __shfl(share, j, XRT_WAVE);
                if (x > 0.f) {
                    last = j;
                    if (target < before + x) pick = j; else before += x;
                }
            }
            if (pick < 0 && last >= 0) { pick = last; before -= __shfl(share, last, XRT_WAVE); }     // rounding at the very end: the last slice with mass
            if (tid == 0) { whole_slice = pick; whole_target = target - before; whole_best = best; }
        }
        if (tid < SLICE / 32) whole_seen[tid] = 0u;
        __syncthreads();
        const int slice = whole_slice;
        if (slice < 0) {                                        // no token has a weight (all -inf or NaN): the reference's fallback
            if (tid == 0) out.put(r, 0);
            return;
        }
        const int first = slice * SLICE;
        const float factor = penalty[r], best = whole_best;
        const int h_begin = history_spans[2 * r], h_end = history_spans[2 * r + 1];
        if (factor > 1.0f && h_end > h_begin) {
            for (int i = h_begin + tid; i < h_end; i += THREADS) {
                const int token = history[i] - first;
                if (token >= 0 && token < SLICE && token + first < vocab) atomicOr(&whole_seen[token >> 5], 1u << (token & 31));
            }
            __syncthreads();
        }
        const float* row = logits + (long)r * vocab;
        for (int local = tid; local < SLICE; local += THREADS) {
            const float v = row[min(first + local, vocab - 1)];
            const float changed = v > 0.f ? v / factor : v * factor;
            const float adjusted = (whole_seen[local >> 5] >> (local & 31)) & 1u ? changed : v;
            whole_weight[local] = first + local < vocab ? expf((adjusted - best) * inv_temp) : 0.f;
        }
        __syncthreads();
        if (tid < XRT_WAVE) {
            const float target = whole_target;
            float running = 0.f;
            int pick = -1, last_kept = -1;
            for (int base = 0; base < SLICE && pick < 0; base += XRT_WAVE) {
                const float w = whole_weight[base + tid];
                float through = w;                              // inclusive sum over the lanes, in lane order
#pragma unroll
                for (int offset = 1; offset < XRT_WAVE; offset <<= 1) {
                    const float below = __shfl_up(through, offset, XRT_WAVE);
                    if (tid >= offset) through += below;
                }
                const unsigned long long hits = __ballot(w > 0.f && running + through > target);
                const unsigned long long kepts = __ballot(w > 0.f);
                if (hits != 0ull) pick = base + __builtin_ctzll(hits);
                if (kepts != 0ull) last_kept = base + 63 - __builtin_clzll(kepts);
                running += __shfl(through, XRT_WAVE - 1, XRT_WAVE);
            }
            if (pick < 0) pick = last_kept;                     // rounding at the slice's end: its last token with a weight
            if (tid == 0) out.put(r, pick >= 0 ? first + pick : 0);
        }
        return;
    }
    const bool no_top_k = top_k[r] == 0;                        // a top-p alone: see top_k_by_slices
    const int k = no_top_k ? FAST_TOP_K : top_k[r];
    if (tid < XRT_WAVE) {
        const int count = tid < slices ? mine[tid].count : 0;
        const bool bad = count < 0 || count > SLICE_HOLDS;
        int through = max(count, 0);
#pragma unroll
        for (int offset = 1; offset < XRT_WAVE; offset <<= 1) {
            const int below = __shfl_up(through, offset, XRT_WAVE);
            if (tid >= offset) through += below;
        }
        if (tid < slices) first_place[tid + 1] = through;
        if (tid == 0) { first_place[0] = 0; kept = 0; survivors = 0; bound = 0u; }
        if (__ballot(bad) != 0ull) {
            if (tid == 0) first_place[0] = -1;
        } else {
            // A lower bound of the row's k-th largest key: the k-th largest of the slices' tops, which are all
            // different tokens. A lane holds two of them; `depth` per slice make at least FAST_TOP_K in all.
            const int depth = min(SLICE_TOPS, 2 * XRT_WAVE / slices);
            unsigned held[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int slot = tid + h * XRT_WAVE;
                held[h] = slot < slices * depth ? mine[slot / depth].top[slot % depth] : 0u;
            }
            int before[2] = {0, 0};                             // tops that come before this one (ties: lower slot first)
            for (int j = 0; j < XRT_WAVE; ++j) {
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const unsigned other = __shfl(held[g], j, XRT_WAVE);
                    const int other_slot = j + g * XRT_WAVE;
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        before[h] += other > held[h] || (other == held[h] && other_slot < tid + h * XRT_WAVE) ? 1 : 0;
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
                if (before[h] == k - 1) bound = held[h];        // 0 if fewer than k tops exist
        }
    }
    __syncthreads();
    if (first_place[0] < 0) {                                   // the same for all threads
        __syncthreads();
        sample_row(r, seen, logits, vocab, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms);
        return;
    }
    const int total = first_place[slices];
    // thread t holds candidates t, t + THREADS, ...: at most MOST_SLICES * SLICE_HOLDS / THREADS of them
    constexpr int EACH = (MOST_SLICES * SLICE_HOLDS + THREADS - 1) / THREADS;
    float value[EACH];
    int id[EACH];
    unsigned key[EACH];
#pragma unroll
    for (int e = 0; e < EACH; ++e) {
        const int place = e * THREADS + tid;
        key[e] = 0u; value[e] = 0.f; id[e] = 0;
        if (place < total) {
            int s = 0;
            while (first_place[s + 1] <= place) ++s;            // few slices; places of a wavefront share most of the walk
            const int within = place - first_place[s];
            value[e] = mine[s].value[within];
            id[e] = mine[s].id[within];
            key[e] = order_key(value[e]);
        }
    }
    // what lies at or above the lower bound of the k-th largest goes to a list ...
    const unsigned at_least = bound;
#pragma unroll
    for (int e = 0; e < EACH; ++e) {
        if (key[e] != 0u && key[e] >= at_least) {
            const int place = atomicAdd(&kept, 1);
            if (place < ROW_HOLDS) { kept_id[place] = id[e]; kept_value[place] = value[e]; }
        }
    }
    __syncthreads();
    const int listed = kept;
    if (listed > ROW_HOLDS) {                                   // ties by the thousand
        __syncthreads();
        sample_row(r, seen, logits, vocab, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms);
        return;
    }
    // ... in which the k-th largest is the one that k - 1 others come before (ties: lower id first); it and
    // all that tie with it stay, as on the whole row
    const unsigned my_key = tid < listed ? order_key(kept_value[tid]) : 0u;
    const int my_id = tid < listed ? kept_id[tid] : 0;
    if (tid < listed) {
        int before = 0;
        for (int j = 0; j < listed; ++j) {
            const unsigned other = order_key(kept_value[j]);
            before += other > my_key || (other == my_key && kept_id[j] < my_id) ? 1 : 0;
        }
        if (before == min(k, listed) - 1) exact = my_key;
    }
    __syncthreads();
    const bool survives = tid < listed && my_key >= exact;
    if (survives) atomicAdd(&survivors, 1);
    __syncthreads();
    const int n = survivors;
    // the survivors in the order of their ids: a survivor's place is the number of survivors with smaller ids
    float best = -INFINITY;
    for (int j = 0; j < listed; ++j) best = fmaxf(best, kept_value[j]);
    const float inv_temp = 1.0f / temperature[r];
    float weight = 0.f;
    if (survives) {
        int place = 0;
        for (int j = 0; j < listed; ++j) place += order_key(kept_value[j]) >= exact && kept_id[j] < my_id ? 1 : 0;
        weight = expf((kept_value[tid] - best) * inv_temp);
        sorted_id[place] = my_id;
        sorted_weight[place] = weight;
    }
    __syncthreads();
    const float p = top_p[r];
    if (no_top_k) {
        // The whole row's mass, from the slices (in their order), relative to the row's largest value. If the
        // candidates that stayed hold less than top-p's share of it, the threshold lies below them: the passes
        // over the row find it.
        if (tid < XRT_WAVE) {
            const float share = tid < slices ? mine[tid].mass * expf((mine[tid].largest - best) * inv_temp) : 0.f;
            float total = 0.f;
            for (int j = 0; j < slices; ++j) total += __shfl(share, j, XRT_WAVE);
            if (tid == 0) row_mass = total;
        }
        float stayed[1] = {weight};
        block_sums(stayed, scratch_f);                          // has a barrier before row_mass is read
        if (!(stayed[0] >= p * row_mass)) {
            __syncthreads();
            sample_row(r, seen, logits, vocab, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms);
            return;
        }
    }
    if (n <= XRT_WAVE) {
        // the usual case: one wavefront holds them all, lane j the j-th in the order of ids
        if (tid >= XRT_WAVE) return;
        const float w = tid < n ? sorted_weight[tid] : 0.f;
        float w_threshold = 0.f;
        if (p < 1.0f) {
            // the largest weight whose own and all larger weights together reach p of the total, sums in lane order
            float all = 0.f, with_larger = 0.f;
            for (int j = 0; j < n; ++j) {
                const float other = __shfl(w, j, XRT_WAVE);
                all += other;
                with_larger += other >= w ? other : 0.f;
            }
            const float need = p * (no_top_k ? row_mass : all);
            float reaches = tid < n && with_larger >= need ? w : 0.f;
#pragma unroll
            for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) reaches = fmaxf(reaches, __shfl_xor(reaches, offset, XRT_WAVE));
            w_threshold = fminf(reaches, 1.0f);
        }
        const float mine_kept = w >= w_threshold ? w : 0.f;
        float sum = 0.f;
        for (int j = 0; j < n; ++j) sum += __shfl(mine_kept, j, XRT_WAVE);
        const float target = uniforms[r] * sum;
        float running = 0.f;
        int pick = -1, last_kept = -1;
        for (int j = 0; j < n; ++j) {                           // every lane walks the same list: lane order is id order
            const float x = __shfl(mine_kept, j, XRT_WAVE);
            if (x > 0.f && pick < 0) {
                last_kept = j;
                running += x;
                if (running > target) pick = j;
            }
        }
        if (pick < 0) pick = last_kept;                         // rounding at the end: the last kept token
        if (tid == 0) out.put(r, sorted_id[pick]);                 // n >= 1: the largest candidate has weight 1
        return;
    }
    // top-p: the largest weight threshold whose kept mass reaches p * total, as on the whole row
    float w_threshold = 0.f;
    if (p < 1.0f) {
        float all[1] = {weight};
        block_sums(all, scratch_f);
        const float need = p * (no_top_k ? row_mass : all[0]);
        unsigned low = 0u;
        for (int shift = 28; shift >= 0; shift -= 4) {
            float mass[CANDIDATES];
#pragma unroll
            for (int j = 0; j < CANDIDATES; ++j) mass[j] = __float_as_uint(weight) >= (low | ((unsigned)(j + 1) << shift)) ? weight : 0.f;
            block_sums(mass, scratch_f);
            unsigned digit = 0u;
#pragma unroll
            for (int j = 0; j < CANDIDATES; ++j) if (mass[j] >= need) digit = (unsigned)(j + 1);
            low |= digit << shift;
        }
        w_threshold = __uint_as_float(min(low, __float_as_uint(1.0f)));
    }
    if (tid == 0) {
        float sum = 0.f;
        for (int j = 0; j < n; ++j) sum += sorted_weight[j] >= w_threshold ? sorted_weight[j] : 0.f;
        const float target = uniforms[r] * sum;
        float running = 0.f;
        int pick = -1, last_kept = -1;
        for (int j = 0; j < n && pick < 0; ++j) {
            const float x = sorted_weight[j];
            if (x >= w_threshold && x > 0.f) {
                last_kept = sorted_id[j];
                running += x;
                if (running > target) pick = last_kept;
            }
        }
        if (pick < 0) pick = last_kept;                         // rounding at the end: the last kept token
        out.put(r, pick);                                          // n >= 1: the largest candidate has weight 1
    }
}

}  // namespace

// Bytes of workspace with which small top-ks take the way through slices (0: the vocabulary is too small to gain).
extern "C" long xrt_sample_workspace(int rows, int vocab) {
    if (rows <= 0 || (vocab + SLICE - 1) / SLICE < LEAST_SLICES || vocab > MAX_VOCAB) return 0;
    return (long)rows * ((vocab + SLICE - 1) / SLICE) * (long)sizeof(SliceCandidates);
}

extern "C" int xrt_sample(const float* logits, int rows, int vocab, int* out, const float* temperature,
                          const int* top_k, const float* top_p, const float* penalty, int* history,
                          const int* history_spans, const int* append_at, const float* uniforms, void* workspace,
                          long workspace_bytes, void* stream) {
    XRT_REQUIRE(rows >= 0, "sample: negative row count");
    XRT_REQUIRE(vocab > 0, "sample: cannot sample from an empty logits vector");          // sampler.rs:56-60
    XRT_REQUIRE(vocab <= LARGEST_VOCAB, "sample: vocabulary %d exceeds %d", vocab, LARGEST_VOCAB);
    XRT_REQUIRE(logits && out && temperature && top_k && top_p && penalty && history_spans && uniforms,
                "sample: null operand");
    XRT_REQUIRE(append_at == nullptr || history != nullptr, "sample: tokens to append and no history to append them to");
    if (rows == 0) return 0;
    const Chosen chosen{out, history, append_at};
    const size_t lds = (size_t)((vocab + 31) / 32) * sizeof(unsigned);
    if (lds > 32 * 1024) {
        // a bitmap of seen tokens beyond what a kernel may take of LDS without asking
        static bool configured = false;
        if (!configured) {
            for (const void* kernel : {reinterpret_cast<const void*>(sample_kernel), reinterpret_cast<const void*>(sample_candidates_kernel)}) {
                hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LARGEST_VOCAB / 8);
                XRT_REQUIRE(e == hipSuccess, "sample: cannot reserve %d bytes of LDS: %s", LARGEST_VOCAB / 8, hipGetErrorString(e));
            }
            configured = true;
        }
    }
    const long need = xrt_sample_workspace(rows, vocab);
    if (workspace != nullptr && need > 0 && workspace_bytes >= need) {
        const int slices = (vocab + SLICE - 1) / SLICE;
        sample_slices_kernel<<<dim3(slices, rows), SLICE_THREADS, 0, (hipStream_t)stream>>>(
            logits, vocab, temperature, top_k, top_p, penalty, history, history_spans, (SliceCandidates*)workspace, slices);
        XRT_LAUNCH_CHECK("sample (slices)");
        sample_candidates_kernel<<<rows, THREADS, lds, (hipStream_t)stream>>>(
            logits, vocab, chosen, temperature, top_k, top_p, penalty, history, history_spans, uniforms,
            (const SliceCandidates*)workspace, slices);
        XRT_LAUNCH_CHECK("sample (candidates)");
        return 0;
    }
    sample_kernel<<<rows, THREADS, lds, (hipStream_t)stream>>>(logits, vocab, chosen, temperature, top_k, top_p,
                                                              penalty, history, history_spans, uniforms);
    XRT_LAUNCH_CHECK("sample");
    return 0;
}
