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
#include "common.h"
#include "xrt_hip.h"

namespace {

constexpr int THREADS = 1024;
constexpr int BLOCK_WAVES = THREADS / XRT_WAVE;
constexpr int IN_FLIGHT = 16;          // loads of a thread that a pass keeps in flight
constexpr int MAX_VOCAB = 255 * THREADS;   // a thread sees at most 255 tokens (8-bit counters below); the seen-bitmap takes vocab/8 bytes of LDS
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
template <typename T, int N>
__device__ __forceinline__ void block_sums(T (&v)[N], T* scratch) {
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

__global__ void __launch_bounds__(THREADS) sample_kernel(
    const float* __restrict__ logits, int vocab, int* __restrict__ out, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ history, const int* __restrict__ history_offsets, const float* __restrict__ uniforms) {
    extern __shared__ unsigned seen[];                 // vocab bits
    __shared__ float scratch_f[(BLOCK_WAVES + 1) * SUMS];
    __shared__ unsigned scratch_u[(BLOCK_WAVES + 1) * SUMS];
    __shared__ int survivor_id[BLOCK_WAVES * SEGMENT];      // what top-k leaves, by wavefront run, in the order of ids
    __shared__ float survivor_weight[BLOCK_WAVES * SEGMENT];
    __shared__ int survivors_of[BLOCK_WAVES];
    __shared__ int scratch_i[BLOCK_WAVES];
    __shared__ float wave_mass[BLOCK_WAVES];
    __shared__ float target_in_wave;
    __shared__ int chosen_wave, chosen;

    const int r = blockIdx.x, tid = threadIdx.x;
    const int lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    Row row;
    row.logits = logits + (long)r * vocab;
    row.seen = seen;
    row.penalty = penalty[r];
    row.vocab = vocab;
    const int h_begin = history_offsets[r], h_end = history_offsets[r + 1];
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
        if (tid == 0) out[r] = best_index;
        return;
    }
    const float inv_temp = 1.0f / temp;

    // ---- top-k: the largest key T with count(key >= T) >= k ---------------------
    // Found four bits at a time from the top. With the bits above already fixed in `low`, a pass
    // counts, among the keys that share those bits, how many have each value of the next four
    // (sixteen 8-bit counters packed into two registers: a thread sees at most 255 keys), and
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
            });
            unsigned count[SUMS];
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                count[d] = (unsigned)(packed_low >> (d * 8)) & 255u;
                count[8 + d] = (unsigned)(packed_high >> (d * 8)) & 255u;
            }
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
                out[r] = pick >= 0 ? pick : best_index; // sampler.rs:195: fall back to the top candidate
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
    if (tid == 0) out[r] = chosen >= 0 ? chosen : best_index;   // sampler.rs:195: fall back to the top candidate
}

}  // namespace

extern "C" int xrt_sample(const float* logits, int rows, int vocab, int* out, const float* temperature,
                          const int* top_k, const float* top_p, const float* penalty, const int* history,
                          const int* history_offsets, const float* uniforms, void* stream) {
    XRT_REQUIRE(rows >= 0, "sample: negative row count");
    XRT_REQUIRE(vocab > 0, "sample: cannot sample from an empty logits vector");          // sampler.rs:56-60
    XRT_REQUIRE(vocab <= MAX_VOCAB, "sample: vocabulary %d exceeds %d", vocab, MAX_VOCAB);
    XRT_REQUIRE(logits && out && temperature && top_k && top_p && penalty && history_offsets && uniforms,
                "sample: null operand");
    if (rows == 0) return 0;
    const size_t lds = (size_t)((vocab + 31) / 32) * sizeof(unsigned);
    sample_kernel<<<rows, THREADS, lds, (hipStream_t)stream>>>(logits, vocab, out, temperature, top_k, top_p,
                                                              penalty, history, history_offsets, uniforms);
    XRT_LAUNCH_CHECK("sample");
    return 0;
}
