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
// Where the reference sorts, this kernel finds thresholds by bisection on the bit patterns
// (32 counting passes), so tokens that tie with the last kept one stay too; the CDF runs in
// the order of token ids.
#include "common.h"
#include "xrt_hip.h"

namespace {

constexpr int THREADS = 1024;
constexpr int MAX_VOCAB = 1 << 18;     // the seen-bitmap takes vocab/8 bytes of LDS (32 KiB at most)

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
    __device__ __forceinline__ float value(int i) const {
        float v = logits[i];
        if (penalised && ((seen[i >> 5] >> (i & 31)) & 1u)) v = v > 0.f ? v / penalty : v * penalty;
        return v;
    }
};

__device__ __forceinline__ unsigned block_sum_u32(unsigned v, unsigned* scratch) {
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
#pragma unroll
    for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, XRT_WAVE);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    unsigned total = 0;
    for (int w = 0; w < THREADS / XRT_WAVE; ++w) total += scratch[w];
    return total;
}

__global__ void __launch_bounds__(THREADS) sample_kernel(
    const float* __restrict__ logits, int vocab, int* __restrict__ out, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ history, const int* __restrict__ history_offsets, const float* __restrict__ uniforms) {
    extern __shared__ unsigned seen[];                 // vocab bits
    __shared__ float scratch_f[32];
    __shared__ unsigned scratch_u[32];
    __shared__ int scratch_i[32];
    __shared__ float chunk_sums[THREADS];
    __shared__ int chosen;

    const int r = blockIdx.x, tid = threadIdx.x;
    const int lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    Row row;
    row.logits = logits + (long)r * vocab;
    row.seen = seen;
    row.penalty = penalty[r];
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
    for (int i = tid; i < vocab; i += THREADS) {
        const float v = row.value(i);
        if (v > best) { best = v; best_index = i; }
    }
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
    for (int w = 1; w < THREADS / XRT_WAVE; ++w) {
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
    unsigned k_threshold = 0u;
    const int k = top_k[r];
    if (k > 0 && k < vocab) {
        unsigned low = 0u, high = 0xffffffffu;          // count(>= low) >= k always holds
        while (low < high) {
            const unsigned mid = low + (high - low) / 2u + 1u;
            unsigned count = 0;
            for (int i = tid; i < vocab; i += THREADS) count += order_key(row.value(i)) >= mid ? 1u : 0u;
            count = block_sum_u32(count, scratch_u);
            if (count >= (unsigned)k) low = mid; else high = mid - 1u;
        }
        k_threshold = low;
    }
    auto weight = [&](int i) -> float {
        const float v = row.value(i);
        return order_key(v) >= k_threshold ? expf((v - best) * inv_temp) : 0.f;
    };

    // ---- top-p: the largest weight threshold whose kept mass reaches p * total ------
    float w_threshold = 0.f;
    const float p = top_p[r];
    if (p < 1.0f) {
        float total = 0.f;
        for (int i = tid; i < vocab; i += THREADS) total += weight(i);
        total = block_sum(total, scratch_f);
        const float need = p * total;
        unsigned low = 0u, high = __float_as_uint(1.0f); // weights lie in [0, 1]; non-negative floats order like their bits
        while (low < high) {
            const unsigned mid = low + (high - low) / 2u + 1u;
            const float threshold = __uint_as_float(mid);
            float mass = 0.f;
            for (int i = tid; i < vocab; i += THREADS) { const float w = weight(i); mass += w >= threshold ? w : 0.f; }
            mass = block_sum(mass, scratch_f);
            if (mass >= need) low = mid; else high = mid - 1u;
        }
        w_threshold = __uint_as_float(low);
    }

    // ---- inverse CDF over token ids ----------------------------------------------
    const int chunk = (vocab + THREADS - 1) / THREADS;
    const int begin = min(vocab, tid * chunk), end = min(vocab, begin + chunk);
    float mine = 0.f;
    for (int i = begin; i < end; ++i) { const float w = weight(i); mine += w >= w_threshold ? w : 0.f; }
    chunk_sums[tid] = mine;
    if (tid == 0) chosen = -1;
    __syncthreads();
    if (tid == 0) {
        float running = 0.f;
        for (int t = 0; t < THREADS; ++t) { const float s = chunk_sums[t]; chunk_sums[t] = running; running += s; }
        scratch_f[0] = running;
    }
    __syncthreads();
    const float total = scratch_f[0];
    const float target = uniforms[r] * total;
    const float before = chunk_sums[tid];
    if (mine > 0.f && before <= target && target < before + mine) {
        float running = before;
        int pick = -1;
        for (int i = begin; i < end && pick < 0; ++i) {
            const float w = weight(i);
            if (w >= w_threshold && w > 0.f) {
                running += w;
                if (running > target) pick = i;
            }
        }
        if (pick < 0)                                   // rounding at the chunk's end: its last kept token
            for (int i = end - 1; i >= begin && pick < 0; --i) { const float w = weight(i); if (w >= w_threshold && w > 0.f) pick = i; }
        atomicMax(&chosen, pick);
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
