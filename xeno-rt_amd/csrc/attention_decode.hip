// Decode attention on the matrix cores: every sequence brings one query token; its keys and
// values are read once from the cache, in chunks spread over many wavefronts, and applied to
// all query heads of a key/value head together.
//
// Formulas: crates/xrt-models/src/llama.rs:504-574 of the reference (score = q.k * scale over
// keys 0..pos, online softmax with running maximum and sum, weighted sum of values, division
// by the sum); query head h uses key/value head h / group.
//
// One wavefront takes one chunk of keys of one (token, key/value head, tile of 16 query
// heads). Scores: S[key][head] = K Q^T with v_mfma_f32_16x16x32_bf16, keys as rows (A operand),
// the query heads as columns. Values: O[dim][head] += V^T P, with the transposed value block
// as A operand and the probabilities, still in the registers the scores came in, as B
// operand: key rows are assigned to accumulator rows such that every lane ends up holding
// eight consecutive keys, exactly the K slots of the next product. A cache block lies in
// memory in the order of these operands (cache_layout.h): every load instruction takes one
// contiguous kilobyte, which nobody else reads, and passes the caches by (non-temporal; with
// keys as rows of head_dim elements an instruction took half a line of each of 16 keys and the
// kernel read 6.1 TB/s where it now reads 6.9). A block's values are asked for before its
// scores are computed, the next block's keys right after. The four wavefronts of a workgroup
// merge their results (maximum, sum, O) through LDS into one partial result; a second kernel
// merges the partial results of a token, in order.
//
// The kernel can also finish what follows the q/k/v projection (xrt_qkv_finish: the RMSNorm of every head of q and k,
// the rotation, the write of the new key and value into the cache), so that a decode step of a model with head
// norms needs no kernel between the projection and the attention. The formulas and their order are those of
// qkv_prepare.hip (crates/xrt-models/src/llama.rs:1025-1040, crates/xrt-kernels/src/cpu/rope.rs:59-89). A lane holds
// the dims 32 s + 8 c .. + 7 (s = 0 .. HD/32 - 1) of its query head, so the two dims of a rotation's pair (d and
// d + HD/2) lie in one lane, and the norm's sum over a head is an exchange among four lanes. The new key and
// value are worked out by the wavefront whose keys end with the sequence's newest block: it puts them into the
// registers in which the block came from the cache (where the place of the newest token still holds what was
// there before) and writes them to the cache for the steps to come.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

struct Finish {                       // xrt_qkv_finish with its pointers typed
    const void* q_norm; const void* k_norm; int norm_dtype; float norm_eps;
    const float2* rope_table; int table_positions;     // (cosine, sine) of the positions' angles, [position][pair]; null: no rotation
    bf16* k_cache; bf16* v_cache;
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVES = 4;
constexpr float LOG2E = 1.4426950408889634f;

// Row r of score tile t (0 or 1) of a group of 32 keys stands for key 8 (r / 4) + 4 t + r % 4: accumulator
// register i of lane group c is row 4 c + i, and must be key 8 c + 4 t + i. The cache keeps the keys so:
// lane (r, c) finds its piece of tile ((g * 2 + t) * KS + s) at place r + 16 c, and of the values' tile
// (g * DT + u) likewise.
constexpr int lane_place(int r, int c) { return (r + 16 * c) * 8; }
static_assert(cache_key_offset(32 + 8 * 2 + 4 * 1 + 3, 32 * 3 + 8 * 1, 128) == ((1 * 2 + 1) * 4 + 3) * 512 + lane_place(2 * 4 + 3, 1), "keys of a block");
static_assert(cache_key_offset(8 * 3 + 4 * 0 + 1, 32 * 1 + 8 * 3 + 5, 64) == ((0 * 2 + 0) * 2 + 1) * 512 + lane_place(3 * 4 + 1, 3) + 5, "keys of a block");
static_assert(cache_value_offset(16 * 5 + 9, 32 + 8 * 2 + 6, 128) == (1 * 8 + 5) * 512 + lane_place(9, 2) + 6, "values of a block");

// One head (the dims of this lane: 32 s + 8 c .. + 7) through its RMSNorm (weight `gain`, null: none) and the rotation
// by the token's position, in float32, and back to bfloat16: what qkv_prepare does to a head.
// turns: the (cosine, sine) of this position's HD / 2 angles, as xrt_rope_table has worked them out (the same sincosf of the
// same angles as in qkv_prepare.hip: worked out here, for every workgroup again, they would cost more than the kernel saves);
// null: no rotation.
template <int HD, typename TW>
__device__ __forceinline__ void finish_head(bf16x8 (&x)[HD / 32], const TW* __restrict__ gain, float eps,
                                            const float2* __restrict__ turns, int c) {
    constexpr int KS = HD / 32;
    float inv_rms = 1.0f;
    if (gain != nullptr) {
        float squares = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) squares = fmaf((float)x[ks][e], (float)x[ks][e], squares);
        squares += __shfl_xor(squares, 16, XRT_WAVE);          // the four lanes (r, 0 .. 3) hold the head between them
        squares += __shfl_xor(squares, 32, XRT_WAVE);
        inv_rms = 1.0f / sqrtf(squares / (float)HD + eps);
    }
    // a pair of the rotation at a time (dims d and d + HD / 2 lie in x[ks] and x[ks + KS / 2]): few registers at once
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) {
        float lower[8], upper[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { lower[e] = (float)x[ks][e]; upper[e] = (float)x[ks + KS / 2][e]; }
        if (gain != nullptr) {
            struct alignas(sizeof(TW) * 8) Eight { TW e[8]; };
            const Eight of_lower = *reinterpret_cast<const Eight*>(gain + ks * 32 + c * 8);
            const Eight of_upper = *reinterpret_cast<const Eight*>(gain + (ks + KS / 2) * 32 + c * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                lower[e] = lower[e] * inv_rms * to_float(of_lower.e[e]);
                upper[e] = upper[e] * inv_rms * to_float(of_upper.e[e]);
            }
        }
        if (turns != nullptr) {
            struct alignas(16) Pairs { float2 e[8]; };
            const Pairs read = *reinterpret_cast<const Pairs*>(turns + ks * 32 + c * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float cosine = read.e[e].x, sine = read.e[e].y;
                const float a = lower[e], b = upper[e];
                lower[e] = a * cosine - b * sine;
                upper[e] = a * sine + b * cosine;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) { x[ks][e] = (bf16)lower[e]; x[ks + KS / 2][e] = (bf16)upper[e]; }
    }
}

// FINISH: q, k and v come as the projection left them, and `finish` says what is still to do (see the head of this file).
template <int HD, bool FINISH>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, 2) attention_decode_kernel(
    const bf16* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads,
    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ positions, const int* __restrict__ slots,
    float scale, int chunk_blocks, int n_parts, int q_tiles,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16* __restrict__ out, const Finish finish) {
    constexpr int KS = HD / 32;                    // K steps of the score product
    constexpr int DT = HD / 16;                    // 16-row tiles of the value product
    __shared__ floatx4 merge_o[WAVES][DT][XRT_WAVE];
    __shared__ float merge_ml[WAVES][2][16];

    const int lane = threadIdx.x % XRT_WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / XRT_WAVE);   // in a scalar register, and with it the blocks' numbers
    const int r = lane % 16, c = lane / 16;
    const int part = blockIdx.x;                   // this workgroup's four chunks become one partial result
    const int chunk = part * WAVES + wave;
    const int kv_head = blockIdx.y / q_tiles, q_tile = blockIdx.y % q_tiles;
    const int token = blockIdx.z;
    const int slot = slots[token];
    const int group = n_heads / n_kv_heads;
    if (slot < 0) {                                // padding: the whole workgroup leaves
        // (with one partial result per head there is no merge kernel after this one to write the zeros)
        if (n_parts == 1 && wave == 0 && q_tile * 16 + r < group) {
            bf16* dst = out + ((long)token * n_heads + kv_head * group + q_tile * 16 + r) * HD;
            for (int d = c; d < HD; d += 4) dst[d] = (bf16)0.f;
        }
        return;
    }
    const int n_keys = positions[token] + 1;
    if (part * WAVES * chunk_blocks * XRT_BLOCK_TOKENS >= n_keys) return;      // nothing here for any wavefront
    const int first_block = chunk * chunk_blocks;
    const bool active = first_block * XRT_BLOCK_TOKENS < n_keys;
    const int last_block = min((n_keys - 1) / XRT_BLOCK_TOKENS, first_block + chunk_blocks - 1);
    const int head_in_group = q_tile * 16 + r;             // this lane's query head (column of the products)
    const bool head_valid = head_in_group < group;
    const int head = kv_head * group + min(head_in_group, group - 1);

    const float scale2 = scale * LOG2E;                    // scores are kept in units of log2
    float m = -INFINITY, l = 0.f;
    floatx4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    if (active) {
        bf16x8 q[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            q[ks] = *reinterpret_cast<const bf16x8*>(qkv + (long)token * row_width + (long)head * HD + ks * 32 + c * 8);
        // The sequence's newest token: its block and its place there. What is still to do to q (and, in the wavefront whose
        // keys end with the newest block, to the new key) is done before the first keys are asked for: behind their loads
        // it would wait for them, and with a block's keys and values in registers there is no room for it.
        const int newest_block = (n_keys - 1) / XRT_BLOCK_TOKENS, newest = (n_keys - 1) % XRT_BLOCK_TOKENS;
        const bool has_newest = FINISH && last_block == newest_block;
        bf16x8 new_key[KS];
        bf16 new_value[DT];
        if constexpr (FINISH) {
            const int pos = n_keys - 1;
            const float2* turns = finish.rope_table != nullptr ? finish.rope_table + (long)min(pos, finish.table_positions - 1) * (HD / 2) : nullptr;   // (the host sends only steps that the table covers)
            if (has_newest) {                          // (the same for all lanes of the wavefront)
                const bf16* key_row = qkv + (long)token * row_width + (long)(n_heads + kv_head) * HD;
                const bf16* value_row = key_row + (long)n_kv_heads * HD;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) new_key[ks] = *reinterpret_cast<const bf16x8*>(key_row + ks * 32 + c * 8);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) new_value[dt] = value_row[dt * 16 + r];
            }
            if (finish.norm_dtype == XRT_F32)
                finish_head<HD>(q, (const float*)finish.q_norm, finish.norm_eps, turns, c);
            else
                finish_head<HD>(q, (const bf16*)finish.q_norm, finish.norm_eps, turns, c);
            if (has_newest) {
                if (finish.norm_dtype == XRT_F32)
                    finish_head<HD>(new_key, (const float*)finish.k_norm, finish.norm_eps, turns, c);
                else
                    finish_head<HD>(new_key, (const bf16*)finish.k_norm, finish.norm_eps, turns, c);
            }
        }
        // Loads are always on their way: a block's values are asked for before its scores are computed, and the
        // next block's keys right after, before the softmax and the value product of this one.
        const int* table = block_table + (long)slot * table_stride;
        auto block_of = [&](int b) { return min(max(table[min(b, last_block)], 0), n_blocks - 1); };   // the host never hands out anything else
        bf16x8 kreg[2][2][KS], vreg[2][DT];
        auto ask_keys = [&](int block) {
            const bf16* kb = k_cache + ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * HD;
#pragma unroll
            for (int g = 0; g < 2; ++g)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        kreg[g][t][ks] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(kb + ((g * 2 + t) * KS + ks) * 512 + lane * 8));
        };
        int block = block_of(first_block), next_block = block_of(first_block + 1);
        ask_keys(block);
        for (int b = first_block; b <= last_block; ++b) {
            const bf16* vb = v_cache + ((long)block * n_kv_heads + kv_head) * HD * XRT_BLOCK_TOKENS;
            const int valid = min(XRT_BLOCK_TOKENS, n_keys - b * XRT_BLOCK_TOKENS);   // keys of this block that exist
#pragma unroll
            for (int g = 0; g < 2; ++g)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    vreg[g][dt] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(vb + (g * DT + dt) * 512 + lane * 8));

            if constexpr (FINISH) {
                if (has_newest && b == newest_block) {
                    // The newest key and value take their places in the registers that hold the block (key 32 g + 8 (r / 4) +
                    // 4 t + r % 4 lies in lane r of kreg[g][t], token 32 g + 8 c + e in element e of vreg[g] of the lanes c),
                    // and in the cache (one of the workgroups that share the key/value head writes: q_tile 0).
                    const int g_new = newest / 32, within = newest % 32;
                    const int t_new = within % 8 / 4, r_new = within / 8 * 4 + within % 4, c_new = within / 8, e_new = newest % 8;
#pragma unroll
                    for (int g = 0; g < 2; ++g) {
                        if (g != g_new) continue;
#pragma unroll
                        for (int t = 0; t < 2; ++t)
                            if (t == t_new && r == r_new) {
#pragma unroll
                                for (int ks = 0; ks < KS; ++ks) kreg[g][t][ks] = new_key[ks];
                            }
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (e == e_new && c == c_new) {
#pragma unroll
                                for (int dt = 0; dt < DT; ++dt) vreg[g][dt][e] = new_value[dt];
                            }
                    }
                    if (q_tile == 0) {
                        const long base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * HD;
                        if (r == 0) {
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks)
                                *reinterpret_cast<bf16x8*>(finish.k_cache + base + cache_key_offset(newest, ks * 32 + c * 8, HD)) = new_key[ks];
                        }
                        if (c == 0) {
#pragma unroll
                            for (int dt = 0; dt < DT; ++dt) finish.v_cache[base + cache_value_offset(dt * 16 + r, newest, HD)] = new_value[dt];
                        }
                    }
                }
            }
            // ---- scores of 64 keys: two groups of 32, two tiles of 16 rows each
            floatx4 s[2][2];
#pragma unroll
            for (int g = 0; g < 2; ++g)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    s[g][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        s[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[g][t][ks], q[ks], s[g][t], 0, 0, 0);
                }
            block = next_block;
            next_block = block_of(b + 2);
            if (b < last_block) ask_keys(block);
            // register i of s[g][t] is key g*32 + c*8 + t*4 + i, for query head r
            float block_max = -INFINITY;
#pragma unroll
            for (int g = 0; g < 2; ++g)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = g * 32 + c * 8 + t * 4 + i;
                        const float v = key < valid ? s[g][t][i] * scale2 : -INFINITY;   // also drops whatever lies past the end
                        s[g][t][i] = v;
                        block_max = fmaxf(block_max, v);
                    }
            block_max = fmaxf(block_max, __shfl_xor(block_max, 16, XRT_WAVE));
            block_max = fmaxf(block_max, __shfl_xor(block_max, 32, XRT_WAVE));
            const float m_new = fmaxf(m, block_max);           // finite: key 0 of the block exists
            const float correction = __builtin_amdgcn_exp2f(m - m_new);
            m = m_new;
            l *= correction;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] *= correction;

            // ---- probabilities, and the value product
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                bf16x8 p;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float e = __builtin_amdgcn_exp2f(s[g][t][i] - m_new);
                        l += e;
                        p[t * 4 + i] = (bf16)e;
                    }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    bf16x8 v = vreg[g][dt];
                    if (valid < XRT_BLOCK_TOKENS) {
                        // the block's tail belongs to nobody: whatever it holds must not meet the zeros of p
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (g * 32 + c * 8 + e >= valid) v[e] = (bf16)0.f;
                    }
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, p, o[dt], 0, 0, 0);
                }
            }
        }
        l += __shfl_xor(l, 16, XRT_WAVE);
        l += __shfl_xor(l, 32, XRT_WAVE);
    }

    // ---- the four wavefronts' results become one, in wavefront order
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) merge_o[wave][dt][lane] = o[dt];
    if (c == 0) {
        merge_ml[wave][0][r] = m;                  // -inf for a wavefront without keys
        merge_ml[wave][1][r] = l;
    }
    __syncthreads();
    if (wave == 0 && head_valid) {
        float m_all = merge_ml[0][0][r];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) m_all = fmaxf(m_all, merge_ml[w][0][r]);
        float l_all = 0.f;
        floatx4 total[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) total[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float weight = __builtin_amdgcn_exp2f(merge_ml[w][0][r] - m_all);     // 0 for a wavefront without keys
            l_all += weight * merge_ml[w][1][r];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) total[dt] += merge_o[w][dt][lane] * weight;
        }
        if (n_parts == 1) {
            // the workgroup has seen all keys of the sequence: this is the result, and no merge kernel follows
            const float inv = l_all > 0.f ? 1.0f / l_all : 0.f;
            bf16* final_row = out + ((long)token * n_heads + head) * HD;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                struct alignas(8) Four { bf16 e[4]; } four;
#pragma unroll
                for (int i = 0; i < 4; ++i) four.e[i] = (bf16)(total[dt][i] * inv);
                *reinterpret_cast<Four*>(final_row + dt * 16 + c * 4) = four;
            }
            return;
        }
        const long index = ((long)token * n_heads + head) * n_parts + part;
        float* dst = part_o + index * HD;
        // accumulator register i of tile dt is dimension dt*16 + c*4 + i, for query head r
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<floatx4*>(dst + dt * 16 + c * 4) = total[dt];
        if (c == 0) {
            part_ml[index * 2] = m_all;
            part_ml[index * 2 + 1] = l_all;
        }
    }
}

// Merges the partial results of one (token, head): out = sum_k w_k O_k / sum_k w_k l_k with
// w_k = 2^(m_k - max m), in order. One thread per dimension. The weights are worked out once,
// by one thread per partial result, and shared through LDS; maximum and sum are wavefront
// reductions in a fixed order.
template <int HD>
__global__ void __launch_bounds__(HD) attention_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ positions,
    const int* __restrict__ slots, int n_heads, int part_keys, int n_parts, bf16* __restrict__ out) {
    extern __shared__ float weights[];                    // n_parts
    __shared__ float reduce[HD / XRT_WAVE][2];
    const int token = blockIdx.y, head = blockIdx.x, d = threadIdx.x;
    const int lane = d % XRT_WAVE, wave = d / XRT_WAVE;
    bf16* dst = out + ((long)token * n_heads + head) * HD;
    const long base = ((long)token * n_heads + head) * n_parts;
    const float* column = part_o + base * HD + d;
    // Everything this thread may need is asked for at once, before it is known how many partial
    // results count: the loads then cost one trip to memory instead of one after the other.
    // What lies beyond the partial results that count is read (it is inside the workspace) and
    // never used.
    constexpr int EARLY = 16;
    float early_o[EARLY];
#pragma unroll
    for (int k = 0; k < EARLY; ++k) early_o[k] = k < n_parts ? column[(long)k * HD] : 0.f;
    const float2 early_ml = d < n_parts ? *reinterpret_cast<const float2*>(part_ml + (base + d) * 2) : make_float2(0.f, 0.f);
    const int slot = slots[token];
    const int n_keys = positions[token] + 1;
    if (slot < 0) {
        dst[d] = (bf16)0.f;
        return;
    }
    const int parts = min(n_parts, (n_keys + part_keys - 1) / part_keys);
    float m = d < parts ? early_ml.x : -INFINITY;
    for (int k = d + HD; k < parts; k += HD) m = fmaxf(m, part_ml[(base + k) * 2]);
    m = wave_max(m);
    if (lane == 0) reduce[wave][0] = m;
    __syncthreads();
    m = reduce[0][0];
#pragma unroll
    for (int w = 1; w < HD / XRT_WAVE; ++w) m = fmaxf(m, reduce[w][0]);
    float l = 0.f;
    if (d < parts) {
        const float weight = __builtin_amdgcn_exp2f(early_ml.x - m);
        weights[d] = weight;
        l = weight * early_ml.y;
    }
    for (int k = d + HD; k < parts; k += HD) {
        const float weight = __builtin_amdgcn_exp2f(part_ml[(base + k) * 2] - m);
        weights[k] = weight;
        l = fmaf(weight, part_ml[(base + k) * 2 + 1], l);
    }
    l = wave_sum(l);
    if (lane == 0) reduce[wave][1] = l;
    __syncthreads();
    l = reduce[0][1];
#pragma unroll
    for (int w = 1; w < HD / XRT_WAVE; ++w) l += reduce[w][1];
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < EARLY; ++k)
        if (k < parts) acc = fmaf(weights[k], early_o[k], acc);
#pragma unroll 8
    for (int k = EARLY; k < parts; ++k) acc = fmaf(weights[k], column[(long)k * HD], acc);
    dst[d] = (bf16)(l > 0.f ? acc / l : 0.f);
}

// How the keys of the longest sequence are cut: blocks per wavefront, and partial results
// (each from the four wavefronts of a workgroup) per (token, head).
struct Cut { int chunk_blocks, n_parts; };

Cut cut_for(int tokens, int n_kv_heads, int q_tiles, int max_context, int head_dim) {
    const int max_blocks = (max_context + XRT_BLOCK_TOKENS - 1) / XRT_BLOCK_TOKENS;
    // How long the kernel takes is set by the compute unit with the most to do: workgroups are dealt out to
    // the 256 compute units in turn, and a compute unit works off its share at its own pace (two workgroups
    // at a time are no faster than one after the other). Measured at head size 128: 6.3 us for a block of 64
    // keys per wavefront, 0.7 us per workgroup, about 5 us for the merge kernel. So the cut is chosen for
    // the fewest blocks per compute unit: 384 workgroups of 16 blocks (two on every second compute unit) are
    // slower than 768 of 8. The longer chunk wins among equals (less to merge); with one workgroup per (token,
    // key/value head) pair nothing is left to merge and the merge kernel is not launched.
    const long pairs = (long)tokens * n_kv_heads * q_tiles;
    const long block_ns = 6300L * head_dim / 128, group_ns = 700, merge_ns = 5000;
    const int longest = (max_blocks + WAVES - 1) / WAVES;
    long best_ns = -1;
    Cut best{longest, 1};
    for (int chunk_blocks = longest; chunk_blocks >= 1; --chunk_blocks) {
        const int n_chunks = (max_blocks + chunk_blocks - 1) / chunk_blocks;
        const int n_parts = (n_chunks + WAVES - 1) / WAVES;
        if ((long)(n_parts - 1) * WAVES * chunk_blocks >= max_blocks) continue;         // a part without keys: a shorter chunk does the same
        const long per_unit = (pairs * n_parts + XRT_COMPUTE_UNITS - 1) / XRT_COMPUTE_UNITS;
        const long ns = per_unit * (chunk_blocks * block_ns + group_ns) + (n_parts > 1 ? merge_ns : 0);
        if (best_ns < 0 || ns < best_ns) { best_ns = ns; best = Cut{chunk_blocks, n_parts}; }
    }
    return best;
}

template <int HD>
int launch(const bf16* qkv, int tokens, int n_heads, int n_kv_heads, const bf16* k_cache, const bf16* v_cache,
           const int* block_table, int table_stride, int n_blocks, const int* positions, const int* slots, bf16* out,
           float scale, int max_context, float* workspace, long workspace_floats, const Finish* finish, hipStream_t s) {
    const int group = n_heads / n_kv_heads;
    const int q_tiles = (group + 15) / 16;
    const Cut cut = cut_for(tokens, n_kv_heads, q_tiles, max_context, HD);
    const long need = cut.n_parts == 1 ? 0 : (long)tokens * n_heads * cut.n_parts * (HD + 2);
    XRT_REQUIRE(need == 0 || (workspace != nullptr && workspace_floats >= need),
                "attention (decode): workspace of %ld floats given, %ld needed", workspace_floats, need);
    float* part_o = workspace;
    float* part_ml = workspace + (long)tokens * n_heads * cut.n_parts * HD;
    const int row_width = (n_heads + 2 * n_kv_heads) * HD;
    XRT_REQUIRE(tokens <= 65535 && n_kv_heads * q_tiles <= 65535, "attention (decode): grid too large");
    const dim3 grid(cut.n_parts, n_kv_heads * q_tiles, tokens);
    if (finish != nullptr)
        attention_decode_kernel<HD, true><<<grid, WAVES * XRT_WAVE, 0, s>>>(
            qkv, row_width, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks, positions, slots,
            scale, cut.chunk_blocks, cut.n_parts, q_tiles, part_o, part_ml, out, *finish);
    else
        attention_decode_kernel<HD, false><<<grid, WAVES * XRT_WAVE, 0, s>>>(
            qkv, row_width, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks, positions, slots,
            scale, cut.chunk_blocks, cut.n_parts, q_tiles, part_o, part_ml, out, Finish{});
    XRT_LAUNCH_CHECK("attention (decode)");
    if (cut.n_parts == 1) return 0;
    const int part_keys = cut.chunk_blocks * WAVES * XRT_BLOCK_TOKENS;
    attention_decode_merge_kernel<HD><<<dim3(n_heads, tokens), HD, cut.n_parts * sizeof(float), s>>>(
        part_o, part_ml, positions, slots, n_heads, part_keys, cut.n_parts, out);
    XRT_LAUNCH_CHECK("attention (decode merge)");
    return 0;
}

}  // namespace

bool xrt_attention_decode_accepts(int head_dim) { return head_dim == 64 || head_dim == 128; }

// floats of workspace that a decode step of `tokens` sequences needs: the partial results of the cut that
// the launcher will choose (none where one workgroup sees all keys of a sequence)
long xrt_attention_decode_workspace(int tokens, int n_heads, int n_kv_heads, int head_dim, int max_context) {
    const int q_tiles = (n_heads / n_kv_heads + 15) / 16;
    const Cut cut = cut_for(tokens, n_kv_heads, q_tiles, max_context, head_dim);
    return cut.n_parts == 1 ? 0 : (long)tokens * n_heads * cut.n_parts * (head_dim + 2);
}

int xrt_attention_decode(const void* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const void* k_cache,
                         const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                         const int* positions, const int* slots, void* out, float scale, int max_context,
                         float* workspace, long workspace_floats, const xrt_qkv_finish* finish, hipStream_t s) {
    Finish typed{};
    if (finish != nullptr) {
        XRT_REQUIRE((finish->q_norm == nullptr) == (finish->k_norm == nullptr), "attention (decode): q_norm and k_norm come together");
        XRT_REQUIRE(finish->q_norm == nullptr || finish->norm_dtype == XRT_F32 || finish->norm_dtype == XRT_BF16,
                    "attention (decode): unknown norm dtype %d", finish->norm_dtype);
        XRT_REQUIRE(finish->rope_table == nullptr || (finish->rope_dim == head_dim && finish->table_positions >= max_context),
                    "attention (decode): the rotation that is finished here spans the whole head (%d of %d dims) and its table covers the step's positions (%d of %d)",
                    finish->rope_dim, head_dim, finish->table_positions, max_context);
        XRT_REQUIRE((uintptr_t)k_cache % 16 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)finish->q_norm % 32 == 0 &&
                    (uintptr_t)finish->k_norm % 32 == 0 && (uintptr_t)finish->rope_table % 16 == 0,
                    "attention (decode): operands must be aligned to 16 bytes (norm weights to 32)");
        // the new keys and values go where the old ones are read from
        typed = Finish{finish->q_norm, finish->k_norm, finish->norm_dtype, finish->norm_eps,
                       (const float2*)finish->rope_table, finish->rope_table ? finish->table_positions : 0,
                       (bf16*)const_cast<void*>(k_cache), (bf16*)const_cast<void*>(v_cache)};
    }
    const Finish* typed_or_none = finish != nullptr ? &typed : nullptr;
    if (head_dim == 64)
        return launch<64>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                          block_table, table_stride, n_blocks, positions, slots, (bf16*)out, scale, max_context,
                          workspace, workspace_floats, typed_or_none, s);
    return launch<128>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                       block_table, table_stride, n_blocks, positions, slots, (bf16*)out, scale, max_context,
                       workspace, workspace_floats, typed_or_none, s);
}
