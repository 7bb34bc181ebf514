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
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

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

template <int HD>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, 2) attention_decode_kernel(
    const bf16* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads,
    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ positions, const int* __restrict__ slots,
    float scale, int chunk_blocks, int n_parts, int q_tiles,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16* __restrict__ out) {
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
           float scale, int max_context, float* workspace, long workspace_floats, hipStream_t s) {
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
    attention_decode_kernel<HD><<<grid, WAVES * XRT_WAVE, 0, s>>>(
        qkv, row_width, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks, positions, slots,
        scale, cut.chunk_blocks, cut.n_parts, q_tiles, part_o, part_ml, out);
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
                         float* workspace, long workspace_floats, hipStream_t s) {
    if (head_dim == 64)
        return launch<64>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                          block_table, table_stride, n_blocks, positions, slots, (bf16*)out, scale, max_context,
                          workspace, workspace_floats, s);
    return launch<128>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                       block_table, table_stride, n_blocks, positions, slots, (bf16*)out, scale, max_context,
                       workspace, workspace_floats, s);
}
