// Prefill attention on the matrix cores: causal attention of the new tokens of every sequence
// of a step over that sequence's cache (which already holds the new keys and values), without
// ever forming the score matrix in memory.
//
// Formulas: crates/xrt-models/src/llama.rs:727-770 of the reference (the token at position P
// sees keys 0..P; score = q.k * scale; softmax; weighted sum of values; query head h uses
// key/value head h / group), computed with the running maximum and sum of its decode loop
// (:514-574) instead of a stored row of scores.
//
// A workgroup owns 256 (or 128) consecutive query tokens of one sequence and one head: eight (or
// four) wavefronts with 32 queries each; a compute unit then holds eight wavefronts, two per
// SIMD, so that one can do its softmax while the other multiplies. The workgroup walks the
// sequence's cache blocks (64 keys) in order; every block
// travels once from global memory into LDS (keys as they lie, values transposed as they lie),
// the next block while the current one is used, and all wavefronts read their operands
// from there. Everything is kept transposed so that one lane owns one query:
// S^T[key][query] = K Q^T and O^T[dim][query] += V^T P^T with v_mfma_f32_32x32x16_bf16.
// Maximum, sum and rescaling of a query are then private to a lane (plus its partner 32 lanes
// away), and the probabilities are already in the registers, and the order, that the second
// product wants as its B operand: key rows are assigned to accumulator rows such that a lane
// holds eight consecutive keys per K step, which are also 16 contiguous bytes of the
// transposed value block. LDS rows are padded by 16 bytes, which spreads the 16-byte operand
// reads of consecutive rows over the banks.
#include "common.h"
#include "xrt_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int QT = 32;                 // query tokens per wavefront
constexpr int BT = XRT_BLOCK_TOKENS;   // keys per cache block
constexpr int PER_STAGE = 2;           // cache blocks between two barriers
constexpr float LOG2E = 1.4426950408889634f;

// Key (0..31 within a tile of 32 keys) that row r of the score tile stands for. Accumulator
// register i of lane half h is row (i/4)*8 + h*4 + i%4 and must be key (i/8)*16 + h*8 + i%8.
__device__ __forceinline__ int key_of_row(int r) { return (r / 16) * 16 + ((r % 8) / 4) * 8 + ((r / 8) % 2) * 4 + r % 4; }

// WAVES wavefronts of 32 queries each share the cache blocks that the workgroup moves through LDS.
template <int HD, int WAVES>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) attention_prefill_kernel(
    const bf16* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads,
    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ seq_offsets, const int* __restrict__ seq_slots,
    const int* __restrict__ seq_starts, int n_seqs, bf16* __restrict__ out, float scale) {
    constexpr int QW = WAVES * QT;         // query tokens per workgroup
    constexpr int KS = HD / 16;            // K steps of the score product
    constexpr int DT = HD / 32;            // 32-row tiles of the value product
    constexpr int K_CHUNKS = HD / 8;       // 16-byte chunks of a key row (16 or 8)
    constexpr int V_CHUNKS = BT / 8;       // of a transposed value row (8)
    constexpr int LOADS = BT * HD * 2 / 1024 / WAVES;           // load instructions per wavefront for a block's keys (and as many for its values)
    static_assert(BT * HD * 2 % (1024 * WAVES) == 0, "a cache block does not divide among the wavefronts");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    // two buffers of PER_STAGE cache blocks each: one barrier per PER_STAGE blocks
    bf16 (*lds_k)[BT * HD] = reinterpret_cast<bf16 (*)[BT * HD]>(lds_raw);                                  // [2 * PER_STAGE][BT * HD]
    bf16 (*lds_v)[HD * BT] = reinterpret_cast<bf16 (*)[HD * BT]>(lds_raw + 2 * PER_STAGE * BT * HD * sizeof(bf16));   // [2 * PER_STAGE][HD * BT]
    // Rows are not padded (a load instruction fills 1024 consecutive bytes of LDS); instead the
    // 16-byte chunks of a row lie in permuted places, place = chunk ^ swizzle(row), chosen so
    // that the operand reads of consecutive rows at one chunk fall into different banks.
    auto k_swizzle = [](int row) { return K_CHUNKS == 16 ? row % 16 : (row % 8) ^ (row / 8 % 2); };
    auto v_swizzle = [](int row) { return (row % 8) ^ (row / 8 % 2); };

    const int tid = threadIdx.x, lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    const int col = lane % 32, half = lane / 32;
    const int head = blockIdx.x;

    // which sequence and which of its query tiles this workgroup has; tiles are walked backwards
    // and heads change fastest, so that the tiles with the most keys before them (the last of a
    // sequence) start first, for all heads
    int tile = gridDim.y - 1 - blockIdx.y, seq = 0, count = 0;
    for (; seq < n_seqs; ++seq) {
        count = seq_offsets[seq + 1] - seq_offsets[seq];
        const int tiles = (count + QW - 1) / QW;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (seq >= n_seqs) return;                               // the whole workgroup leaves
    const int slot = seq_slots[seq];
    const int start = seq_starts[seq];                       // tokens in the cache before this step
    const int wg_first = tile * QW;                          // index among the sequence's new tokens
    const int wg_last_key = start + min(count, wg_first + QW) - 1;    // the furthest key any query of the workgroup sees
    const int q_first = wg_first + wave * QT;
    const int q_count = max(0, min(QT, count - q_first));    // queries of this wavefront that exist
    const bool q_valid = col < q_count;
    const long token = (long)seq_offsets[seq] + min(q_first + col, count - 1);   // row of qkv and out (clamped: loads need no guard)
    const int q_pos = start + q_first + col;                 // absolute position of this lane's query
    const int last_key = start + q_first + q_count - 1;      // the furthest key any query of the wavefront sees
    const int first_masked = start + q_first;                // key tiles that end at or before this need no mask
    const int kv_head = head / (n_heads / n_kv_heads);

    bf16x8 q[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        q[ks] = *reinterpret_cast<const bf16x8*>(qkv + token * row_width + (long)head * HD + ks * 16 + half * 8);

    const float scale2 = scale * LOG2E;
    float m = -INFINITY, l = 0.f;
    floatx16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;

    // ---- moving a cache block into LDS: both parts are contiguous in global memory, and go
    // straight there (global_load_lds_dwordx4): lane l of an instruction fills the l-th 16 bytes
    // of a 1024-byte stretch with the chunk that belongs in that place
    const int wave_uniform = __builtin_amdgcn_readfirstlane(wave);
    unsigned k_from[LOADS], v_from[LOADS];                   // byte offsets of this lane's chunks within a block
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int place = ((i * WAVES + wave) * XRT_WAVE + lane);          // 16-byte place within the block's LDS image
        const int k_row = place / K_CHUNKS, v_row = place / V_CHUNKS;
        k_from[i] = (unsigned)((k_row * K_CHUNKS + ((place % K_CHUNKS) ^ k_swizzle(k_row))) * 16);
        v_from[i] = (unsigned)((v_row * V_CHUNKS + ((place % V_CHUNKS) ^ v_swizzle(v_row))) * 16);
    }
    const unsigned lds_k0 = lds_address(lds_raw), lds_v0 = lds_k0 + 2 * PER_STAGE * BT * HD * (unsigned)sizeof(bf16);
    auto fetch = [&](int b, int buffer) {
        int block = block_table[(long)slot * table_stride + b];
        block = min(max(block, 0), n_blocks - 1);            // the host never hands out anything else
        const bf16* kb = k_cache + ((long)block * n_kv_heads + kv_head) * BT * HD;
        const bf16* vb = v_cache + ((long)block * n_kv_heads + kv_head) * HD * BT;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const unsigned at = (unsigned)((buffer * BT * HD) * 2 + (i * WAVES + wave_uniform) * 1024);
            load_to_lds(kb, k_from[i], lds_k0 + at);
            load_to_lds(vb, v_from[i], lds_v0 + at);
        }
    };

    const int row_key = key_of_row(col);                     // the key this lane's A-operand row stands for

    // one tile of 32 keys (half a block) against this wavefront's 32 queries
    auto tile32 = [&](int buffer, int k0, int in_block) {
        const bf16* kb = &lds_k[buffer][(in_block + row_key) * HD];
        const int k_turn = k_swizzle(in_block + row_key);     // in_block is 0 or 32: the swizzle of this lane's key row
        const bf16* vb = &lds_v[buffer][0];
        const int v_first = in_block / 8 + half;              // chunk of a value row that step 0 reads
        auto k_at = [&](int ks) { return kb + ((ks * 2 + half) ^ k_turn) * 8; };
        // two accumulators, used in turn, so that consecutive products do not wait on each other
        floatx16 s, s_odd;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] = s_odd[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks += 2) {
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(k_at(ks)), q[ks], s, 0, 0, 0);
            s_odd = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(k_at(ks + 1)), q[ks + 1], s_odd, 0, 0, 0);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] += s_odd[e];

        // register i is key k0 + (i/8)*16 + half*8 + i%8, for this lane's query
        const bool edge = k0 + 31 > first_masked;            // some key of the tile may lie beyond some query
        float tile_max = -INFINITY;                          // of the raw products: the scale is positive
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int key = k0 + (i / 8) * 16 + half * 8 + i % 8;
            if (edge && key > q_pos) s[i] = -INFINITY;        // causal: keys after the query do not exist for it
            tile_max = fmaxf(tile_max, s[i]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, XRT_WAVE));
        // m is the exponent that the sums so far are relative to: the largest score seen when it was
        // last moved, not necessarily the largest seen. It moves, and the sums are scaled down,
        // only when some query of the wavefront meets a score more than 8 (in log2) above its m;
        // until then the probabilities are at most 2^8 and the quotient at the end is the same.
        // After the first tiles that is rare.
        const float tile_top = tile_max * scale2;
        if (__builtin_amdgcn_ballot_w64(tile_top > m + 8.0f) != 0) {
            const float m_new = fmaxf(m, tile_top);
            const float correction = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.f : m_new));
            l *= correction;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[dt][e] *= correction;
            m = m_new;
        }
        const float m_safe = m == -INFINITY ? 0.f : m;        // a query that sees none of these keys yet

        bf16x8 p[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s[i], scale2, -m_safe));
            l += e;
            p[i / 8][i % 8] = (bf16)e;
        }
#pragma unroll
        for (int step = 0; step < 2; ++step)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int v_row = dt * 32 + col;
                bf16x8 v = *reinterpret_cast<const bf16x8*>(vb + v_row * BT + ((v_first + step * 2) ^ v_swizzle(v_row)) * 8);
                if (edge) {
                    // beyond the sequence's last key the block holds nothing of ours: keep it away from the zeros of p
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + step * 16 + half * 8 + e > last_key) v[e] = (bf16)0.f;
                }
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v, p[step], o[dt], 0, 0, 0);
            }
    };

    // ---- the blocks of the sequence, in order: block b+1 travels while block b is used
    const int last_block = wg_last_key / BT;
#pragma unroll
    for (int i = 0; i < PER_STAGE; ++i)
        if (i <= last_block) fetch(i, i);
    wait_loads_and_barrier<0>();
    for (int first = 0; first <= last_block; first += PER_STAGE) {
        const int stage = (first / PER_STAGE) & 1;
        // the other stage's buffers were read in the step before, ahead of the last barrier
#pragma unroll
        for (int i = 0; i < PER_STAGE; ++i)
            if (first + PER_STAGE + i <= last_block) fetch(first + PER_STAGE + i, (stage ^ 1) * PER_STAGE + i);
#pragma unroll
        for (int i = 0; i < PER_STAGE; ++i) {
        const int b = first + i, buffer = stage * PER_STAGE + i;
        if (b > last_block) continue;
        if (q_count > 0) {
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                const int k0 = b * BT + sub * 32;
                if (k0 <= last_key) tile32(buffer, k0, sub * 32);        // uniform in the wavefront
            }
        }
        }
        wait_loads_and_barrier<0>();                         // the next blocks have arrived from every wavefront, these have been read by all
    }
    l += __shfl_xor(l, 32, XRT_WAVE);

    if (q_valid) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16* dst = out + (token * n_heads + head) * HD;
        // accumulator register i of tile dt is dimension dt*32 + (i/4)*8 + half*4 + i%4, for this lane's query
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                struct alignas(8) Four { bf16 e[4]; } four;
#pragma unroll
                for (int i = 0; i < 4; ++i) four.e[i] = (bf16)(o[dt][g * 4 + i] * inv);
                *reinterpret_cast<Four*>(dst + dt * 32 + g * 8 + half * 4) = four;
            }
    }
}

template <int HD, int WAVES>
int launch_waves(const bf16* qkv, int tokens, int n_heads, int n_kv_heads, const bf16* k_cache, const bf16* v_cache,
                 const int* block_table, int table_stride, int n_blocks, const int* seq_offsets, const int* seq_slots,
                 const int* seq_starts, int n_seqs, bf16* out, float scale, hipStream_t s) {
    constexpr int QW = WAVES * QT;
    const int row_width = (n_heads + 2 * n_kv_heads) * HD;
    // every sequence has at most ceil(count / QW) tiles; their sum is at most tokens / QW + n_seqs
    const long tiles = (tokens + QW - 1) / QW + n_seqs;
    XRT_REQUIRE(tiles <= 65535, "attention (prefill): too many query tiles for the grid");
    const dim3 grid(n_heads, (unsigned)tiles);
    constexpr size_t lds = (size_t)2 * PER_STAGE * (BT * HD + HD * BT) * sizeof(bf16);
    static bool configured = false;          // per instantiation
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_prefill_kernel<HD, WAVES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        XRT_REQUIRE(e == hipSuccess, "attention (prefill): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    attention_prefill_kernel<HD, WAVES><<<grid, WAVES * XRT_WAVE, lds, s>>>(
        qkv, row_width, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks, seq_offsets,
        seq_slots, seq_starts, n_seqs, out, scale);
    XRT_LAUNCH_CHECK("attention (prefill)");
    return 0;
}

template <int HD>
int launch(const bf16* qkv, int tokens, int n_heads, int n_kv_heads, const bf16* k_cache, const bf16* v_cache,
           const int* block_table, int table_stride, int n_blocks, const int* seq_offsets, const int* seq_slots,
           const int* seq_starts, int n_seqs, bf16* out, float scale, hipStream_t s) {
    // Tiles of 128 queries (four wavefronts, two workgroups to a compute unit) would spread the
    // uneven work of causal tiles better, but were measured slower at 2048 tokens (121 against
    // 101 us): every workgroup moves all its cache blocks through LDS, and with half the
    // wavefronts per block that work doubles. Nor do they help where tiles of 256 leave compute
    // units empty, with a tile of many keys and one of few sharing a compute unit: 50.6 against
    // 48.3 us at 1024 tokens, 93.6 against 93.2 at 2048.
    return launch_waves<HD, 8>(qkv, tokens, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks,
                               seq_offsets, seq_slots, seq_starts, n_seqs, out, scale, s);
}

}  // namespace

bool xrt_attention_prefill_accepts(int head_dim) { return head_dim == 64 || head_dim == 128; }

int xrt_attention_prefill(const void* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const void* k_cache,
                          const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                          const int* seq_offsets, const int* seq_slots, const int* seq_starts, int n_seqs, void* out,
                          float scale, hipStream_t s) {
    if (head_dim == 64)
        return launch<64>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                          block_table, table_stride, n_blocks, seq_offsets, seq_slots, seq_starts, n_seqs, (bf16*)out, scale, s);
    return launch<128>((const bf16*)qkv, tokens, n_heads, n_kv_heads, (const bf16*)k_cache, (const bf16*)v_cache,
                       block_table, table_stride, n_blocks, seq_offsets, seq_slots, seq_starts, n_seqs, (bf16*)out, scale, s);
}
