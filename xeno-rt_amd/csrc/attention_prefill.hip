// Prefill attention on the matrix cores: causal attention of the new tokens of every sequence
// of a step over that sequence's cache (which already holds the new keys and values), without
// ever forming the score matrix in memory.
//
// Formulas: crates/xrt-models/src/llama.rs:727-770 of the reference (the token at position P
// sees keys 0..P; score = q.k * scale; softmax; weighted sum of values; query head h uses
// key/value head h / group), computed with the running maximum and sum of its decode loop
// (:514-574) instead of a stored row of scores.
//
// A workgroup of eight wavefronts (two per SIMD, so that one can do its softmax while the other
// multiplies) has two tiles of 128 query tokens of one sequence and one head, a late and an
// early one, and 32 queries per wavefront; how the two tiles share the wavefronts is told at
// the kernel. The workgroup walks the sequence's cache blocks (64 keys) in order; every block
// travels once from global memory into LDS (keys in rows, values transposed),
// the next blocks while the current ones are used, and all wavefronts read their operands
// from there. Everything is kept transposed so that one lane owns one query:
// S^T[key][query] = K Q^T and O^T[dim][query] += V^T P^T with v_mfma_f32_32x32x16_bf16.
// Maximum, sum and rescaling of a query are then private to a lane (plus its partner 32 lanes
// away), and the probabilities are already in the registers, and the order, that the second
// product wants as its B operand: key rows are assigned to accumulator rows such that a lane
// holds eight consecutive keys per K step, which are also 16 contiguous bytes of the
// transposed value block.
#include "cache_layout.h"
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

// Eight wavefronts share the cache blocks that the workgroup moves through LDS. They work on two tiles of 128
// queries of one sequence and one head: a late one, which sees many keys, and an early one, which sees few
// (tile T-1-p with tile p; a middle tile alone). Wavefronts 0..3 take the late tile's four groups of 32 queries.
// Wavefronts 4..7 first take the early tile's; when its last block of keys is done they write its result and
// turn to the late tile as well: from then on the blocks of a stage are dealt out in turn, one to wavefront w
// and one to wavefront w + 4, which hold the same 32 queries, and in the end the two merge what they have
// (maximum, sum, weighted values) through LDS. Every workgroup of a sequence thus has the same work: with tiles
// that stand alone the last one of a causal sequence has twice the mean, and the step ends when it does.
constexpr int GROUPS = 4;              // groups of 32 queries in a tile
constexpr int WAVES = 2 * GROUPS;
constexpr int QW = GROUPS * QT;        // queries of a tile

template <int HD>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) attention_prefill_kernel(
    const bf16* __restrict__ qkv, int row_width, int n_heads, int n_kv_heads,
    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_stride, int n_blocks, const int* __restrict__ seq_offsets, const int* __restrict__ seq_slots,
    const int* __restrict__ seq_starts, int n_seqs, bf16* __restrict__ out, float scale) {
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
    // Workgroup ids are dealt to the 8 XCDs round-robin: the heads are renumbered so that the heads of one group of
    // key/value heads run on one XCD, at the same time, and find each other's cache blocks in its L2.
    const int head = n_heads % 8 == 0 ? (int)(blockIdx.x % 8) * (n_heads / 8) + (int)blockIdx.x / 8 : (int)blockIdx.x;
    const int wave_uniform = __builtin_amdgcn_readfirstlane(wave);      // in a scalar register: what depends on it alone is decided by scalar branches
    const int group = wave_uniform % GROUPS;                 // the 32 queries of a tile that this wavefront holds
    const bool helper = wave_uniform >= GROUPS;              // early tile first, then half of the late tile's blocks

    // which sequence and which pair of its tiles this workgroup has
    int pair = blockIdx.y, seq = 0, count = 0, tiles = 0;
    for (; seq < n_seqs; ++seq) {
        count = seq_offsets[seq + 1] - seq_offsets[seq];
        tiles = (count + QW - 1) / QW;
        const int pairs = (tiles + 1) / 2;
        if (pair < pairs) break;
        pair -= pairs;
    }
    if (seq >= n_seqs) return;                               // the whole workgroup leaves
    const int slot = seq_slots[seq];
    const int start = seq_starts[seq];                       // tokens in the cache before this step
    const int late_tile = tiles - 1 - pair, early_tile = pair;
    const bool has_early = early_tile < late_tile;
    // blocks of keys that the two tiles see: the early tile 0 .. early_blocks - 1, the late tile 0 .. late_blocks - 1
    const int late_blocks = (start + min(count, (late_tile + 1) * QW) - 1) / BT + 1;
    const int early_blocks = has_early ? (start + (early_tile + 1) * QW - 1) / BT + 1 : 0;
    const int kv_head = head / (n_heads / n_kv_heads);
    const float scale2 = scale * LOG2E;

    // ---- the queries a wavefront is working on
    long token = 0;                                          // row of qkv and out (clamped: loads need no guard)
    int q_count = 0, q_pos = 0, last_key = -1, first_masked = 0;
    bool q_valid = false;
    bf16x8 q[KS];
    float m = -INFINITY, l = 0.f;
    floatx16 o[DT];
    auto take = [&](int tile) {
        const int q_first = tile * QW + group * QT;
        q_count = max(0, min(QT, count - q_first));          // queries of this wavefront that exist
        q_valid = col < q_count;
        token = (long)seq_offsets[seq] + min(q_first + col, count - 1);
        q_pos = start + q_first + col;                       // absolute position of this lane's query
        last_key = q_count > 0 ? start + q_first + q_count - 1 : -1;     // the furthest key any query of the wavefront sees
        first_masked = start + q_first;                      // key tiles that end at or before this need no mask
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            q[ks] = *reinterpret_cast<const bf16x8*>(qkv + token * row_width + (long)head * HD + ks * 16 + half * 8);
        // The queries are awaited here, once. Left to their first use, the wait would stand inside the loop over the
        // blocks, and there it would also wait for the blocks on their way into LDS (the counter of outstanding loads
        // knows no difference, and the compiler does not see the loads that the assembly issues).
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(q[ks]));
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
    };
    // the result of the queries at hand: out = o / l
    auto write_out = [&]() {
        if (!q_valid) return;
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
    };
    take(helper && has_early ? early_tile : late_tile);
    bool on_early = helper && has_early;

    // ---- moving a cache block into LDS: it goes straight there (global_load_lds_dwordx4): lane l of an
    // instruction fills the l-th 16 bytes of a 1024-byte stretch with the chunk that belongs in that place,
    // 8 dims of a key or 8 tokens of a value dim, which lie together in the cache block too (cache_layout.h:
    // the block itself is in the order of the decode kernel's operands, not in rows)
    unsigned k_from[LOADS], v_from[LOADS];                   // byte offsets of this lane's chunks within a block
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int place = (i * WAVES + wave) * XRT_WAVE + lane;      // 16-byte place within the block's LDS image
        const int k_row = place / K_CHUNKS, v_row = place / V_CHUNKS;
        k_from[i] = (unsigned)cache_key_offset(k_row, ((place % K_CHUNKS) ^ k_swizzle(k_row)) * 8, HD) * 2u;
        v_from[i] = (unsigned)cache_value_offset(v_row, ((place % V_CHUNKS) ^ v_swizzle(v_row)) * 8, HD) * 2u;
    }
    const unsigned lds_k0 = lds_address(lds_raw), lds_v0 = lds_k0 + 2 * PER_STAGE * BT * HD * (unsigned)sizeof(bf16);
    // The table's entries are read a stage before they are used: read where they are used, every stage would begin
    // with the wait for a scalar load.
    const int* table = block_table + (long)slot * table_stride;
    auto block_of = [&](int b) { return table[min(b, table_stride - 1)]; };
    auto fetch = [&](int block, int buffer) {
        block = min(max(block, 0), n_blocks - 1);            // the host never hands out anything else
        const char* kb = reinterpret_cast<const char*>(k_cache + ((long)block * n_kv_heads + kv_head) * BT * HD);
        const char* vb = reinterpret_cast<const char*>(v_cache + ((long)block * n_kv_heads + kv_head) * HD * BT);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const unsigned at = (unsigned)((buffer * BT * HD) * 2 + (i * WAVES + wave_uniform) * 1024);
            load_to_lds(kb, k_from[i], lds_k0 + at);
            load_to_lds(vb, v_from[i], lds_v0 + at);
        }
    };

    // The blocks of the next stage are asked for piece by piece (an instruction for a kilobyte of keys and one of values),
    // one piece at the stage's start and one behind each tile's score products and value products, the rest before the
    // barrier. Asked for all at once right after the barrier, the 64 instructions of eight wavefronts queue up: a
    // wavefront then spends 550 to 1550 cycles of a stage of some 3000 getting its eight accepted (counted with the
    // shader clock), the wavefronts of the early tile, the younger ones, the longest.
    constexpr int PIECES = PER_STAGE * LOADS;
    int next_piece = PIECES, piece_blocks[PER_STAGE], piece_buffer = 0, pieces_wanted = 0;
    auto fetch_piece = [&]() {
        if (next_piece >= pieces_wanted) return;
        const int i = next_piece / LOADS, l = next_piece % LOADS;
        int block = piece_blocks[0];
        unsigned kf = k_from[0], vf = v_from[0];
#pragma unroll
        for (int j = 1; j < PER_STAGE; ++j) if (i == j) block = piece_blocks[j];
#pragma unroll
        for (int j = 1; j < LOADS; ++j) if (l == j) { kf = k_from[j]; vf = v_from[j]; }
        block = min(max(block, 0), n_blocks - 1);            // the host never hands out anything else
        const char* kb = reinterpret_cast<const char*>(k_cache + ((long)block * n_kv_heads + kv_head) * BT * HD);
        const char* vb = reinterpret_cast<const char*>(v_cache + ((long)block * n_kv_heads + kv_head) * HD * BT);
        const unsigned at = (unsigned)(((piece_buffer + i) * BT * HD) * 2 + (l * WAVES + wave_uniform) * 1024);
        load_to_lds(kb, kf, lds_k0 + at);
        load_to_lds(vb, vf, lds_v0 + at);
        ++next_piece;
    };
    const int row_key = key_of_row(col);                     // the key this lane's A-operand row stands for

    // The operand of the score product for a tile of 32 keys (half a block: in_block is 0 or 32): this lane's key row.
    auto keys_of = [&](bf16x8 (&k)[KS], int buffer, int in_block) {
        const bf16* kb = &lds_k[buffer][(in_block + row_key) * HD];
        const int k_turn = k_swizzle(in_block + row_key);     // the swizzle of this lane's key row
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) k[ks] = *reinterpret_cast<const bf16x8*>(kb + ((ks * 2 + half) ^ k_turn) * 8);
    };
    // One tile of 32 keys against this wavefront's 32 queries. edge: some key of the tile may lie beyond
    // some query, or beyond the sequence's end; the other tiles, nearly all, skip the masks (a scalar branch each).
    // k: the tile's keys, already asked for; behind_the_scores: what the caller wants issued right behind the score
    // products (the read of the next tile's keys, which then has the softmax and the value products to arrive in).
    auto tile32 = [&](bool edge, int buffer, int k0, int in_block, bf16x8 (&k)[KS], auto&& behind_the_scores) {
        const bf16* vb = &lds_v[buffer][0];
        const int v_first = in_block / 8 + half;              // chunk of a value row that step 0 reads
        auto v_at = [&](int step, int dt) {
            const int v_row = dt * 32 + col;
            return *reinterpret_cast<const bf16x8*>(vb + v_row * BT + ((v_first + step * 2) ^ v_swizzle(v_row)) * 8);
        };
        // The values of the first 16 keys are asked for right behind the score products (left to itself the compiler reads
        // one operand, waits for it, multiplies, reads the next): they have the products and half the softmax to arrive in,
        // and the wait for the keys before the first product of a block does not wait for them too.
        floatx16 s;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k[ks], q[ks], s, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 v[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v[dt] = v_at(0, dt);
        behind_the_scores();
        __builtin_amdgcn_sched_barrier(0);
        fetch_piece();

        // register i is key k0 + (i/8)*16 + half*8 + i%8, for this lane's query
        if (edge) {
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (k0 + (i / 8) * 16 + half * 8 + i % 8 > q_pos) s[i] = -INFINITY;     // causal: keys after the query do not exist for it
        }
        float lane_max = s[0];                               // of the raw products: the scale is positive
#pragma unroll
        for (int i = 1; i < 16; ++i) lane_max = fmaxf(lane_max, s[i]);
        // m is the exponent that the sums so far are relative to: the largest score seen when it was
        // last moved, not necessarily the largest seen. It moves, and the sums are scaled down,
        // only when some query of the wavefront meets a score more than 8 (in log2) above its m;
        // until then the probabilities are at most 2^8 and the quotient at the end is the same.
        // After the first tiles that is rare. The two lanes of a query move their m together.
        if (__builtin_amdgcn_ballot_w64(lane_max * scale2 > m + 8.0f) != 0) {
            const float tile_top = fmaxf(lane_max, __shfl_xor(lane_max, 32, XRT_WAVE)) * scale2;
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
        for (int step = 0; step < 2; ++step) {
            if (edge) {
                // beyond the sequence's last key the block holds nothing of ours: keep it away from the zeros of p
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + step * 16 + half * 8 + e > last_key) v[dt][e] = (bf16)0.f;
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v[dt], p[step], o[dt], 0, 0, 0);
                if (step == 0) v[dt] = v_at(1, dt);    // the values of the other 16 keys, behind the product that used the register
            }
        }
        fetch_piece();
    };

    // ---- the blocks of the sequence, in order: the next stage's blocks travel while this stage's are used
    const int last_block = late_blocks - 1;
    // the early tile's blocks end at a stage's end for the helpers: up to there every wavefront takes every block
    // (those beyond its queries' last key fall away by themselves), from there on they take turns
    const int turns_from = (early_blocks + PER_STAGE - 1) / PER_STAGE * PER_STAGE;
    int coming[PER_STAGE];                                   // the blocks that the next fetch asks for
#pragma unroll
    for (int i = 0; i < PER_STAGE; ++i) {
        if (i <= last_block) fetch(block_of(i), i);
        coming[i] = block_of(PER_STAGE + i);
    }
    wait_loads_and_barrier<0>();
    for (int first = 0; first <= last_block; first += PER_STAGE) {
        const int stage = (first / PER_STAGE) & 1;
        // the other stage's buffers were read in the step before, ahead of the last barrier
        pieces_wanted = max(0, min(PER_STAGE, last_block - first - PER_STAGE + 1)) * LOADS;
        next_piece = 0;
        piece_buffer = (stage ^ 1) * PER_STAGE;
#pragma unroll
        for (int i = 0; i < PER_STAGE; ++i) {
            piece_blocks[i] = coming[i];
            coming[i] = block_of(first + 2 * PER_STAGE + i);
        }
        fetch_piece();
        // one body of code for all tiles of the stage: the kernel stays small enough for the instruction cache
#pragma unroll 1
        for (int i = 0; i < PER_STAGE; ++i) {
            const int b = first + i, k0 = b * BT;
            if (b > last_block || k0 > last_key) break;      // uniform in the wavefront, like all that follows
            if (b >= turns_from && ((b - turns_from) % 2 == 1) != helper) continue;
            const int buffer = stage * PER_STAGE + i;
            // The block's two tiles. The second one's keys are read from LDS behind the first one's score products, so
            // that they have a softmax and the value products to arrive in (a prompt of 2048 tokens: 62 -> 57 us; with every
            // tile's keys read a tile ahead, across the blocks of a stage too, 59).
            const bool both = k0 + 32 <= last_key;
            bf16x8 first_keys[KS], second_keys[KS];
            keys_of(first_keys, buffer, 0);
            tile32(k0 + 31 > first_masked, buffer, k0, 0, first_keys, [&] { if (both) keys_of(second_keys, buffer, 32); });
            if (both) tile32(k0 + 63 > first_masked, buffer, k0 + 32, 32, second_keys, [] {});
        }
        if (on_early && first + PER_STAGE >= early_blocks) {  // the early tile is done: its result goes out, the late tile's queries come in
            l += __shfl_xor(l, 32, XRT_WAVE);
            write_out();
            take(late_tile);
            on_early = false;
        }
        while (next_piece < pieces_wanted) fetch_piece();     // a wavefront with few tiles in this stage, or none
        wait_loads_and_barrier<0>();                         // the next blocks have arrived from every wavefront, these have been read by all
    }

    // ---- the two wavefronts of a group of queries merge what they have, through LDS (the blocks' buffers are free now)
    float (*merge_o)[DT * 16][XRT_WAVE] = reinterpret_cast<float (*)[DT * 16][XRT_WAVE]>(lds_raw);          // [GROUPS]
    float (*merge_ml)[2][XRT_WAVE] = reinterpret_cast<float (*)[2][XRT_WAVE]>(lds_raw + GROUPS * DT * 16 * XRT_WAVE * sizeof(float));
    if (helper) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) merge_o[group][dt * 16 + e][lane] = o[dt][e];
        merge_ml[group][0][lane] = m;
        merge_ml[group][1][lane] = l;
    }
    __syncthreads();
    if (helper) return;
    {
        const float other_m = merge_ml[group][0][lane], other_l = merge_ml[group][1][lane];
        const float m_all = fmaxf(m, other_m);
        const float m_safe = m_all == -INFINITY ? 0.f : m_all;
        const float mine = __builtin_amdgcn_exp2f(m - m_safe), theirs = __builtin_amdgcn_exp2f(other_m - m_safe);   // 0 for a side that saw no key
        l = l * mine + other_l * theirs;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[dt][e] = o[dt][e] * mine + merge_o[group][dt * 16 + e][lane] * theirs;
    }
    l += __shfl_xor(l, 32, XRT_WAVE);
    write_out();
}

template <int HD>
int launch_waves(const bf16* qkv, int tokens, int n_heads, int n_kv_heads, const bf16* k_cache, const bf16* v_cache,
                 const int* block_table, int table_stride, int n_blocks, const int* seq_offsets, const int* seq_slots,
                 const int* seq_starts, int n_seqs, bf16* out, float scale, hipStream_t s) {
    const int row_width = (n_heads + 2 * n_kv_heads) * HD;
    // a sequence of `count` tokens has ceil(ceil(count / QW) / 2) pairs of tiles; their sum is at most this
    const long pairs = ((tokens + QW - 1) / QW + n_seqs) / 2 + n_seqs;
    XRT_REQUIRE(pairs <= 65535, "attention (prefill): too many query tiles for the grid");
    const dim3 grid(n_heads, (unsigned)pairs);
    constexpr size_t lds = (size_t)2 * PER_STAGE * (BT * HD + HD * BT) * sizeof(bf16);
    static_assert(lds >= GROUPS * (HD / 32 * 16 + 2) * XRT_WAVE * sizeof(float), "the merge does not fit the blocks' buffers");
    static bool configured = false;          // per instantiation
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_prefill_kernel<HD>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        XRT_REQUIRE(e == hipSuccess, "attention (prefill): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    attention_prefill_kernel<HD><<<grid, WAVES * XRT_WAVE, lds, s>>>(
        qkv, row_width, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks, seq_offsets,
        seq_slots, seq_starts, n_seqs, out, scale);
    XRT_LAUNCH_CHECK("attention (prefill)");
    return 0;
}

template <int HD>
int launch(const bf16* qkv, int tokens, int n_heads, int n_kv_heads, const bf16* k_cache, const bf16* v_cache,
           const int* block_table, int table_stride, int n_blocks, const int* seq_offsets, const int* seq_slots,
           const int* seq_starts, int n_seqs, bf16* out, float scale, hipStream_t s) {
    return launch_waves<HD>(qkv, tokens, n_heads, n_kv_heads, k_cache, v_cache, block_table, table_stride, n_blocks,
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
