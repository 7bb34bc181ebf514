// Matrix product for few rows (M <= 64: decode steps and short prompts) with w kept in tiles (packing.h):
// out[m, n] = sum_k x[m, k] * w[n, k], bfloat16 operands, float32 accumulation on the matrix cores.
//
// Such a product is bound by reading w once from HBM. A workgroup of 8 wavefronts owns one group of 16
// packed rows of w; each wavefront takes one eighth of the group's tiles along k, which lie one after
// another in memory, and streams them straight into the A operand of v_mfma_f32_16x16x32_bf16: one load
// instruction of the wavefront is one whole tile, a contiguous kilobyte. Because every instruction takes
// whole cache lines that nobody else reads, the loads are marked non-temporal (they pass the caches by),
// which is what brings the stream from about 5.5 to 6.4 TB/s here; with rows contiguous along k an
// instruction takes half a line of each of 16 rows, and the same mark makes it fetch every line twice.
// The B operand holds the activations x (16 rows of m per tile). Loads run one step (two tiles) ahead of
// the matrix cores; the eight partial sums are added in wavefront order through LDS, so the result does
// not depend on timing.
//
// Epilogues, as in the product for rows contiguous along k (gemm_skinny.hip): store, accumulate into
// float32, the gated pair silu(gate) * up (the packing puts the gate and up rows of eight outputs into
// one tile: a lane finds its partner 32 lanes away), an RMSNorm's halves around the product, and what
// follows a q/k/v projection (rotation of q and k, cache write; the packing puts the two halves of a
// rotated head's pairs into one tile).
#include "packing.h"
#include "gemm_skinny.h"
#include "activation.h"

namespace {

using LinearNorm = xrt_linear_norm;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVES = 8;
constexpr int JL = 2;              // tiles of 32 along k per step of a wavefront
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };


// MT: tiles of 16 rows of x. EXTRA 1: the kernel also does its share of an RMSNorm before or after the
// product; 2: and what follows a q/k/v projection (both: one tile of x).
// N: output columns (the row length of out); the gated product has 2 N rows of w.
template <int MT, int MODE, typename TO, int EXTRA = 0>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, (MT == 1 ? 4 : 2)) gemm_packed_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    const Packing packing, const LinearNorm norm, const QkvAfter after, int activation) {
    constexpr bool AROUND = EXTRA != 0, QKV = EXTRA == 2;
    static_assert(!AROUND || MT == 1, "the norm around a product: one tile of x");
    static_assert(!QKV || (MODE == MODE_STORE && sizeof(TO) == 2), "after a q/k/v projection: a bfloat16 store");
    constexpr int SQUARES_AHEAD = 8;                            // sums of squares a lane asks for when the kernel starts
    __shared__ floatx4 partial[MT > 1 ? 2 : 1][WAVES][XRT_WAVE];
    __shared__ float squares[WAVES][16];
    // what the accumulating epilogue needs from global memory is asked for when the kernel starts and
    // goes straight into LDS, past the registers: it is there when the stream of w has run through
    __shared__ floatx4 early_out[XRT_WAVE];
    __shared__ float early_gain[XRT_WAVE];
    // for the q/k/v epilogue, worked out while the first loads are on their way: cosine and sine of
    // the lane's four angles, and where the lane's token lies in the cache
    __shared__ float early_cos[QKV ? XRT_WAVE : 1][4], early_sin[QKV ? XRT_WAVE : 1][4];
    __shared__ long early_base[QKV ? 16 : 1];
    __shared__ int early_within[QKV ? 16 : 1];

    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int r = lane % 16, c = lane / 16;
    const long first = (long)blockIdx.x * 16;                   // the group's first packed row
    // after a q/k/v projection: the tile's head, and the dims of the head that its rows 0..7 and 8..15 make
    int head = 0, lower_dim = 0, upper_dim = 8;
    bool rotates = false;
    if constexpr (QKV) {
        head = (int)(first / after.head_dim);
        const int within = (int)(first % after.head_dim);
        const bool is_value = head >= after.n_heads + after.n_kv_heads;
        rotates = after.rope_theta != nullptr && !is_value;      // (the launcher checks that the packing pairs exactly these heads)
        lower_dim = rotates ? within / 2 : within;
        upper_dim = rotates ? after.head_dim / 2 + within / 2 : within + 8;
    }

    const int k_tiles = K / 32;
    const int per_wave = (k_tiles + WAVES - 1) / WAVES;
    const int first_tile = wave * per_wave;
    const int count = max(0, min(per_wave, k_tiles - first_tile));     // tiles of this wavefront

    constexpr int CHAINS = MT <= 2 ? 2 : 1;                     // accumulators per output tile, used in turn
    floatx4 chain[CHAINS][MT];
#pragma unroll
    for (int h = 0; h < CHAINS; ++h)
#pragma unroll
        for (int m = 0; m < MT; ++m) chain[h][m] = floatx4{0.f, 0.f, 0.f, 0.f};

    const bf16* w_ptr = w + ((long)blockIdx.x * k_tiles + first_tile) * 512 + lane * 8;
    const bf16* x_ptr[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) x_ptr[m] = x + (long)min(m * 16 + r, M - 1) * K + first_tile * 32 + c * 8;   // rows beyond M: the last row again

    auto load_w = [&](bf16x8 (&regs)[JL], int tile) {
#pragma unroll
        for (int j = 0; j < JL; ++j) regs[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w_ptr + (long)(tile + j) * 512));
    };
    auto load_x = [&](bf16x8 (&regs)[MT][JL], int tile) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < JL; ++j) regs[m][j] = *reinterpret_cast<const bf16x8*>(x_ptr[m] + (tile + j) * 32);
    };
    auto multiply = [&](const bf16x8 (&wregs)[JL], const bf16x8 (&xregs)[MT][JL]) {
#pragma unroll
        for (int j = 0; j < JL; ++j)
#pragma unroll
            for (int m = 0; m < MT; ++m)
                chain[j % CHAINS][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wregs[j], xregs[m][j], chain[j % CHAINS][m], 0, 0, 0);
    };

    // The sums of squares of this wavefront's eighth of the tiles of columns (lane (r, c): row r, every
    // fourth tile from c): the first ones are asked for now and added up when the stream of w has run through.
    const int square_tiles = AROUND && norm.squares_in ? norm.tiles_in : 0;
    const bool out_ahead = AROUND && MODE == MODE_ACCUMULATE && N % 4 == 0;     // 16 bytes of out per lane, aligned
    auto square_range = [&](int thread, int& begin, int& end) {
        const int per = (square_tiles + WAVES - 1) / WAVES;
        begin = thread / XRT_WAVE * per + thread % XRT_WAVE / 16;
        end = min(square_tiles, (thread / XRT_WAVE + 1) * per);
    };
    float early_squares[AROUND ? SQUARES_AHEAD : 1] = {};
    if constexpr (AROUND) {
        if (square_tiles > 0) {
            int begin, end;
            square_range(threadIdx.x, begin, end);
            const float* row = norm.squares_in + min(r, M - 1);
#pragma unroll
            for (int i = 0; i < SQUARES_AHEAD; ++i) {
                const int t = begin + 4 * i;
                early_squares[i] = t < end ? row[(long)t * XRT_SQUARES_STRIDE] : 0.f;
            }
        }
    }
    int early_pos = 0, early_slot = -1, early_block = -1;
    float early_theta = 1.f;
    // asked for behind the first loads of w (those have the longer way), used after the first products
    auto ask_early = [&]() {
        if constexpr (QKV) {
            const int token = min(r, M - 1);
            if (rotates && wave < 4) {                          // the lane's four angles, one per wavefront; read by wavefront 0
                early_pos = after.positions[token];
                early_theta = after.rope_theta[min(lower_dim + (c % 2) * 4 + wave, after.rope_dim / 2 - 1)];
            }
            if (wave == 4 && c == 0) {
                early_pos = after.positions[token];
                if (after.k_cache && head >= after.n_heads) early_slot = after.slots[token];
            }
        }
        if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
            if (wave == 0) {                                    // the wavefront that writes the tile
                if (out_ahead) {
                    const long column = min(first + c * 4, (long)N - 4);
                    load_to_lds(out, (unsigned)(((long)min(r, M - 1) * N + column) * 4), lds_address(&early_out[0]));
                }
                if (norm.squares_out) {                         // the tile's 16 gains: N is a multiple of 8 here
                    const unsigned at = norm.gain_dtype == XRT_F32 ? (unsigned)min(first + lane, (long)N - 1) * 4u
                                                                   : (unsigned)min(first + 2 * lane, (long)N - 2) * 2u;
                    load_dword_to_lds(norm.gain, at, lds_address(&early_gain[0]));
                }
            }
        }
    };
    auto use_early = [&]() {
        if constexpr (QKV) {
            if (rotates && wave < 4) {
                const float angle = (float)early_pos * after.rope_scale / early_theta;
                sincosf(angle, &early_sin[lane][wave], &early_cos[lane][wave]);     // lanes c and c ^ 2 hold the two halves of a pair
            }
            if (wave == 4 && c == 0 && early_slot >= 0)
                early_block = after.block_table[(long)early_slot * after.table_stride + early_pos / XRT_BLOCK_TOKENS];
        }
    };
    auto place_in_cache = [&]() {
        if constexpr (QKV) {
            if (wave == 4 && c == 0) {
                long base = -1;
                if (early_block >= 0 && early_block < after.n_blocks) {
                    const int kv_head = (head - after.n_heads) % after.n_kv_heads;
                    base = ((long)early_block * after.n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * after.head_dim;
                }
                early_base[r] = base;
                early_within[r] = early_pos % XRT_BLOCK_TOKENS;
            }
        }
    };
    // (the lane's place is worked out again from the thread index, behind a fence for the compiler's
    // eyes, so that nothing of this is kept in registers while the stream of w runs)
    auto add_squares = [&]() {
        if constexpr (AROUND) {
            if constexpr (MODE == MODE_ACCUMULATE) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // what went to LDS has arrived
            if (square_tiles > 0) {
                int thread = threadIdx.x;
                asm volatile("" : "+v"(thread));
                int begin, end;
                square_range(thread, begin, end);
                const int row = min(thread % 16, M - 1);
                float sum = 0.f;
#pragma unroll
                for (int i = 0; i < SQUARES_AHEAD; ++i) sum += early_squares[i];
                for (int t = begin + 4 * SQUARES_AHEAD; t < end; t += 4)
                    sum += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + row];
                sum += __shfl_xor(sum, 16);
                sum += __shfl_xor(sum, 32);
                if (thread % XRT_WAVE < 16) squares[thread / XRT_WAVE][thread % 16] = sum;   // read after the barrier of the first tile below
            }
        }
    };

    // Steps of two tiles run through a pipeline of two register sets: while the matrix cores consume
    // one step, the loads of the next are in flight. The steady-state loop body has no branch.
    const int full = count / JL;
    if (full > 0) {
        bf16x8 w_a[JL], w_b[JL];
        bf16x8 x_a[MT][JL], x_b[MT][JL];
        load_x(x_a, 0);
        load_w(w_a, 0);
        ask_early();
        int i = 0;
        for (; i + 2 < full; i += 2) {
            load_x(x_b, (i + 1) * JL);
            load_w(w_b, (i + 1) * JL);
            multiply(w_a, x_a);
            if constexpr (QKV) if (i == 0) use_early();
            load_x(x_a, (i + 2) * JL);
            load_w(w_a, (i + 2) * JL);
            multiply(w_b, x_b);
        }
        if (full - i == 2) {
            load_x(x_b, (i + 1) * JL);
            load_w(w_b, (i + 1) * JL);
            multiply(w_a, x_a);
            multiply(w_b, x_b);
        } else {
            multiply(w_a, x_a);
        }
        if constexpr (QKV) if (full <= 2) use_early();         // the loop above did not run
    } else {
        ask_early();
        use_early();
    }
    if (count % JL != 0) {                                      // the wavefront's odd last tile
        const int tile = full * JL;
        const bf16x8 a = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w_ptr + (long)tile * 512));
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const bf16x8 b = *reinterpret_cast<const bf16x8*>(x_ptr[m] + tile * 32);
            chain[0][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, chain[0][m], 0, 0, 0);
        }
    }
    place_in_cache();
    add_squares();
    floatx4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        acc[m] = chain[0][m];
#pragma unroll
        for (int h = 1; h < CHAINS; ++h) acc[m] += chain[h][m];
    }

    // add the wavefronts' partial sums tile by tile, in wavefront order; the wavefront that sums a tile writes it
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int slot = MT > 1 ? m & 1 : 0;
        partial[slot][wave][lane] = acc[m];
        __syncthreads();
        if (wave != m % WAVES) continue;                        // (slots alternate: a slot is rewritten two tiles later, after the next barrier)
        floatx4 total = partial[slot][0][lane];
#pragma unroll
        for (int other = 1; other < WAVES; ++other) total += partial[slot][other][lane];
        const int mm = m * 16 + r;                              // the lane holds row mm of x ...
        float g[4] = {total[0], total[1], total[2], total[3]};  // ... against packed rows first + c * 4 + i of w
        if constexpr (AROUND) {
            if (square_tiles > 0) {                             // the rows of x were not divided by their rms yet
                float sum = squares[0][r];
#pragma unroll
                for (int other = 1; other < WAVES; ++other) sum += squares[other][r];
                const float inv_rms = 1.0f / sqrtf(sum / (float)norm.width_in + norm.eps);
#pragma unroll
                for (int i = 0; i < 4; ++i) g[i] *= inv_rms;
            }
        }
        if constexpr (QKV) {
            // as the two-kernel way does it: the projection rounded to bfloat16, then rotated in float32
            float mine[4], other[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                mine[i] = to_float(from_float<bf16>(g[i]));
                other[i] = __shfl_xor(mine[i], 32);
            }
            struct alignas(8) Four { bf16 e[4]; } packed;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float value = mine[i];
                if (rotates) {
                    const float cosine = early_cos[lane][i], sine = early_sin[lane][i];
                    value = c < 2 ? mine[i] * cosine - other[i] * sine : other[i] * sine + mine[i] * cosine;
                }
                packed.e[i] = from_float<bf16>(value);
            }
            if (mm < M) {
                const int dim = (c < 2 ? lower_dim : upper_dim) + (c % 2) * 4;
                *reinterpret_cast<Four*>((bf16*)out + (long)mm * N + (long)head * after.head_dim + dim) = packed;
                const long base = early_base[r];
                if (base >= 0) {
                    const int within = early_within[r];
                    if (head < after.n_heads + after.n_kv_heads) {
                        *reinterpret_cast<Four*>(after.k_cache + base + cache_key_offset(within, dim, after.head_dim)) = packed;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            after.v_cache[base + cache_value_offset(dim + i, within, after.head_dim)] = packed.e[i];
                    }
                }
            }
            continue;
        }
        if constexpr (MODE == MODE_GATED) {
            // lanes c = 0, 1 hold the gate sums of outputs first / 2 + c * 4 + i, lanes c = 2, 3 the up sums of the same
            float u[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) u[i] = __shfl_xor(g[i], 32);
            const long nn = first / 2 + c * 4;
            if (c < 2 && mm < M) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nn + i < N) out[(long)mm * N + nn + i] = from_float<TO>(gate_activation<sizeof(TO) == 2>(g[i], activation) * u[i]);
            }
            continue;
        }
        const long nn = logical_row(packing, first + c * 4);    // four rows of one packed piece of 8 stay together
        float fresh[4] = {0.f, 0.f, 0.f, 0.f};                  // what out holds now, 0 outside of it
        bool written = false;
        if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
            if (out_ahead && mm < M && nn + 3 < N) {            // the four values in one piece, as they came
                const floatx4 before = early_out[lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) fresh[i] = before[i] + g[i];
                *reinterpret_cast<floatx4*>(out + (long)mm * N + nn) = floatx4{fresh[0], fresh[1], fresh[2], fresh[3]};
                written = true;
            }
        }
        if (mm < M && !written) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (nn + i >= N) continue;                      // (fresh stays 0: it counts for nothing below)
                TO* dst = out + (long)mm * N + nn + i;
                if constexpr (MODE == MODE_STORE) *dst = from_float<TO>(g[i]);
                if constexpr (MODE == MODE_ACCUMULATE) {
                    fresh[i] = to_float(*dst) + g[i];
                    *dst = from_float<TO>(fresh[i]);
                }
            }
        }
        if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
            if (norm.squares_out) {
                float sum = fmaf(fresh[3], fresh[3], fmaf(fresh[2], fresh[2], fmaf(fresh[1], fresh[1], fresh[0] * fresh[0])));
                sum += __shfl_xor(sum, 16);
                sum += __shfl_xor(sum, 32);
                if (mm < M) {
                    if (c == 0) norm.squares_out[(long)blockIdx.x * XRT_SQUARES_STRIDE + mm] = sum;
                    if (nn + 3 < N) {                           // N is a multiple of 8: all four or none
                        struct alignas(8) Four { bf16 e[4]; } scaled;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float gain = norm.gain_dtype == XRT_F32 ? early_gain[c * 4 + i]
                                                                          : to_float(((const bf16*)early_gain)[c * 4 + i]);
                            scaled.e[i] = from_float<bf16>(fresh[i] * gain);
                        }
                        *reinterpret_cast<Four*>((bf16*)norm.scaled_out + (long)mm * N + nn) = scaled;
                    }
                }
            }
        }
    }
}


// The same product where a workgroup has several groups of 16 packed rows to do and k is so short that a wavefront's
// eighth of x fits its registers (RESIDENT tiles of 32 columns: k up to 4096): the workgroup walks its groups, x is
// read once, and only w streams, its ring of tiles running on from one group into the next. With 9 to 16 rows of x
// the kernel above reads as many bytes of x from L2 as of w from memory, for every group again (gate/up of 14336 pairs
// at 16 rows: 49 us; this way 41 us; a vocabulary of 128256 rows 212 against 168 us); with 8 rows or fewer, half of
// x's rows are repeats and it gains nothing. Store and gated epilogues, rows of x with or without their RMSNorm's division.
constexpr int RESIDENT = 16;       // tiles of x that a wavefront keeps
constexpr int RING = 4;            // tiles of w on their way per wavefront
static_assert(RESIDENT % RING == 0, "the ring of w tiles runs on from group to group");

template <int MODE, typename TO>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, 2) gemm_packed_resident_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    const Packing packing, const LinearNorm norm, int activation) {
    static_assert(MODE == MODE_STORE || MODE == MODE_GATED, "store or gated");
    __shared__ floatx4 partial[2][WAVES][XRT_WAVE];
    __shared__ float square_parts[WAVES * XRT_WAVE / 16][16];
    __shared__ float inv_rms[16];
    const int lane = threadIdx.x % XRT_WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / XRT_WAVE);
    const int r = lane % 16, c = lane / 16;
    const int k_tiles = K / 32;
    const int per_wave = (k_tiles + WAVES - 1) / WAVES;
    const int first_tile = wave * per_wave;
    const int count = max(0, min(per_wave, k_tiles - first_tile));      // at most RESIDENT: the launcher checks
    const long rows_w = MODE == MODE_GATED ? 2L * N : N;
    const long groups = (rows_w + 15) / 16;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    bf16x8 x_tiles[RESIDENT], ring[RING];
    const bf16* x_ptr = x + (long)min(r, M - 1) * K + first_tile * 32 + c * 8;      // rows beyond M: the last row again
    auto w_of = [&](long group) { return w + (group * k_tiles + first_tile) * 512 + lane * 8; };
    auto ask = [&](const bf16* from, int tile, bool there) {
        return (there && tile < count) ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(from + (long)tile * 512)) : zero;
    };
    {
        const bf16* first = w_of(blockIdx.x);                  // the grid has no more workgroups than w has groups
#pragma unroll
        for (int t = 0; t < RING; ++t) ring[t] = ask(first, t, true);
    }
#pragma unroll
    for (int t = 0; t < RESIDENT; ++t) x_tiles[t] = t < count ? *reinterpret_cast<const bf16x8*>(x_ptr + t * 32) : zero;
    // 1 / rms of the rows of x, if they come without it: every thread adds up its share of the sums of squares (asked
    // for now, behind the first tiles of w and x), the shares meet at the first group's barrier, and the wavefront that
    // writes the first group leaves the result for those that write the others. A fixed order throughout.
    float my_squares = 0.f;
    if (norm.squares_in != nullptr) {
        const int row = threadIdx.x % 16, part = threadIdx.x / 16;
        for (int t = part; t < norm.tiles_in; t += WAVES * XRT_WAVE / 16)
            my_squares += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + min(row, M - 1)];
    }

    int turn = 0;
    for (long group = blockIdx.x; group < groups; group += gridDim.x, ++turn) {
        const bf16* here = w_of(group);
        const long next = group + gridDim.x;
        const bool more = next < groups;
        const bf16* there = w_of(more ? next : group);
        floatx4 chain[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int t = 0; t < RESIDENT; ++t) {
            const bf16x8 a = ring[t % RING];
            // the tile RING further on: of this group, or the first ones of the next, before this group's sums meet
            ring[t % RING] = t + RING < RESIDENT ? ask(here, t + RING, true) : ask(there, t + RING - RESIDENT, more);
            chain[t % 2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, x_tiles[t], chain[t % 2], 0, 0, 0);
        }
        const int slot = turn & 1;                              // a slot is rewritten two groups later, after the next barrier
        partial[slot][wave][lane] = chain[0] + chain[1];
        if (turn == 0 && norm.squares_in != nullptr) square_parts[threadIdx.x / 16][threadIdx.x % 16] = my_squares;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // (not __syncthreads: that would wait for the ring's loads too)
        if (wave != turn % WAVES) continue;                     // the wavefronts take turns at adding up and writing
        floatx4 total = partial[slot][0][lane];
#pragma unroll
        for (int other = 1; other < WAVES; ++other) total += partial[slot][other][lane];
        float g[4] = {total[0], total[1], total[2], total[3]};  // row r of x against packed rows group * 16 + c * 4 + i of w
        if (norm.squares_in != nullptr) {
            float by;
            if (turn == 0) {
                float sum = 0.f;
                for (int other = 0; other < WAVES * XRT_WAVE / 16; ++other) sum += square_parts[other][r];
                by = 1.0f / sqrtf(sum / (float)norm.width_in + norm.eps);
                if (c == 0) inv_rms[r] = by;                    // read after later barriers
            } else {
                by = inv_rms[r];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) g[i] *= by;
        }
        if constexpr (MODE == MODE_GATED) {
            float u[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) u[i] = __shfl_xor(g[i], 32);
            const long nn = group * 8 + c * 4;                  // lanes c = 0, 1 hold the gate sums, c = 2, 3 the up sums of the same outputs
            if (c < 2 && r < M) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nn + i < N) out[(long)r * N + nn + i] = from_float<TO>(gate_activation<sizeof(TO) == 2>(g[i], activation) * u[i]);
            }
        } else {
            const long nn = logical_row(packing, group * 16 + c * 4);
            if (r < M) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nn + i < N) out[(long)r * N + nn + i] = from_float<TO>(g[i]);
            }
        }
    }
}

// Whether the kernel above takes the product, and with how many workgroups. Two fit a compute unit, and a compute
// unit works its workgroups off at one pace: what counts is the number of groups that the busiest one has.
int resident_grid(int M, int K, long rows_w, int mode, bool norm_out, bool after) {
    const long groups = (rows_w + 15) / 16;
    if (M <= 8 || M > 16 || mode == MODE_ACCUMULATE || norm_out || after) return 0;
    if ((K / 32 + WAVES - 1) / WAVES > RESIDENT || groups < 512) return 0;
    constexpr int ONCE = XRT_COMPUTE_UNITS, TWICE = 2 * XRT_COMPUTE_UNITS;
    const long most_once = (groups + ONCE - 1) / ONCE, most_twice = 2 * ((groups + TWICE - 1) / TWICE);
    return most_twice < most_once ? TWICE : ONCE;
}

template <int MT, typename TO>
int launch_mode(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const Packing& packing,
                const LinearNorm& norm, const QkvAfter* after, hipStream_t s) {
    const long rows_w = mode == MODE_GATED ? 2L * N : N;
    const unsigned grid = (unsigned)((rows_w + 15) / 16);
    const dim3 block(WAVES * XRT_WAVE);
    const QkvAfter none = {};
    if constexpr (MT == 1) {
        if (const int resident = resident_grid(M, K, rows_w, mode, norm.squares_out != nullptr || norm.scaled_out != nullptr, after != nullptr)) {
            if (mode == MODE_STORE)
                gemm_packed_resident_kernel<MODE_STORE, TO><<<resident, block, 0, s>>>(x, w, out, M, N, K, packing, norm, activation);
            else
                gemm_packed_resident_kernel<MODE_GATED, TO><<<resident, block, 0, s>>>(x, w, out, M, N, K, packing, norm, activation);
            XRT_LAUNCH_CHECK("linear (packed, x resident)");
            return 0;
        }
        if (after) {
            if constexpr (sizeof(TO) == 2) {
                gemm_packed_kernel<1, MODE_STORE, TO, 2><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, *after, activation);
                XRT_LAUNCH_CHECK("linear (packed, q/k/v)");
                return 0;
            }
        } else if (norm.squares_in || norm.squares_out) {
            if (mode == MODE_STORE)
                gemm_packed_kernel<1, MODE_STORE, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
            else if (mode == MODE_ACCUMULATE)
                gemm_packed_kernel<1, MODE_ACCUMULATE, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
            else
                gemm_packed_kernel<1, MODE_GATED, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
            XRT_LAUNCH_CHECK("linear (packed, with norm)");
            return 0;
        }
    }
    if (after || norm.squares_in || norm.squares_out) {
        xrt_set_error("linear (packed): a norm's half or what follows a q/k/v projection takes one tile of rows");
        return 1;
    }
    if (mode == MODE_STORE)
        gemm_packed_kernel<MT, MODE_STORE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
    else if (mode == MODE_ACCUMULATE)
        gemm_packed_kernel<MT, MODE_ACCUMULATE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
    else
        gemm_packed_kernel<MT, MODE_GATED, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, packing, norm, none, activation);
    XRT_LAUNCH_CHECK("linear (packed)");
    return 0;
}

template <typename TO>
int launch_tiles(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const Packing& packing,
                 const LinearNorm& norm, const QkvAfter* after, hipStream_t s) {
    switch ((M + 15) / 16) {
        case 1: return launch_mode<1, TO>(x, w, out, M, N, K, mode, activation, packing, norm, after, s);
        case 2: return launch_mode<2, TO>(x, w, out, M, N, K, mode, activation, packing, norm, after, s);
        case 3: return launch_mode<3, TO>(x, w, out, M, N, K, mode, activation, packing, norm, after, s);
        default: return launch_mode<4, TO>(x, w, out, M, N, K, mode, activation, packing, norm, after, s);
    }
}

}  // namespace

// Whether this kernel takes the product (bfloat16 operands assumed by the caller): few rows, a packed w
// whose grouping of rows fits the epilogue.
bool xrt_linear_packed_accepts(const void* a, const void* w, int M, int K, int mode, const Packing* packing) {
    if (!packing || !is_packed(*packing) || M < 1 || M > 64 || K % 32 != 0) return false;
    if ((uintptr_t)a % 16 != 0 || (uintptr_t)w % 16 != 0) return false;
    return (mode == MODE_GATED) == (packing->kind == XRT_PACK_GATED);
}

bool xrt_linear_packed_takes_norm(int M) { return M <= 16; }

// What follows a q/k/v projection: the packing must pair exactly the heads that the rotation turns, over the whole head.
bool xrt_linear_packed_takes_qkv(int M, int N, const Packing& packing, const QkvAfter& after) {
    if (M > 16 || after.head_dim % 16 != 0 || N != (after.n_heads + 2 * after.n_kv_heads) * after.head_dim) return false;
    const int rotated = after.rope_theta ? after.n_heads + after.n_kv_heads : 0;
    if (after.rope_theta && after.rope_dim != after.head_dim) return false;
    if (packing.kind == XRT_PACK_TILES) return rotated == 0;
    return packing.kind == XRT_PACK_ROTARY && packing.head_dim == after.head_dim && packing.rotated_heads == rotated;
}

int xrt_linear_packed(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                      const Packing* packing, const LinearNorm* norm, const QkvAfter* after, hipStream_t s) {
    const LinearNorm none = {};
    if (norm && !xrt_linear_packed_takes_norm(M)) {
        xrt_set_error("linear (packed): the norm around a product takes at most 16 rows, found %d", M);
        return 1;
    }
    if (after && !(xrt_linear_packed_takes_qkv(M, N, *packing, *after) && mode == MODE_STORE && out_dtype == XRT_BF16)) {
        xrt_set_error("linear (packed): M=%d N=%d mode %d is no q/k/v projection whose epilogue this kernel does", M, N, mode);
        return 1;
    }
    if (norm && mode == MODE_ACCUMULATE && packing->kind != XRT_PACK_TILES) {
        xrt_set_error("linear (packed): an accumulating product next to a norm takes a w packed in plain tiles");
        return 1;
    }
    if (norm && norm->squares_out && N % 16 != 0) {
        xrt_set_error("linear (packed): sums of squares per tile of 16 columns need N = %d to be a multiple of 16", N);
        return 1;
    }
    const LinearNorm& around = norm ? *norm : none;
    if (out_dtype == XRT_F32) return launch_tiles<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, activation, *packing, around, after, s);
    return launch_tiles<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, activation, *packing, around, after, s);
}
