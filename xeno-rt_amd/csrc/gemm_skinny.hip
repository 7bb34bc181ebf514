// Matrix product for few rows (M <= 64: decode steps and short prompts), bfloat16 operands,
// float32 accumulation on the matrix cores: out[m, n] = sum_k x[m, k] * w[n, k].
//
// Such a product is bound by reading w once from HBM, so the kernel is built around that
// stream. A workgroup of 8 wavefronts owns 16 (or 32, or fewer than 16: see balanced_rows) rows of w. Each wavefront takes one
// eighth of K and streams its part of those rows straight from global memory into the A
// operand of v_mfma_f32_16x16x32_bf16: a 64-wide K step is two load instructions, and in each
// the four lanes (r, 0..3) of a row read 64 contiguous bytes of it, so that a step takes one
// whole cache line of each of 16 rows. (Steps of 128 cost 20 registers more and with them
// wavefronts in flight: 2 us more on the largest product; steps of 32, half a line at a time,
// are a quarter slower.) The B operand holds the
// activations x (16 rows of m per tile), read with the same K permutation. Loads carry no
// branches (addresses are clamped into the operands instead), run one step ahead of the
// matrix cores, and the products of a step go to accumulators that do not wait on each other:
// all three matter, because a wavefront that stalls stops issuing its next loads.
// The eight partial sums are added in wavefront order through LDS, so the result does not
// depend on timing. Epilogues: store (bfloat16 or float32), accumulate into float32, or the
// gated pair silu(gate) * up with the two halves of w (rows n and n + N).
//
// Around an RMSNorm between two products (x += a w^T; y = rmsnorm(x) * gain; z = y v^T) a step of
// up to 16 rows needs no kernel for the norm: the accumulating product also writes
// bfloat16(x * gain) and, for every tile of columns, each row's sum of squares; the product
// after it takes those as its activations and multiplies its rows by 1 / sqrt(sum / width + eps).
// The sums are added in a fixed order (tiles in eighths by wavefront, then wavefront by wavefront).
//
// The q/k/v projection of such a step can also rotate q and k and write k and v into the cache: a
// tile of 16 rows of w is then the 8 + 8 rows of a head whose outputs the rotation pairs (dims d and
// d + rope_dim / 2), so that a lane finds its partner 32 lanes away.
#include "common.h"
#include "xrt_hip.h"
#include "gemm_skinny.h"
#include "activation.h"

namespace {

using LinearNorm = xrt_linear_norm;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVES = 8;
constexpr int KSTEP = 64;         // K covered by one step of a wavefront
constexpr int JL = KSTEP / 32;   // load instructions per operand tile and step: 4 lane groups x 8 elements each
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };


// MT: tiles of 16 rows of x; RT: tiles of 16 rows of w per wavefront; GATED doubles the w tiles.
// With one tile of x (the common decode case) the kernel is held to 128 registers at most (it takes
// 62 to 92), so that two to four workgroups fit a compute unit: the stream from HBM needs the
// wavefronts in flight.
// EXTRA 1: the kernel also does its share of an RMSNorm before or after the product (one tile of x,
// one tile of w per wavefront); 2: and what follows a q/k/v projection. Kernels without keep their
// registers for the stream.
template <int MT, int RT, int MODE, typename TO, int EXTRA = 0>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, (MT == 1 ? 4 : 2)) gemm_skinny_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K, int given_rows,
    const LinearNorm norm, const QkvAfter after, int activation) {
    // given_rows: rows of w that a workgroup's tile holds, 16 or fewer (with RT == 1): the host picks them so
    // that the workgroups divide evenly among the compute units. Lanes beyond read the tile's last row again.
    // After a q/k/v projection the tiles of the query heads have 16 rows and come first; those of the key
    // and value heads have after.kv_rows (16 or 8).
    constexpr bool AROUND = EXTRA != 0, QKV = EXTRA == 2;
    static_assert(!AROUND || (MT == 1 && RT == 1), "the norm around a product: one tile of x, one of w per wavefront");
    static_assert(!QKV || (MODE == MODE_STORE && sizeof(TO) == 2), "after a q/k/v projection: a bfloat16 store");
    constexpr int WT = RT * (MODE == MODE_GATED ? 2 : 1);       // w tiles per wavefront
    constexpr int SQUARES_AHEAD = 8;                            // sums of squares a lane asks for when the kernel starts
    __shared__ floatx4 partial[RT * MT > 1 ? 2 : 1][WAVES][XRT_WAVE];
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
    int rows = given_rows;
    const long n0 = (long)blockIdx.x * (RT == 1 ? rows : 16 * RT);
    // after a q/k/v projection: the tile's head, and the dims of the head its rows 0..7 and 8..15 make
    int head = 0, lower_dim = 0, upper_dim = 8;
    bool rotates = false;
    if constexpr (QKV) {
        // a tile: rows / 2 dims and the rows / 2 that the rotation pairs them with (beyond rope_dim and in
        // value heads: the rows / 2 dims that follow), in lanes r = 0.. and r = 8..
        const int query_tiles = after.n_heads * (after.head_dim / 16);
        int tile = blockIdx.x;
        rows = 16;
        if (tile >= query_tiles) {
            tile -= query_tiles;
            rows = after.kv_rows;
        }
        const int tiles_per_head = after.head_dim / rows;
        head = (blockIdx.x >= query_tiles ? after.n_heads : 0) + tile / tiles_per_head;
        const int s = tile % tiles_per_head;
        const bool is_value = head >= after.n_heads + after.n_kv_heads;
        const int rotated_tiles = (after.rope_theta && !is_value) ? after.rope_dim / rows : 0;
        rotates = s < rotated_tiles;
        lower_dim = rotates ? rows / 2 * s : rows * s;
        upper_dim = rotates ? after.rope_dim / 2 + rows / 2 * s : rows * s + rows / 2;
    }

    const int steps = (K + KSTEP - 1) / KSTEP;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int k_begin = wave * steps_per_wave * KSTEP;
    const int k_end = min(K, k_begin + steps_per_wave * KSTEP);

    // CHAINS accumulators per output tile, used in turn and added at the end
    constexpr int CHAINS = MT <= 2 ? 2 : 1;
    floatx4 chain[CHAINS][WT][MT];
#pragma unroll
    for (int h = 0; h < CHAINS; ++h)
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m) chain[h][t][m] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Clamped addresses: a row of w beyond N (or of x beyond M) reads the last row, and what it
    // contributes lands in outputs that are never written.
    const bf16* w_ptr[WT];
#pragma unroll
    for (int t = 0; t < WT; ++t) {
        const int rt = t % RT, half = t / RT;                   // half 1: the "up" rows of a gated product
        long n = min(n0 + rt * 16 + min(r, rows - 1), (long)N - 1);
        if constexpr (QKV) n = (long)head * after.head_dim + (r < 8 ? lower_dim + min(r, rows / 2 - 1) : upper_dim + min(r - 8, rows / 2 - 1));
        w_ptr[t] = w + (n + (long)half * N) * K + c * 8;
    }
    const bf16* x_ptr[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) x_ptr[m] = x + (long)min(m * 16 + r, M - 1) * K + c * 8;

    auto load_w = [&](bf16x8 (&regs)[WT][JL], int kb) {
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int j = 0; j < JL; ++j) regs[t][j] = *reinterpret_cast<const bf16x8*>(w_ptr[t] + kb + j * 32);
    };
    auto load_x = [&](bf16x8 (&regs)[MT][JL], int kb) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < JL; ++j) regs[m][j] = *reinterpret_cast<const bf16x8*>(x_ptr[m] + kb + j * 32);
    };
    auto multiply = [&](const bf16x8 (&wregs)[WT][JL], const bf16x8 (&xregs)[MT][JL]) {
#pragma unroll
        for (int j = 0; j < JL; ++j)
#pragma unroll
            for (int t = 0; t < WT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    chain[j % CHAINS][t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wregs[t][j], xregs[m][j], chain[j % CHAINS][t][m], 0, 0, 0);
    };

    // Whole steps along k run through a pipeline of two register sets: while the matrix
    // cores consume one step, the loads of the next are in flight. The steady-state loop body has
    // no branch; the last one or two steps are peeled off.
    // The sums of squares of this wavefront's eighth of the tiles (lane (r, c): row r, every fourth
    // tile from c): the first ones are asked for now and added up when the stream of w has run through.
    const int square_tiles = AROUND && norm.squares_in ? norm.tiles_in : 0;
    const bool out_ahead = AROUND && MODE == MODE_ACCUMULATE && N % 4 == 0;     // 16 bytes of out per lane, aligned
    auto square_range = [&](int thread, int& first, int& end) {
        const int per_wave = (square_tiles + WAVES - 1) / WAVES;
        first = thread / XRT_WAVE * per_wave + thread % XRT_WAVE / 16;
        end = min(square_tiles, (thread / XRT_WAVE + 1) * per_wave);
    };
    float early_squares[AROUND ? SQUARES_AHEAD : 1] = {};
    if constexpr (AROUND) {
        if (square_tiles > 0) {
            int first, end;
            square_range(threadIdx.x, first, end);
            const float* row = norm.squares_in + min(r, M - 1);
#pragma unroll
            for (int i = 0; i < SQUARES_AHEAD; ++i) {
                const int t = first + 4 * i;
                early_squares[i] = t < end ? row[(long)t * XRT_SQUARES_STRIDE] : 0.f;
            }
        }
    }
    int early_pos = 0, early_slot = -1, early_block = -1;
    float early_theta = 1.f;
    // (what the accumulating epilogue reads is asked for behind the first loads of w: those have the longer way)
    auto ask_early = [&]() {
        if constexpr (QKV) {
            // only asked for here: a wavefront that waited for them now would have one step of w in flight meanwhile
            const int token = min(r, M - 1);
            if (rotates && wave < 4) {                          // the lane's four angles, one per wavefront; read by wavefront 0
                early_pos = after.positions[token];
                early_theta = after.rope_theta[min(lower_dim + (c % 2) * 4 + wave, after.rope_dim / 2 - 1)];   // (lanes beyond a tile of 8 rows: unused)
            }
            if (wave == 4 && c == 0) {
                early_pos = after.positions[token];
                if (after.k_cache && head >= after.n_heads) early_slot = after.slots[token];
            }
        }
        if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
            if (wave == 0) {                                    // the wavefront that writes the tile
                if (out_ahead) {
                    const long column = min(n0 + c * 4, (long)N - 4);
                    load_to_lds(out, (unsigned)(((long)min(r, M - 1) * N + column) * 4), lds_address(&early_out[0]));
                }
                if (norm.squares_out) {                         // the tile's 16 gains: N is a multiple of 8 here
                    const unsigned at = norm.gain_dtype == XRT_F32 ? (unsigned)min(n0 + lane, (long)N - 1) * 4u
                                                                   : (unsigned)min(n0 + 2 * lane, (long)N - 2) * 2u;
                    load_dword_to_lds(norm.gain, at, lds_address(&early_gain[0]));
                }
            }
        }
    };
    // After the first step of w has been multiplied, what was asked for above has arrived as well (loads come
    // back in order): sine and cosine are worked out, and the cache block's number is asked for, while the
    // next steps are in flight.
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
    // when the stream of w has run through: where the lane's token lies in the cache (-1: nowhere)
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
                int first, end;
                square_range(thread, first, end);
                const int row = min(thread % 16, M - 1);
                float sum = 0.f;
#pragma unroll
                for (int i = 0; i < SQUARES_AHEAD; ++i) sum += early_squares[i];
                for (int t = first + 4 * SQUARES_AHEAD; t < end; t += 4)
                    sum += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + row];
                sum += __shfl_xor(sum, 16);
                sum += __shfl_xor(sum, 32);
                if (thread % XRT_WAVE < 16) squares[thread / XRT_WAVE][thread % 16] = sum;   // read after the barrier of the first tile below
            }
        }
    };

    const int full = max(0, (min(k_end, K / KSTEP * KSTEP) - k_begin) / KSTEP);     // whole steps of this wavefront
    if (full > 0) {
        bf16x8 w_a[WT][JL], w_b[WT][JL];
        bf16x8 x_a[MT][JL], x_b[MT][JL];
        load_x(x_a, k_begin);
        load_w(w_a, k_begin);
        ask_early();
        int i = 0;
        for (; i + 2 < full; i += 2) {
            load_x(x_b, k_begin + (i + 1) * KSTEP);
            load_w(w_b, k_begin + (i + 1) * KSTEP);
            multiply(w_a, x_a);
            if constexpr (QKV) if (i == 0) use_early();
            load_x(x_a, k_begin + (i + 2) * KSTEP);
            load_w(w_a, k_begin + (i + 2) * KSTEP);
            multiply(w_b, x_b);
        }
        if (full - i == 2) {
            load_x(x_b, k_begin + (i + 1) * KSTEP);
            load_w(w_b, k_begin + (i + 1) * KSTEP);
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
    // what is left of K when it is no multiple of the step: one guarded step, in the wavefront that owns it
    const int tail_begin = k_begin + full * KSTEP;
    if (tail_begin < k_end) {
#pragma unroll
        for (int j = 0; j < JL; ++j) {
            const bool inside = tail_begin + j * 32 + c * 8 + 8 <= K;       // K is a multiple of 8
            bf16x8 b[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m)
                b[m] = inside ? *reinterpret_cast<const bf16x8*>(x_ptr[m] + tail_begin + j * 32) : bf16x8{};
#pragma unroll
            for (int t = 0; t < WT; ++t) {
                const bf16x8 a = inside ? *reinterpret_cast<const bf16x8*>(w_ptr[t] + tail_begin + j * 32) : bf16x8{};
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    chain[0][t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[m], chain[0][t][m], 0, 0, 0);
            }
        }
    }
    place_in_cache();
    add_squares();
    floatx4 acc[WT][MT];
#pragma unroll
    for (int t = 0; t < WT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            acc[t][m] = chain[0][t][m];
#pragma unroll
            for (int h = 1; h < CHAINS; ++h) acc[t][m] += chain[h][t][m];
        }

    // add the wavefronts' partial sums tile by tile, in wavefront order; the wavefront that
    // sums a tile also writes it
    constexpr int TILES = RT * MT;
#pragma unroll
    for (int tile = 0; tile < TILES; ++tile) {
        const int rt = tile / MT, m = tile % MT;
        const int slot = RT * MT > 1 ? tile & 1 : 0;
        float4 gate_sum = {0.f, 0.f, 0.f, 0.f}, up_sum = {0.f, 0.f, 0.f, 0.f};
        constexpr int PASSES = MODE == MODE_GATED ? 2 : 1;
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            partial[slot][wave][lane] = acc[rt + pass * RT][m];
            __syncthreads();
            if (wave == tile % WAVES) {
                floatx4 total = partial[slot][0][lane];
#pragma unroll
                for (int other = 1; other < WAVES; ++other) total += partial[slot][other][lane];
                if (pass == 0) gate_sum = {total[0], total[1], total[2], total[3]};
                else up_sum = {total[0], total[1], total[2], total[3]};
            }
            if (PASSES == 2) __syncthreads();
        }
        if (wave == tile % WAVES) {
            const int mm = m * 16 + r;                          // lane holds column m = lane % 16 ...
            const long nn = n0 + rt * 16 + c * 4;               // ... and rows n = (lane / 16) * 4 + i
            float g[4] = {gate_sum.x, gate_sum.y, gate_sum.z, gate_sum.w};
            float u[4] = {up_sum.x, up_sum.y, up_sum.z, up_sum.w};
            if constexpr (AROUND) {
                if (square_tiles > 0) {                         // the rows of a were not divided by their rms yet
                    float total = squares[0][r];
#pragma unroll
                    for (int other = 1; other < WAVES; ++other) total += squares[other][r];
                    const float inv_rms = 1.0f / sqrtf(total / (float)norm.width_in + norm.eps);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { g[i] *= inv_rms; u[i] *= inv_rms; }
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
                if (mm < M && (c % 2) * 4 < rows / 2) {          // (rows / 2 is 8 or 4: all four of a lane's dims or none)
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
            float fresh[4] = {0.f, 0.f, 0.f, 0.f};              // what out holds now, 0 outside of it
            bool written = false;
            if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
                if (out_ahead && mm < M && nn < N && c * 4 < rows) {   // the four values in one piece, as they came (rows is a multiple of 4 here)
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
                    if (nn + i >= N || c * 4 + i >= rows) continue;        // (fresh stays 0: it counts for nothing below)
                    TO* dst = out + (long)mm * N + nn + i;
                    if constexpr (MODE == MODE_STORE) *dst = from_float<TO>(g[i]);
                    if constexpr (MODE == MODE_ACCUMULATE) {
                        fresh[i] = to_float(*dst) + g[i];
                        *dst = from_float<TO>(fresh[i]);
                    }
                    if constexpr (MODE == MODE_GATED) *dst = from_float<TO>(gate_activation<sizeof(TO) == 2>(g[i], activation) * u[i]);
                }
            }
            if constexpr (AROUND && MODE == MODE_ACCUMULATE) {
                if (norm.squares_out) {
                    float sum = fmaf(fresh[3], fresh[3], fmaf(fresh[2], fresh[2], fmaf(fresh[1], fresh[1], fresh[0] * fresh[0])));
                    sum += __shfl_xor(sum, 16);
                    sum += __shfl_xor(sum, 32);
                    if (mm < M) {
                        if (c == 0) norm.squares_out[(long)blockIdx.x * XRT_SQUARES_STRIDE + mm] = sum;
                        if (nn < N && c * 4 < rows) {           // N is a multiple of 8 and rows one of 4: all four or none
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
        // slots alternate, and a slot is rewritten only two tiles later, after this tile's barrier
    }
}

// Rows of w in a workgroup's tile (one tile of 16 or fewer per wavefront).
// Workgroups are dealt out to the 256 compute units in turn, and the kernel takes about as long as the
// compute unit with the most of them: 384 tiles of 16 rows take as long as 512. So, with as many rounds
// over the compute units as tiles of 16 rows make, a tile gets the fewest rows (8 at least) that still fit
// those rounds: 512 tiles of 12 rows instead of 384 of 16. (More rounds of still smaller tiles lose to what
// every workgroup costs, about as much as three rows.) Accumulating products take a multiple of 4 (their
// epilogue moves four values at a time). The tile that the rotation after a q/k/v projection pairs stays at
// 16 (768 tiles of 8 rows were slower than 384 of 16).
int balanced_rows(int N, int mode) {
    const long rounds = ((N + 15) / 16 + XRT_COMPUTE_UNITS - 1) / XRT_COMPUTE_UNITS;
    int rows = (int)((N + XRT_COMPUTE_UNITS * rounds - 1) / (XRT_COMPUTE_UNITS * rounds));
    if (mode == MODE_ACCUMULATE) rows = (rows + 3) / 4 * 4;
    return rows < 8 ? 8 : (rows > 16 ? 16 : rows);
}

template <int MT, int RT, typename TO>
int launch_mode(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const LinearNorm& norm,
                const QkvAfter* after, hipStream_t s) {
    const int rows = RT == 1 && !after ? balanced_rows(N, mode) : 16;
    unsigned grid = (unsigned)(RT == 1 ? (N + rows - 1) / rows : (N + 16 * RT - 1) / (16 * RT));
    QkvAfter then = after ? *after : QkvAfter{};
    if (after) {
        // tiles of 8 rows for the key and value heads, if the compute unit with the most rows then has fewer
        // (32 query heads and 8 key/value heads of 128: 256 + 256 tiles, 24 rows each, instead of 384 of 16)
        const long query_tiles = (long)after->n_heads * (after->head_dim / 16), kv_tiles = 2L * after->n_kv_heads * (after->head_dim / 16);
        auto most = [&](int kv_rows) {                          // rows of the fullest compute unit (the first)
            const long kv = kv_tiles * (16 / kv_rows);
            long sum = 0;
            for (long group = 0; group < query_tiles + kv; group += XRT_COMPUTE_UNITS) sum += group < query_tiles ? 16 : kv_rows;
            return sum;
        };
        then.kv_rows = most(8) < most(16) ? 8 : 16;
        grid = (unsigned)(query_tiles + kv_tiles * (16 / then.kv_rows));
    }
    const dim3 block(WAVES * XRT_WAVE);
    const QkvAfter none = {};
    if constexpr (MT == 1 && RT == 1) {
        if (after) {
            if constexpr (sizeof(TO) == 2) {
                gemm_skinny_kernel<1, 1, MODE_STORE, TO, 2><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, then, activation);
                XRT_LAUNCH_CHECK("linear (skinny, q/k/v)");
                return 0;
            }
        } else if (norm.squares_in || norm.squares_out) {
            if (mode == MODE_STORE)
                gemm_skinny_kernel<1, 1, MODE_STORE, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
            else if (mode == MODE_ACCUMULATE)
                gemm_skinny_kernel<1, 1, MODE_ACCUMULATE, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
            else
                gemm_skinny_kernel<1, 1, MODE_GATED, TO, 1><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
            XRT_LAUNCH_CHECK("linear (skinny, with norm)");
            return 0;
        }
    }
    if (after) {
        xrt_set_error("linear (skinny): what follows a q/k/v projection takes one tile of bfloat16 rows");
        return 1;
    }
    if (mode == MODE_STORE)
        gemm_skinny_kernel<MT, RT, MODE_STORE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
    else if (mode == MODE_ACCUMULATE)
        gemm_skinny_kernel<MT, RT, MODE_ACCUMULATE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
    else if constexpr (RT == 1)
        gemm_skinny_kernel<MT, RT, MODE_GATED, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K, rows, norm, none, activation);
    else {
        xrt_set_error("linear (skinny): a gated product takes one row tile per wavefront");
        return 1;
    }
    XRT_LAUNCH_CHECK("linear (skinny)");
    return 0;
}

template <typename TO>
int launch_tiles(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const LinearNorm& norm,
                 const QkvAfter* after, hipStream_t s) {
    const int mt = (M + 15) / 16;
    // two row tiles per wavefront keep more loads in flight and halve the reads of x, if enough
    // workgroups remain to fill the chip
    // (with three or four tiles of x the reads of x from L2 outweigh those of w from HBM: then
    // the wider tile pays as soon as it leaves most compute units a workgroup)
    const bool around = norm.squares_in || norm.squares_out || after;
    const bool wide = !around && mode != MODE_GATED && (N / 32) >= (mt >= 3 ? 160 : 1024);
#define XRT_SKINNY(MT_) (wide ? launch_mode<MT_, 2, TO>(x, w, out, M, N, K, mode, activation, norm, after, s) : launch_mode<MT_, 1, TO>(x, w, out, M, N, K, mode, activation, norm, after, s))
    switch (mt) {
        case 1: return XRT_SKINNY(1);
        case 2: return XRT_SKINNY(2);
        case 3: return XRT_SKINNY(3);
        default: return XRT_SKINNY(4);
    }
#undef XRT_SKINNY
}

}  // namespace

// Whether the skinny kernel takes this product (bfloat16 operands assumed by the caller).
bool xrt_linear_skinny_accepts(const void* a, const void* w, int M, int K) {
    return M >= 1 && M <= 64 && K % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
}

// The norm around a product needs one tile of x.
bool xrt_linear_skinny_takes_norm(int M) { return M <= 16; }

// Tiles of columns for which an accumulating product of N columns writes sums of squares.
int xrt_linear_skinny_norm_tiles(int N) { const int rows = balanced_rows(N, MODE_ACCUMULATE); return (N + rows - 1) / rows; }

// So does what follows a q/k/v projection; and the rotation must pair whole groups of 8 dims.
bool xrt_linear_skinny_takes_qkv(int M, int N, const QkvAfter& after) {
    return M <= 16 && after.head_dim % 16 == 0 && N == (after.n_heads + 2 * after.n_kv_heads) * after.head_dim &&
           (after.rope_theta == nullptr || (after.rope_dim % 16 == 0 && after.rope_dim <= after.head_dim));
}

int xrt_linear_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                      const LinearNorm* norm, const QkvAfter* after, hipStream_t s) {
    const LinearNorm none = {};
    if (norm && !xrt_linear_skinny_takes_norm(M)) {
        xrt_set_error("linear (skinny): the norm around a product takes at most 16 rows, found %d", M);
        return 1;
    }
    if (after && !(xrt_linear_skinny_takes_qkv(M, N, *after) && mode == MODE_STORE && out_dtype == XRT_BF16)) {
        xrt_set_error("linear (skinny): M=%d N=%d mode %d is no q/k/v projection whose epilogue this kernel does", M, N, mode);
        return 1;
    }
    const LinearNorm& around = norm ? *norm : none;
    if (out_dtype == XRT_F32) return launch_tiles<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, activation, around, after, s);
    return launch_tiles<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, activation, around, after, s);
}
