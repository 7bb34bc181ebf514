// Matrix product for many rows (prefill), bfloat16 operands, float32 accumulation on the
// matrix cores: out[m, n] = sum_k a[m, k] * w[n, k]; both operands are contiguous along k.
//
// A workgroup computes a BM x BN tile of the output with v_mfma_f32_32x32x16_bf16. Tiles of
// a and w travel through LDS, several steps ahead of the matrix cores, with one barrier per
// step. When K is a multiple of 64 they are loaded from global memory straight into LDS, in a
// swizzled layout; otherwise they pass through registers into rows padded by 16 bytes (64 wide
// in k, the last tile filled with zeros). Either layout keeps the 16-byte operand reads of
// consecutive rows in different banks. Each wavefront owns a (BM/WM) x (BN/WN) part of the
// tile and keeps its accumulators in registers for the whole K loop.
//
// Workgroup ids are remapped so that the workgroups that run on one XCD (ids are dealt
// round-robin to the 8 XCDs) work on neighbouring tiles and share their operands in that
// XCD's L2.
//
// Epilogues: store (bfloat16 or float32), accumulate into float32, or the gated pair
// silu(gate) * up: then the w tile holds BN/2 gate rows and the BN/2 up rows that belong to
// them (rows n and n + N of w), arranged so that each wavefront holds both of a pair.
#include <climits>
#include <cstdlib>
#include "packing.h"
#include "gemm_skinny.h"
#include "activation.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 64;
constexpr int PITCH = BK + 8;          // bf16 elements per LDS row
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };


// One tile of the product, by one workgroup: `id` is the workgroup's number among those that work
// on the output columns from n_first on, tiles_m x tiles_n of them.
// The rows of a that come without their RMSNorm's division (see xrt_linear_norm in xrt_hip.h): the sums of
// squares per tile of 16 columns, from which a tile of up to 64 rows works out 1 / rms of its rows and
// multiplies its sums by it before the epilogue. squares null: nothing of the kind.
struct RowScale { const float* squares; int tiles; int width; float eps; int activation; };     // (activation: of a gated epilogue)

template <int BM, int BN, int WM, int WN, int MODE, int DK, int STAGES, typename TO>
__device__ __forceinline__ void gemm_tile(
    const bf16* __restrict__ a, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    int id, int tiles_m, int tiles_n, int n_first, int k_per_split, const Packing packing, const RowScale scale = RowScale{}) {
    constexpr int THREADS = WM * WN * XRT_WAVE;
    constexpr int WAVE_M = BM / WM, WAVE_N = BN / WN;        // part of the tile owned by one wavefront
    constexpr int TM = WAVE_M / 32, TN = WAVE_N / 32;        // 32x32 accumulator tiles of a wavefront
    constexpr int CHUNKS_A = BM * BK / 8 / THREADS;          // 16-byte chunks each thread moves per step
    constexpr int CHUNKS_B = BN * BK / 8 / THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    bf16* lds_a = reinterpret_cast<bf16*>(lds_raw);                    // [2][BM][PITCH]; laid out differently on the direct path
    bf16* lds_b = lds_a + 2 * BM * PITCH;                              // [2][BN][PITCH]

    // ---- which tile: ids are dealt to XCDs round-robin; give each XCD a contiguous run of tiles,
    // and walk a run m-fastest inside panels of 8 n-tiles so that concurrent tiles share w
    const int total = tiles_m * tiles_n;
    {
        const int xcds = 8;
        const int per = (total + xcds - 1) / xcds;
        const int mapped = (id % xcds) * per + id / xcds;
        id = mapped;
    }
    if (id >= total) return;
    constexpr int PANEL = 8;
    const int panel = id / (PANEL * tiles_m);
    const int in_panel = id % (PANEL * tiles_m);
    const int panel_width = min(PANEL, tiles_n - panel * PANEL);
    const int tile_n = panel * PANEL + in_panel % panel_width;
    const int tile_m = in_panel / panel_width;
    const long m0 = (long)tile_m * BM;
    constexpr int BN_OUT = MODE == MODE_GATED ? BN / 2 : BN;          // output columns of a tile
    const long n0 = n_first + (long)tile_n * BN_OUT;      // this launch covers output columns from n_first on

    const int tid = threadIdx.x, lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    const int wave_m = wave / WN, wave_n = wave % WN;

    // Row of w behind row r of the tile. In the gated mode the rows that one wavefront owns are
    // half gate rows and half the up rows of the same outputs (rows n and n + N of w), so that the
    // pair meets in that wavefront's registers. Rows beyond the operands are clamped to the last
    // row: loads then need no guard, and what such a row contributes lands in outputs that are
    // not written.
    auto w_row = [&](int r) -> long {
        if constexpr (MODE == MODE_GATED) {
            constexpr int HALF = WAVE_N / 2;
            const int within = r % WAVE_N;
            return min(n0 + (r / WAVE_N) * HALF + within % HALF, (long)N - 1) + (long)(within / HALF) * N;
        } else {
            return min(n0 + r, (long)N - 1);
        }
    };
    // 1 / rms of the tile's rows, if the rows of a come without it. The sums of squares are asked for now,
    // all at once (a thread takes four neighbouring rows of every sixteenth tile, 16 bytes a load), and added
    // up after the main loop, when they have long arrived.
    constexpr int SQUARE_LOADS = 16;                           // tiles of 16 columns per thread: rows of up to 16 * 16 * 16 columns
    __shared__ float row_scale[BM <= 64 ? 64 : 1];
    __shared__ float row_parts[BM <= 64 ? 16 : 1][64];
    float4 early_squares[BM <= 64 ? SQUARE_LOADS : 1];
    const bool scaled = BM <= 64 && scale.squares != nullptr;
    if constexpr (BM <= 64) {
        if (scaled && tid < 256) {
#pragma unroll
            for (int u = 0; u < SQUARE_LOADS; ++u) {
                const int t = tid / 16 + 16 * u;
                early_squares[u] = t < scale.tiles
                    ? *reinterpret_cast<const float4*>(scale.squares + (long)t * XRT_SQUARES_STRIDE + (tid % 16) * 4)
                    : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if constexpr (DK != 0) {
        // Tiles go from global memory straight into LDS (global_load_lds_dwordx4): no registers and
        // no LDS write instructions in between. Tiles are DK wide in k and LDS holds STAGES of
        // them: while one is multiplied, the next is complete and STAGES - 2 more are on their
        // way. One load instruction of a wavefront fills 64 consecutive 16-byte places of LDS,
        // lane by lane, which is 64 / CHUNKS whole rows; rows can therefore not be padded. Instead
        // the chunks of a row are stored in permuted places, place = chunk ^ swizzle(row), and
        // each lane fetches the chunk that belongs in its place. The swizzles are chosen so that
        // the operand reads of 8 and of 16 consecutive rows at one chunk fall into different
        // 16-byte bank groups.
        constexpr int CHUNKS = DK / 8;                             // 16-byte chunks per row: 4 or 8
        constexpr int ROWS = 64 / CHUNKS;                          // rows that one load instruction fills
        constexpr int WAVES = WM * WN;
        // load instructions per wavefront and tile; where the row blocks do not divide among the
        // wavefronts, the spare instructions fetch the last block once more (same bytes, same place)
        constexpr int BLOCKS_A = BM / ROWS, BLOCKS_B = BN / ROWS;
        constexpr int LOADS_A = (BLOCKS_A + WAVES - 1) / WAVES, LOADS_B = (BLOCKS_B + WAVES - 1) / WAVES;
        constexpr int SLICES = DK / 16;
        static_assert(DK == 32 || DK == 64, "swizzles exist for rows of 4 and of 8 chunks");
        static_assert(BM % ROWS == 0 && BN % ROWS == 0, "tile rows do not divide into load instructions");
        bf16* stage_a = lds_a;                                     // [STAGES][BM][DK]
        bf16* stage_b = lds_a + STAGES * BM * DK;                  // [STAGES][BN][DK]
        auto swizzle_of = [](int r) { return CHUNKS == 4 ? (r / 2 % 4) ^ (r / 8 % 2) : (r % 8) ^ (r / 8 % 2); };
        const int sub = lane / CHUNKS;                             // row within the rows of one instruction
        auto chunk_of = [&](int row) { return ((lane % CHUNKS) ^ swizzle_of(row)) * 8; };   // what belongs in this lane's place
        unsigned off_a[LOADS_A], off_b[LOADS_B];                   // bytes
#pragma unroll
        for (int i = 0; i < LOADS_A; ++i) {
            const int r = min(i * WAVES + wave, BLOCKS_A - 1) * ROWS + sub;
            off_a[i] = (unsigned)(min(m0 + r, (long)M - 1) * K + chunk_of(r)) * 2u;
        }
        // A packed w is copied as it lies: an instruction takes one whole tile of the packing (16 packed rows x 32
        // columns, a contiguous kilobyte, lane by lane), and the stage holds the tile's groups of 16 packed rows
        // one after another, two tiles of 32 columns each. The 16 lanes that read an operand's 16 rows at one
        // piece of 8 columns then read 256 contiguous bytes of LDS. (Fetched piece by piece into the layout of
        // rows contiguous along k, every four lanes would touch four cache lines: a fifth slower, measured.)
        // The tile's rows are then packed rows first_packed .. + BN, and the epilogue finds the outputs they make.
        const bool packed_b = is_packed(packing);
        const long first_packed = MODE == MODE_GATED ? 2 * n0 : n0;
        const long last_group = ((MODE == MODE_GATED ? 2L * N : (long)N) + 15) / 16 - 1;
#pragma unroll
        for (int i = 0; i < LOADS_B; ++i) {
            const int block = min(i * WAVES + wave, BLOCKS_B - 1);
            if (packed_b) {
                const long group = min(first_packed / 16 + block / 2, last_group);       // groups beyond the matrix: the last one again
                off_b[i] = (unsigned)(((group * (K / 32) + block % 2) * 512 + lane * 8) * 2);
            } else {
                const int r = block * ROWS + sub;
                off_b[i] = (unsigned)(w_row(r) * K + chunk_of(r)) * 2u;
            }
        }
        // a step of k0 columns along k moves a row contiguous along k by k0 elements, a packed one by k0 / 32 tiles
        const unsigned w_step = packed_b ? 32u : 2u;                // bytes per column of k
        const int wave_uniform = __builtin_amdgcn_readfirstlane(wave);
        const unsigned lds_a0 = lds_address(stage_a), lds_b0 = lds_address(stage_b);
        auto issue = [&](int stage, int k0) {
#pragma unroll
            for (int i = 0; i < LOADS_A; ++i) {
                const int block = min(i * WAVES + wave_uniform, BLOCKS_A - 1);
                load_to_lds(a, off_a[i] + (unsigned)k0 * 2u, lds_a0 + (unsigned)((stage * BM + block * ROWS) * DK * 2));
            }
#pragma unroll
            for (int i = 0; i < LOADS_B; ++i) {
                const int block = min(i * WAVES + wave_uniform, BLOCKS_B - 1);
                load_to_lds(w, off_b[i] + (unsigned)k0 * w_step, lds_b0 + (unsigned)((stage * BN + block * ROWS) * DK * 2));
            }
        };
        const int swizzle = swizzle_of(lane % 16);                 // of every row this lane reads: they differ by multiples of 32
        // where this lane finds its piece of the w operand for each slice, from the start of its wavefront's rows
        int b_place[SLICES];
#pragma unroll
        for (int slice = 0; slice < SLICES; ++slice)
            b_place[slice] = packed_b ? (lane % 32 / 16 * 2 + slice / 2) * 512 + ((slice % 2 * 2 + lane / 32) * 16 + lane % 16) * 8
                                      : (lane % 32) * DK + ((slice * 2 + lane / 32) ^ swizzle) * 8;
        // operands of one 16-wide slice of k: TM row blocks of a, TN row blocks of w
        struct Operands { bf16x8 a[TM], b[TN]; };
        auto read = [&](Operands& r, int stage, int slice) {
            const int place = ((slice * 2 + lane / 32) ^ swizzle) * 8;
            const bf16* tile_a = stage_a + ((long)stage * BM + wave_m * WAVE_M + lane % 32) * DK + place;
            const bf16* tile_b = stage_b + ((long)stage * BN + wave_n * WAVE_N) * DK + b_place[slice];
#pragma unroll
            for (int i = 0; i < TM; ++i) r.a[i] = *reinterpret_cast<const bf16x8*>(tile_a + i * 32 * DK);
#pragma unroll
            for (int j = 0; j < TN; ++j) r.b[j] = *reinterpret_cast<const bf16x8*>(tile_b + j * 32 * DK);
        };
        auto multiply = [&](const Operands& r) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(r.a[i], r.b[j], acc[i][j], 0, 0, 0);
        };
        // The launcher sends only K that is a multiple of DK here. Every step issues the loads of
        // the tile STAGES - 1 steps ahead; beyond the end of k it repeats the last tile (into a
        // stage nobody uses any more), so that the number of loads in flight is the same at every
        // wait. The operands of each slice are read from LDS while the matrix cores work on the
        // slice before it, across the barrier too: the first slice of the next tile is read right
        // after the barrier, under the products of the last slice of this one.
        constexpr int AHEAD = STAGES - 1;
        constexpr int IN_FLIGHT = (AHEAD - 1) * (LOADS_A + LOADS_B);   // loads that may be outstanding when the next tile is needed
        // a launch with several grid rows splits k among them: row y takes k_per_split from
        // y * k_per_split on (less at the end) and writes its sums to the y-th copy of out
        const int k_begin = blockIdx.y * k_per_split;
        const int steps = min(k_per_split, K - k_begin) / DK;
        const int last_k = k_begin + (steps - 1) * DK;
        out += (long)blockIdx.y * M * N;
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) issue(i, min(k_begin + i * DK, last_k));
        wait_loads_and_barrier<IN_FLIGHT>();                      // tile 0 is in LDS
        Operands operands[2];
        read(operands[0], 0, 0);
        for (int t = 0; t < steps; ++t) {
            issue((t + AHEAD) % STAGES, min(k_begin + (t + AHEAD) * DK, last_k));   // that stage was read in step t-1, before the last barrier
#pragma unroll
            for (int slice = 0; slice + 1 < SLICES; ++slice) {
                read(operands[(slice + 1) % 2], t % STAGES, slice + 1);
                __builtin_amdgcn_sched_barrier(0);                // keeps the reads ahead of the products that hide them
                multiply(operands[slice % 2]);
                __builtin_amdgcn_sched_barrier(0);
            }
            wait_loads_and_barrier<IN_FLIGHT>();                  // tile t+1 has arrived from every wavefront, tile t has been read by all
            read(operands[0], (t + 1) % STAGES, 0);               // after the last step: a repeated tile, not used
            __builtin_amdgcn_sched_barrier(0);
            multiply(operands[(SLICES - 1) % 2]);
        }
        wait_loads_and_barrier<0>();                              // nothing lands in LDS after this
    } else {
        // element offsets of this thread's chunks from the operands' bases (32 bits: the launcher checks)
        unsigned off_a[CHUNKS_A], off_b[CHUNKS_B];
    #pragma unroll
        for (int i = 0; i < CHUNKS_A; ++i) {
            const int chunk = tid + i * THREADS;
            off_a[i] = (unsigned)(min(m0 + chunk / 8, (long)M - 1) * K + (chunk % 8) * 8);
        }
    #pragma unroll
        for (int i = 0; i < CHUNKS_B; ++i) {
            const int chunk = tid + i * THREADS;
            off_b[i] = (unsigned)weight_offset(packing, w_row(chunk / 8), (chunk % 8) * 8, K);
        }
        const unsigned w_step = is_packed(packing) ? 16u : 1u;      // elements per column of k (tiles are 64 wide here: whole tiles of the packing)

        struct Stage { bf16x8 a[CHUNKS_A], b[CHUNKS_B]; };
        auto fetch = [&](Stage& stage, int k0) {                  // a whole tile of 64 along k, no guards
    #pragma unroll
            for (int i = 0; i < CHUNKS_A; ++i) stage.a[i] = *reinterpret_cast<const bf16x8*>(a + (off_a[i] + (unsigned)k0));
    #pragma unroll
            for (int i = 0; i < CHUNKS_B; ++i) stage.b[i] = *reinterpret_cast<const bf16x8*>(w + (off_b[i] + (unsigned)k0 * w_step));
        };
        auto fetch_tail = [&](Stage& stage, int k0) {             // the last tile when K is no multiple of 64: zeros beyond K
    #pragma unroll
            for (int i = 0; i < CHUNKS_A; ++i) {
                const int k = k0 + ((tid + i * THREADS) % 8) * 8;
                stage.a[i] = k + 8 <= K ? *reinterpret_cast<const bf16x8*>(a + (off_a[i] + (unsigned)k0)) : bf16x8{};
            }
    #pragma unroll
            for (int i = 0; i < CHUNKS_B; ++i) {
                const int k = k0 + ((tid + i * THREADS) % 8) * 8;
                stage.b[i] = k + 8 <= K ? *reinterpret_cast<const bf16x8*>(w + (off_b[i] + (unsigned)k0 * w_step)) : bf16x8{};
            }
        };
        auto stash = [&](const Stage& stage, int buffer) {
    #pragma unroll
            for (int i = 0; i < CHUNKS_A; ++i) {
                const int chunk = tid + i * THREADS, r = chunk / 8, kc = chunk % 8;
                *reinterpret_cast<bf16x8*>(lds_a + ((long)buffer * BM + r) * PITCH + kc * 8) = stage.a[i];
            }
    #pragma unroll
            for (int i = 0; i < CHUNKS_B; ++i) {
                const int chunk = tid + i * THREADS, r = chunk / 8, kc = chunk % 8;
                *reinterpret_cast<bf16x8*>(lds_b + ((long)buffer * BN + r) * PITCH + kc * 8) = stage.b[i];
            }
        };

        // The products of one LDS buffer. `between` runs ahead of them: it writes the next tile to the
        // other LDS buffer and requests the tile after it. (Placing it halfway through the products
        // was measured slower: the fetched registers then stay live across all of them.)
        auto compute = [&](int buffer, auto between) {
            const bf16* tile_a = lds_a + ((long)buffer * BM + wave_m * WAVE_M + lane % 32) * PITCH + (lane / 32) * 8;
            const bf16* tile_b = lds_b + ((long)buffer * BN + wave_n * WAVE_N + lane % 32) * PITCH + (lane / 32) * 8;
    #pragma unroll
            for (int ks = 0; ks < BK / 16; ++ks) {
                if (ks == 0) between();
                bf16x8 ra[TM], rb[TN];
    #pragma unroll
                for (int i = 0; i < TM; ++i) ra[i] = *reinterpret_cast<const bf16x8*>(tile_a + i * 32 * PITCH + ks * 16);
    #pragma unroll
                for (int j = 0; j < TN; ++j) rb[j] = *reinterpret_cast<const bf16x8*>(tile_b + j * 32 * PITCH + ks * 16);
    #pragma unroll
                for (int i = 0; i < TM; ++i)
    #pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ra[i], rb[j], acc[i][j], 0, 0, 0);
            }
        };
        auto nothing = [] {};

        // Tiles travel global -> registers -> LDS ahead of the matrix cores. During step t the
        // registers hold tile t+1 (fetched a step ago): it is written into the LDS buffer that step t-1
        // has finished with, the registers are refilled with tile t+2, and tile t is multiplied. The steady-state loop has no branch.
        const int whole = K / BK;                                 // tiles of 64 that lie inside K
        Stage s0;
        if (whole > 0) {
            fetch(s0, 0);
            stash(s0, 0);
            if (whole > 1) fetch(s0, BK);
            __syncthreads();
            int t = 0;                                            // LDS buffer 0 holds tile t, the registers tile t+1
            for (; t + 3 < whole; t += 2) {
                compute(0, [&] { stash(s0, 1); fetch(s0, (t + 2) * BK); });
                __syncthreads();
                compute(1, [&] { stash(s0, 0); fetch(s0, (t + 3) * BK); });
                __syncthreads();
            }
            const int left = whole - t;                           // 1, 2 or 3
            compute(0, [&] { if (left >= 2) stash(s0, 1); if (left == 3) fetch(s0, (t + 2) * BK); });
            if (left >= 2) {
                __syncthreads();
                compute(1, [&] { if (left == 3) stash(s0, 0); });
            }
            if (left == 3) {
                __syncthreads();
                compute(0, nothing);
            }
        }
        if (whole * BK < K) {
            fetch_tail(s0, whole * BK);
            __syncthreads();                                      // everyone is done with buffer 0
            stash(s0, 0);
            __syncthreads();
            compute(0, nothing);
        }
    }

    // ---- epilogue: accumulator element e of tile (i, j) is row (e/4)*8 + (lane/32)*4 + e%4, column lane%32
    if constexpr (BM <= 64) {
        if (scaled) {                                          // the same for all threads of the workgroup
            if (tid < 256) {
                float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int u = 0; u < SQUARE_LOADS; ++u) {
                    sum.x += early_squares[u].x; sum.y += early_squares[u].y; sum.z += early_squares[u].z; sum.w += early_squares[u].w;
                }
                // rows of more than 4096 columns: the tiles beyond, one after the other
                for (int t = tid / 16 + 16 * SQUARE_LOADS; t < scale.tiles; t += 16) {
                    const float4 more = *reinterpret_cast<const float4*>(scale.squares + (long)t * XRT_SQUARES_STRIDE + (tid % 16) * 4);
                    sum.x += more.x; sum.y += more.y; sum.z += more.z; sum.w += more.w;
                }
                *reinterpret_cast<float4*>(&row_parts[tid / 16][(tid % 16) * 4]) = sum;
            }
            __syncthreads();
            if (tid < 64) {
                float total = 0.f;
#pragma unroll
                for (int part = 0; part < 16; ++part) total += row_parts[part][tid];
                row_scale[tid] = 1.0f / sqrtf(total / (float)scale.width + scale.eps);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float by = row_scale[wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4];
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j][e] *= by;
                }
        }
    }
    // With a packed w that was copied as it lies (whole tiles along k), column q of the tile is packed row
    // first_packed + q of w: the outputs are found through the packing.
    const bool packed_columns = DK != 0 && is_packed(packing);
    if (MODE == MODE_GATED && packed_columns) {
        // A group of 16 packed rows: the gate rows of 8 outputs, then their up rows: a lane's partner is 8 lanes away.
        // The two share the work: of two neighbouring rows of the tile the lane with the gates finishes the first
        // (with its partner's up sum), the lane with the ups the second (with its partner's gate sum).
        const int q = lane % 32;
        const bool has_gates = q % 16 < 8;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const long n = n0 + (wave_n * WAVE_N + j * 32) / 2 + q / 16 * 8 + q % 8;
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    const float first = acc[i][j][e], second = acc[i][j][e + 1];
                    const float partner_first = from_eight_lanes_away(first), partner_second = from_eight_lanes_away(second);
                    const float gate = has_gates ? first : partner_second, up = has_gates ? partner_first : second;
                    const long m = m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4 + (has_gates ? 0 : 1);
                    if (m < M && n < N) out[m * (long)N + n] = from_float<TO>(gate_activation<sizeof(TO) == 2>(gate, scale.activation) * up);
                }
            }
    } else if constexpr (MODE == MODE_GATED) {
        static_assert(TN % 2 == 0, "a wavefront holds as many gate blocks as up blocks");
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN / 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const long m = m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4;
                    const long n = n0 + wave_n * (WAVE_N / 2) + j * 32 + lane % 32;
                    if (m < M && n < N) out[m * (long)N + n] = from_float<TO>(gate_activation<sizeof(TO) == 2>(acc[i][j][e], scale.activation) * acc[i][j + TN / 2][e]);
                }
    } else {
        long column[TN];                                        // the output column of this lane in each block of 32
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            column[j] = n0 + wave_n * WAVE_N + j * 32 + lane % 32;
            if (packed_columns) column[j] = column[j] < N ? logical_row(packing, column[j]) : (long)N;     // (packed rows beyond w make nothing)
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            // When accumulating, what the outputs of one row block hold is read in one go, from
            // addresses clamped into the matrix, before any of them is written: guarded, each
            // read would wait for the one before it.
            float before[TN][16];
            if constexpr (MODE == MODE_ACCUMULATE) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const long m = min(m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4, (long)M - 1);
                        const long n = min(column[j], (long)N - 1);
                        before[j][e] = to_float(out[m * (long)N + n]);
                    }
            }
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const long m = m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4;
                    const long n = column[j];
                    if (m < M && n < N) {
                        if constexpr (MODE == MODE_STORE) out[m * (long)N + n] = from_float<TO>(acc[i][j][e]);
                        else out[m * (long)N + n] = from_float<TO>(before[j][e] + acc[i][j][e]);
                    }
                }
        }
    }
}

template <int BM, int BN, int WM, int WN, int MODE, int DK, int STAGES, typename TO>
__global__ void __launch_bounds__(WM * WN * XRT_WAVE) gemm_mfma_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    int tiles_m, int tiles_n, int n_first, int k_per_split, const Packing packing, const RowScale scale) {
    gemm_tile<BM, BN, WM, WN, MODE, DK, STAGES, TO>(a, w, out, M, N, K, blockIdx.x, tiles_m, tiles_n, n_first, k_per_split, packing, scale);
}

// Two tile shapes in one launch: the first `large_blocks` workgroups take 256 x 256 tiles of the
// output columns below `split`, the others 128 x 256 tiles of the columns from `split` on. The
// large tiles are handed out first and fill whole rounds over the compute units; the small ones
// follow as compute units become free, so the last round is full of half-sized work and there is
// no gap between the two.
template <int MODE, typename TO>
__global__ void __launch_bounds__(8 * XRT_WAVE) gemm_mfma_mixed_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    int large_blocks, int large_tiles_m, int large_tiles_n, int split, int small_tiles_m, int small_tiles_n,
    const Packing packing, const RowScale scale) {
    if ((int)blockIdx.x < large_blocks)
        gemm_tile<256, 256, 2, 4, MODE, 64, 2, TO>(a, w, out, M, N, K, blockIdx.x, large_tiles_m, large_tiles_n, 0, K, packing, scale);
    else
        gemm_tile<128, 256, 2, 4, MODE, 64, 2, TO>(a, w, out, M, N, K, blockIdx.x - large_blocks, small_tiles_m,
                                                   small_tiles_n, split, K, packing, scale);
}

// Launches the tiles of output columns [n_first, n_first + n_count).
template <int BM, int BN, int WM, int WN, int MODE, int DK, int STAGES, typename TO>
int launch_kernel(const bf16* a, const bf16* w, TO* out, int M, int N, int K, int n_first, int n_count, const Packing& packing,
                  hipStream_t s, int splits = 1, int k_per_split = 0, const RowScale scale = RowScale{}) {
    constexpr int BN_OUT = MODE == MODE_GATED ? BN / 2 : BN;
    constexpr int THREADS = WM * WN * XRT_WAVE;
    constexpr size_t staging = DK != 0 ? (size_t)STAGES * (BM + BN) * DK * sizeof(bf16) : (size_t)2 * (BM + BN) * PITCH * sizeof(bf16);
    constexpr size_t lds = staging;
    static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a compute unit");
    auto kernel = gemm_mfma_kernel<BM, BN, WM, WN, MODE, DK, STAGES, TO>;
    static bool configured = false;          // per instantiation
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        XRT_REQUIRE(e == hipSuccess, "linear (mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (n_count + BN_OUT - 1) / BN_OUT;
    const int total = tiles_m * tiles_n;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);           // a whole number of rounds over the XCDs
    XRT_REQUIRE(splits == 1 || DK != 0, "linear (mfma): only whole tiles along k can be split");
    XRT_REQUIRE(scale.squares == nullptr || (BM <= 64 && splits == 1), "linear (mfma): rows are scaled by tiles of up to 64 rows that see all of k");
    kernel<<<dim3(grid, splits), THREADS, lds, s>>>(a, w, out, M, N, K, tiles_m, tiles_n, n_first,
                                                    splits == 1 ? K : k_per_split, packing, scale);
    XRT_LAUNCH_CHECK("linear (mfma)");
    return 0;
}

template <int BM, int BN, int WM, int WN, int MODE, typename TO>
int launch(const bf16* a, const bf16* w, TO* out, int M, int N, int K, int n_first, int n_count, const Packing& packing, int activation,
           hipStream_t s) {
    const RowScale plain = {nullptr, 0, 0, 0.f, activation};
    // Whole tiles along k go straight into LDS, in two stages of 64; a ragged last tile needs the
    // path through registers. (Four stages of 32 keep a load in flight for longer but meet at
    // twice as many barriers, and measured slower: 1.03 against 1.06 to 1.16 PFLOP/s on the large tiles.)
    if (K % 64 == 0) return launch_kernel<BM, BN, WM, WN, MODE, 64, 2, TO>(a, w, out, M, N, K, n_first, n_count, packing, s, 1, 0, plain);
    if constexpr (BM == 256 && BN == 256 || BM == 128 && BN == 128) {
        return launch_kernel<BM, BN, WM, WN, MODE, 0, 0, TO>(a, w, out, M, N, K, n_first, n_count, packing, s, 1, 0, plain);
    } else {
        XRT_REQUIRE(false, "linear (mfma): this tile takes only K that is a multiple of 64 (K=%d)", K);
    }
}

// Time of tiles of `tile_elements` outputs, in units of tile elements per compute unit: the tiles
// run in rounds over the 256 compute units (`share` workgroups of that tile fit one unit and
// share its matrix cores), and a partly filled last round costs a whole one. `penalty` is what a
// tile shape loses against the largest, in percent, from reading its operands more often.
long rounds_cost(long tiles, int tile_elements, int share, int penalty) {
    const long rounds = (tiles + (long)XRT_COMPUTE_UNITS * share - 1) / ((long)XRT_COMPUTE_UNITS * share);
    return rounds * share * tile_elements * (100 + penalty) / 100;
}

template <int MODE, typename TO>
int launch_mode(const bf16* a, const bf16* w, TO* out, int M, int N, int K, const Packing& packing, int activation, hipStream_t s) {
    // output columns per tile are half the tile's w rows in the gated mode
    constexpr int DIV = MODE == MODE_GATED ? 2 : 1;
    auto tiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn / DIV - 1) / (bn / DIV)); };
    const bool whole_k = K % 64 == 0;
    // Up to 128 rows of a, gated: one round of tiles of 128 x 128 (or nearly), bound by reading w: three stages keep more of
    // it on its way than the two that the tiles below have (gate/up of 14336 pairs and 128 rows: 76 us split in three
    // with a second kernel, 49 us so).
    if constexpr (MODE == MODE_GATED)
        if (whole_k && M <= 128) return launch_kernel<128, 128, 2, 2, MODE, 64, 3, TO>(a, w, out, M, N, K, 0, N, packing, s, 1, 0, RowScale{nullptr, 0, 0, 0.f, activation});
    const long large = rounds_cost(tiles(256, 256), 256 * 256, 1, 0);
    const long medium = whole_k && MODE != MODE_GATED ? rounds_cost(tiles(256, 192), 256 * 192, 1, 5) : LONG_MAX;
    const long small = rounds_cost(tiles(128, 128), 128 * 128, 2, 18);
    // Large tiles for as many columns as make whole rounds, and tiles of half the height for the
    // rest, if those then fit one round: the last round is full of half-sized work instead of
    // half empty.
    const int tiles_m = (M + 255) / 256, tiles_n = (N + 256 / DIV - 1) / (256 / DIV);
    const int whole_columns = (int)((long)tiles_m * tiles_n / XRT_COMPUTE_UNITS * XRT_COMPUTE_UNITS / tiles_m);     // n-tiles that run in full rounds
    const long rest_tiles = (long)((M + 127) / 128) * (tiles_n - whole_columns);
    long mixed = LONG_MAX;
    if (whole_k && whole_columns > 0 && whole_columns < tiles_n && rest_tiles <= XRT_COMPUTE_UNITS)
        mixed = rounds_cost((long)tiles_m * whole_columns, 256 * 256, 1, 0) + rounds_cost(rest_tiles, 128 * 256, 1, 8);
    if (mixed < large && mixed <= medium && mixed <= small) {
        const int split = whole_columns * (256 / DIV);
        const int small_tiles_m = (M + 127) / 128, small_tiles_n = tiles_n - whole_columns;
        const int large_blocks = (tiles_m * whole_columns + 7) / 8 * 8;      // whole rounds over the XCDs
        const int small_blocks = (small_tiles_m * small_tiles_n + 7) / 8 * 8;
        constexpr size_t lds = (size_t)2 * (256 + 256) * 64 * sizeof(bf16);
        auto kernel = gemm_mfma_mixed_kernel<MODE, TO>;
        static bool configured = false;      // per instantiation
        if (!configured) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            XRT_REQUIRE(e == hipSuccess, "linear (mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
            configured = true;
        }
        kernel<<<large_blocks + small_blocks, 8 * XRT_WAVE, lds, s>>>(a, w, out, M, N, K, large_blocks, tiles_m, whole_columns,
                                                                      split, small_tiles_m, small_tiles_n, packing, RowScale{nullptr, 0, 0, 0.f, activation});
        XRT_LAUNCH_CHECK("linear (mfma, two tile shapes)");
        return 0;
    }
    if (large <= medium && large <= small) return launch<256, 256, 2, 4, MODE, TO>(a, w, out, M, N, K, 0, N, packing, activation, s);
    if constexpr (MODE != MODE_GATED)
        if (medium <= small) return launch<256, 192, 4, 2, MODE, TO>(a, w, out, M, N, K, 0, N, packing, activation, s);
    return launch<128, 128, 2, 2, MODE, TO>(a, w, out, M, N, K, 0, N, packing, activation, s);
}

template <typename TO>
int launch_shape(const bf16* a, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const Packing& packing, hipStream_t s) {
    if (mode == MODE_STORE) return launch_mode<MODE_STORE, TO>(a, w, out, M, N, K, packing, activation, s);
    if (mode == MODE_ACCUMULATE) return launch_mode<MODE_ACCUMULATE, TO>(a, w, out, M, N, K, packing, activation, s);
    return launch_mode<MODE_GATED, TO>(a, w, out, M, N, K, packing, activation, s);
}

// ---- 17 to 64 rows of x: too many for the kernel that streams w through registers (it would read
// x from L2 up to four times as often as w from HBM), too few for the tiles above to fill the chip.
// Tiles of 64 x 128 take their x through LDS; k is split among workgroups as far as every compute
// unit still gets at most one of them (one long stream per unit pulls w faster than several short
// ones, measured); each writes float32 sums of its part of k to a workspace, and a second kernel
// adds the parts in order and applies the epilogue. Where w has tiles enough without a split, the
// tiles apply the epilogue themselves and there is no second kernel.
// With more rows of x (up to a few hundred) the tiles of 128 x 128 do the same when they are too
// few to fill the chip: such products are still bound by reading w.
constexpr int SPLIT_BM = 64, SPLIT_BN = 128;

struct SplitPlan { int splits, k_per_split; long rows_w; int tile, columns; };      // tile: rows of x per tile (64, 128 or 256), columns: rows of w

// whole_norm: an RMSNorm follows that the second kernel can do outright, which is worth a split in two where the product alone
// would do as well without (k from 4096 on instead of from 8192 on).
SplitPlan split_plan(int M, int N, int K, int mode, bool whole_norm = false) {
    const long rows_w = mode == MODE_GATED ? 2L * N : N;
    const long tiles_n = (rows_w + SPLIT_BN - 1) / SPLIT_BN;
    const int units = K / 64;                                  // k is dealt out in pieces of 64
    int splits, least, tile = SPLIT_BM, columns = SPLIT_BN;    // least: pieces of k that a part should have
    const long large_tiles = (long)((M + 255) / 256) * ((rows_w + 255) / 256);
    if (M <= SPLIT_BM) {
        splits = (int)(XRT_COMPUTE_UNITS / tiles_n);                         // one workgroup per compute unit, or fewer
        least = 1;
    } else if (large_tiles <= 128 && M >= 512 && mode != MODE_GATED && units >= (whole_norm ? 64 : 128)) {
        // Many rows and a very long k, but so few columns that the largest tiles would leave half of the compute
        // units idle (the projection back from the feed-forward's width): the large tiles split k between them.
        // The tiles of 128 x 128, which fill the chip without a second kernel, read their operands from LDS
        // more often for the same products and take longer here.
        splits = (int)(XRT_COMPUTE_UNITS / large_tiles);
        splits = splits > 8 ? 8 : splits;
        least = 24;
        tile = columns = 256;
    } else {
        // Some hundred rows of x: still bound by reading w, and too few tiles to fill the chip without a split.
        // Every part of k writes its sums and the second kernel reads them again (16 parts of a square w and 128 rows
        // of x: as many bytes as w has), so the parts are few and long (1024 of k at least), and where tiles of 128 x 128
        // are fewer than the compute units and k is short, tiles of 128 x 64 make up the number instead of further parts.
        // With a long k the partial sums are small against w and the wider tile, which reads x half as often, is kept
        // (at the sizes of the 8B models, 128 rows: q/k/v 31 -> 25 us, o 24 -> 18, down 40 -> 37).
        // Beyond 256 rows the matrix cores begin to count: tiles of 128 x 128, two to a compute unit, in as many parts as
        // fill those places.
        long tiles = (long)((M + 127) / 128) * tiles_n;
        tile = columns = 128;
        if (M <= 256) {
            if (tiles < XRT_COMPUTE_UNITS && mode != MODE_GATED && K < 8192) {
                columns = 64;
                tiles = (long)((M + 127) / 128) * ((rows_w + 63) / 64);
            }
            // a gated product with a round of tiles or nearly so does without a split: its tiles apply the epilogue themselves
            const int target = M <= 128 && columns == 64 ? 2 * XRT_COMPUTE_UNITS : XRT_COMPUTE_UNITS;
            splits = tiles >= 384 || (mode == MODE_GATED && tiles >= 200) ? 1 : (int)((target + tiles - 1) / tiles);
            least = columns == 64 ? 16 : 8;
        } else {
            // The workgroups run two to a compute unit: as many parts as still fit those 512 places at once, and none where
            // that is one. A few workgroups over (96 tiles in 6 parts) run a second round for a few; so do parts enough for
            // two rounds of shorter workgroups, which an estimate by rounds prefers and the clock does not. (The four products
            // of a layer at 384 rows 295 -> 251 us; q/k/v at 512 rows 54 -> 45 us, at 768 rows 77 -> 65; o at 768 rows 55 -> 47.)
            splits = (int)(2 * XRT_COMPUTE_UNITS / tiles);
            least = 4;
        }
    }
    splits = splits < 1 ? 1 : (splits > 16 ? 16 : splits);
    splits = splits > units / least ? (units / least < 1 ? 1 : units / least) : splits;
    const int per = (units + splits - 1) / splits;
    splits = (units + per - 1) / per;                          // no empty part
    return SplitPlan{splits, per * 64, rows_w, tile, columns};
}

// NORM 1: the rows of a came without their RMSNorm's division (norm.squares_in): the sums are multiplied by
// 1 / rms of their row first. NORM 2 (accumulating): bfloat16(out * gain) and the sums of squares of out per
// tile of 16 columns are written as well (N a multiple of 16: the 16 lanes of a tile then share a row).
template <int MODE, typename TO, int NORM = 0>
__global__ void __launch_bounds__(256) split_reduce_kernel(const float* __restrict__ parts, int splits, int M, int N,
                                                            TO* __restrict__ out, const xrt_linear_norm norm, int activation) {
    __shared__ float wave_sums[256 / XRT_WAVE];
    const long rows_w = MODE == MODE_GATED ? 2L * N : N;
    const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool inside = index < (long)M * N;
    const long m = inside ? index / N : M - 1, n = inside ? index % N : 0;
    // the row's sums of squares are asked for before the partial sums and used after them. A block lies
    // within one row if N is a multiple of 256: then its threads share the work; else every thread adds
    // up its row's sums itself, in the order of the tiles.
    float mine = 0.f;
    if constexpr (NORM == 1) {
        if (N % 256 == 0)
            for (int t = threadIdx.x; t < norm.tiles_in; t += 256) mine += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + m];
        else
            for (int t = 0; t < norm.tiles_in; ++t) mine += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + m];
    }
    float sum = 0.f, up = 0.f;
    if (inside) {
        for (int p = 0; p < splits; ++p) {
            const float* part = parts + ((long)p * M + m) * rows_w;
            sum += part[n];
            if constexpr (MODE == MODE_GATED) up += part[N + n];
        }
    }
    float by = 1.0f;
    if constexpr (NORM == 1) {
        float total = mine;
        if (N % 256 == 0) {
            mine = wave_sum(mine);
            if (threadIdx.x % XRT_WAVE == 0) wave_sums[threadIdx.x / XRT_WAVE] = mine;
            __syncthreads();
            total = 0.f;
            for (int w = 0; w < 256 / XRT_WAVE; ++w) total += wave_sums[w];
        }
        by = 1.0f / sqrtf(total / (float)norm.width_in + norm.eps);
    }
    sum *= by;
    up *= by;
    float fresh = 0.f;
    if (inside) {
        if constexpr (MODE == MODE_STORE) out[index] = from_float<TO>(sum);
        else if constexpr (MODE == MODE_ACCUMULATE) { fresh = to_float(out[index]) + sum; out[index] = from_float<TO>(fresh); }
        else out[index] = from_float<TO>(gate_activation<sizeof(TO) == 2>(sum, activation) * up);
    }
    if constexpr (NORM == 2) {
        float squares = fresh * fresh;
        squares += __shfl_xor(squares, 1, XRT_WAVE);
        squares += __shfl_xor(squares, 2, XRT_WAVE);
        squares += __shfl_xor(squares, 4, XRT_WAVE);
        squares += __shfl_xor(squares, 8, XRT_WAVE);
        if (inside) {
            if (n % 16 == 0) norm.squares_out[(n / 16) * XRT_SQUARES_STRIDE + m] = squares;
            const float gain = norm.gain_dtype == XRT_F32 ? ((const float*)norm.gain)[n] : to_float(((const bf16*)norm.gain)[n]);
            ((bf16*)norm.scaled_out)[index] = from_float<bf16>(fresh * gain);
        }
    }
}

// The same for store and accumulate without a norm, four neighbouring columns a thread (N a multiple of 4):
// what products of many rows use, whose partial sums are tens of megabytes.
template <int MODE, typename TO>
__global__ void __launch_bounds__(256) split_reduce_wide_kernel(const float* __restrict__ parts, int splits, long count, TO* __restrict__ out) {
    const long index = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (index >= count) return;
    float4 sum = *reinterpret_cast<const float4*>(parts + index);
    for (int p = 1; p < splits; ++p) {
        const float4 part = *reinterpret_cast<const float4*>(parts + p * count + index);
        sum.x += part.x; sum.y += part.y; sum.z += part.z; sum.w += part.w;
    }
    if constexpr (MODE == MODE_ACCUMULATE) {
        static_assert(sizeof(TO) == 4, "accumulation needs a float32 output");
        const float4 before = *reinterpret_cast<const float4*>(out + index);
        // the order of the one-column kernel: the parts first, in order, then onto what was there
        sum.x = before.x + sum.x; sum.y = before.y + sum.y; sum.z = before.z + sum.z; sum.w = before.w + sum.w;
    }
    if constexpr (sizeof(TO) == 4) {
        *reinterpret_cast<float4*>(out + index) = sum;
    } else {
        struct alignas(8) Four { TO e[4]; } four;
        four.e[0] = from_float<TO>(sum.x); four.e[1] = from_float<TO>(sum.y); four.e[2] = from_float<TO>(sum.z); four.e[3] = from_float<TO>(sum.w);
        *reinterpret_cast<Four*>(out + index) = four;
    }
}

// The second kernel of an accumulating product of many rows that an RMSNorm follows: a workgroup takes a whole row, adds the
// parts onto the residual and writes the row's norm as well. The norm is the norm kernel's (elementwise.hip) to the bit: the same
// four columns a thread, the same order of the sum of squares, (x * 1/rms) * gain.
constexpr int NORM_QUADS = 8;                      // four-column pieces a thread holds: rows of up to 8 * 256 * 4 columns
template <typename T> struct alignas(sizeof(T) * 4) Four { T e[4]; };
template <typename TW>
__global__ void __launch_bounds__(256) split_reduce_rmsnorm_kernel(const float* __restrict__ parts, int splits, long count, int N,
                                                                    float* __restrict__ out, const TW* __restrict__ gain, float eps,
                                                                    bf16* __restrict__ normed) {
    __shared__ float scratch[32];
    const long row = (long)blockIdx.x * N;
    const int quads = N / 4;
    float4 kept[NORM_QUADS];
    Four<TW> weight[NORM_QUADS];
#pragma unroll
    for (int i = 0; i < NORM_QUADS; ++i) {
        const int q = threadIdx.x + i * 256;
        kept[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        weight[i] = Four<TW>{};
        if (q < quads) {
            const long index = row + 4L * q;
            typedef float floatx4 __attribute__((ext_vector_type(4)));
            const floatx4 first = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(parts + index));     // read once, by nobody else
            float4 sum = make_float4(first[0], first[1], first[2], first[3]);
            for (int p = 1; p < splits; ++p) {
                const floatx4 part = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(parts + p * count + index));
                sum.x += part[0]; sum.y += part[1]; sum.z += part[2]; sum.w += part[3];
            }
            const float4 before = *reinterpret_cast<const float4*>(out + index);
            kept[i] = make_float4(before.x + sum.x, before.y + sum.y, before.z + sum.z, before.w + sum.w);
            *reinterpret_cast<float4*>(out + index) = kept[i];
            weight[i] = *reinterpret_cast<const Four<TW>*>(gain + 4 * q);
        }
    }
    float squares = 0.f;
#pragma unroll
    for (int i = 0; i < NORM_QUADS; ++i)
        squares = fmaf(kept[i].x, kept[i].x, fmaf(kept[i].y, kept[i].y, fmaf(kept[i].z, kept[i].z, fmaf(kept[i].w, kept[i].w, squares))));
    squares = block_sum(squares, scratch);
    const float inv_rms = 1.0f / sqrtf(squares / (float)N + eps);
#pragma unroll
    for (int i = 0; i < NORM_QUADS; ++i) {
        const int q = threadIdx.x + i * 256;
        if (q < quads) {
            Four<bf16> r;
            r.e[0] = from_float<bf16>((kept[i].x * inv_rms) * to_float(weight[i].e[0]));
            r.e[1] = from_float<bf16>((kept[i].y * inv_rms) * to_float(weight[i].e[1]));
            r.e[2] = from_float<bf16>((kept[i].z * inv_rms) * to_float(weight[i].e[2]));
            r.e[3] = from_float<bf16>((kept[i].w * inv_rms) * to_float(weight[i].e[3]));
            *reinterpret_cast<Four<bf16>*>(normed + row + 4L * q) = r;
        }
    }
}

// The second kernel of a q/k/v projection split along k (no head norms, the rotation over the whole head):
// a thread adds up the two outputs that the rotation pairs (dims d and d + head_dim / 2 of one head), for
// NORM 1 scales them by the row's 1 / rms, rotates q and k by the token's position, writes bfloat16 q/k/v and
// puts k and v into the cache. One thread per (token, head, d).
template <int NORM>
__global__ void __launch_bounds__(256) split_reduce_qkv_kernel(const float* __restrict__ parts, int splits, int M, int N,
                                                                bf16* __restrict__ qkv, const xrt_linear_norm norm,
                                                                const QkvAfter after) {
    __shared__ float wave_sums[256 / XRT_WAVE];
    const int half = after.head_dim / 2;
    const long per_token = (long)(N / 2);
    const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool inside = index < (long)M * per_token;
    const long m = inside ? index / per_token : M - 1;
    const int pair = inside ? (int)(index % per_token) : 0;
    const int head = pair / half, d = pair % half;
    const long n = (long)head * after.head_dim + d;
    float mine = 0.f;
    if constexpr (NORM == 1) {
        // a block lies within one token if a token's pairs are a multiple of 256: then its threads share the work
        if (per_token % 256 == 0)
            for (int t = threadIdx.x; t < norm.tiles_in; t += 256) mine += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + m];
        else
            for (int t = 0; t < norm.tiles_in; ++t) mine += norm.squares_in[(long)t * XRT_SQUARES_STRIDE + m];
    }
    float lower = 0.f, upper = 0.f;
    for (int p = 0; p < splits; ++p) {
        const float* part = parts + ((long)p * M + m) * N;
        lower += part[n];
        upper += part[n + half];
    }
    const int pos = after.positions[m];
    const bool is_q = head < after.n_heads, is_v = head >= after.n_heads + after.n_kv_heads;
    float sine = 0.f, cosine = 1.f;
    if (after.rope_theta != nullptr && !is_v) sincosf((float)pos * after.rope_scale / after.rope_theta[d], &sine, &cosine);
    if constexpr (NORM == 1) {
        float total = mine;
        if (per_token % 256 == 0) {
            mine = wave_sum(mine);
            if (threadIdx.x % XRT_WAVE == 0) wave_sums[threadIdx.x / XRT_WAVE] = mine;
            __syncthreads();
            total = 0.f;
            for (int w = 0; w < 256 / XRT_WAVE; ++w) total += wave_sums[w];
        }
        const float by = 1.0f / sqrtf(total / (float)norm.width_in + norm.eps);
        lower *= by;
        upper *= by;
    }
    if (!inside) return;
    // rounded as the product alone would have stored them, then rotated: the same values as from two kernels
    lower = to_float(from_float<bf16>(lower));
    upper = to_float(from_float<bf16>(upper));
    const bf16 out_lower = from_float<bf16>(lower * cosine - upper * sine);
    const bf16 out_upper = from_float<bf16>(lower * sine + upper * cosine);
    qkv[m * N + n] = out_lower;
    qkv[m * N + n + half] = out_upper;
    if (is_q || after.k_cache == nullptr) return;
    const int kv_head = head - after.n_heads - (is_v ? after.n_kv_heads : 0);
    const long base = cache_block_base(after.block_table, after.table_stride, after.n_blocks, after.slots[m], pos,
                                       after.n_kv_heads, kv_head, after.head_dim);
    if (base < 0) return;
    const int within = pos % XRT_BLOCK_TOKENS;
    if (is_v) {
        after.v_cache[base + cache_value_offset(d, within, after.head_dim)] = out_lower;
        after.v_cache[base + cache_value_offset(d + half, within, after.head_dim)] = out_upper;
    } else {
        after.k_cache[base + cache_key_offset(within, d, after.head_dim)] = out_lower;
        after.k_cache[base + cache_key_offset(within, d + half, after.head_dim)] = out_upper;
    }
}

template <typename TO>
int launch_split(const bf16* a, const bf16* w, TO* out, int M, int N, int K, int mode, int activation, const Packing& packing,
                 float* workspace, const xrt_linear_norm* norm, const QkvAfter* after, hipStream_t s) {
    // the whole norm after an accumulating product of many rows: normed rows asked for, and no sums of squares
    const bool whole_norm = norm && norm->scaled_out && !norm->squares_out && !norm->squares_in;
    const SplitPlan plan = split_plan(M, N, K, mode, whole_norm);
    const bool scaled = norm && norm->squares_in, emits = norm && norm->squares_out;
    XRT_REQUIRE(!norm || M <= SPLIT_BM || whole_norm, "linear (mfma): the halves of a norm around a product take at most %d rows here", SPLIT_BM);
    if (whole_norm)
        XRT_REQUIRE(M > SPLIT_BM && mode == MODE_ACCUMULATE && sizeof(TO) == 4 && plan.tile == 256 && plan.splits > 1 && N % 4 == 0 &&
                    N <= NORM_QUADS * 256 * 4 && norm->gain && (uintptr_t)out % 16 == 0 && (uintptr_t)norm->scaled_out % 8 == 0,
                    "linear (mfma): M=%d N=%d K=%d is not a product whose second kernel does the norm after it", M, N, K);
    const RowScale scale = scaled ? RowScale{norm->squares_in, norm->tiles_in, norm->width_in, norm->eps, activation}
                                  : RowScale{nullptr, 0, 0, 0.f, activation};
    XRT_REQUIRE(!after || (plan.splits > 1 && mode == MODE_STORE && sizeof(TO) == 2),
                "linear (mfma): only a bfloat16 product split along k does what follows a q/k/v projection");
    if (M <= SPLIT_BM && plan.splits == 1) {                   // tiles enough: each applies the epilogue itself
        XRT_REQUIRE(!emits, "linear (mfma): only a product split along k writes what the norm after it needs");
        if (mode == MODE_STORE) return launch_kernel<SPLIT_BM, SPLIT_BN, 1, 4, MODE_STORE, 64, 3, TO>(a, w, out, M, N, K, 0, N, packing, s, 1, 0, scale);
        if (mode == MODE_GATED) return launch_kernel<SPLIT_BM, SPLIT_BN, 2, 2, MODE_GATED, 64, 3, TO>(a, w, out, M, N, K, 0, N, packing, s, 1, 0, scale);
        if constexpr (sizeof(TO) == 4)
            return launch_kernel<SPLIT_BM, SPLIT_BN, 1, 4, MODE_ACCUMULATE, 64, 3, TO>(a, w, out, M, N, K, 0, N, packing, s, 1, 0, scale);
        XRT_REQUIRE(false, "linear (mfma): accumulation needs a float32 output");
    }
    XRT_REQUIRE(workspace != nullptr, "linear (mfma): a product split along k needs its workspace");
    // the product of all rows of w, ungated, into the workspace: [splits][M][rows_w]
    const int status = M <= SPLIT_BM
        ? launch_kernel<SPLIT_BM, SPLIT_BN, 1, 4, MODE_STORE, 64, 3, float>(
              a, w, workspace, M, (int)plan.rows_w, K, 0, (int)plan.rows_w, packing, s, plan.splits, plan.k_per_split)
        : plan.tile == 256
        ? launch_kernel<256, 256, 2, 4, MODE_STORE, 64, 2, float>(
              a, w, workspace, M, (int)plan.rows_w, K, 0, (int)plan.rows_w, packing, s, plan.splits, plan.k_per_split)
        : plan.columns == 64
        ? launch_kernel<128, 64, 2, 2, MODE_STORE, 64, 3, float>(
              a, w, workspace, M, (int)plan.rows_w, K, 0, (int)plan.rows_w, packing, s, plan.splits, plan.k_per_split)
        : M <= 256          // (one workgroup to a compute unit anyway: a third stage keeps more of w on its way; with more, two share a unit)
        ? launch_kernel<128, 128, 2, 2, MODE_STORE, 64, 3, float>(
              a, w, workspace, M, (int)plan.rows_w, K, 0, (int)plan.rows_w, packing, s, plan.splits, plan.k_per_split)
        : launch_kernel<128, 128, 2, 2, MODE_STORE, 64, 2, float>(
              a, w, workspace, M, (int)plan.rows_w, K, 0, (int)plan.rows_w, packing, s, plan.splits, plan.k_per_split);
    if (status != 0) return status;
    const unsigned blocks = (unsigned)(((long)M * N + 255) / 256);
    const xrt_linear_norm none = {};
    const xrt_linear_norm& around = norm ? *norm : none;
    XRT_REQUIRE(!(scaled && emits), "linear (mfma): one product does one half of a norm");
    if (after != nullptr) {
        if constexpr (sizeof(TO) == 2) {
            const unsigned pair_blocks = (unsigned)(((long)M * (N / 2) + 255) / 256);
            if (scaled) split_reduce_qkv_kernel<1><<<pair_blocks, 256, 0, s>>>(workspace, plan.splits, M, N, out, around, *after);
            else split_reduce_qkv_kernel<0><<<pair_blocks, 256, 0, s>>>(workspace, plan.splits, M, N, out, around, *after);
            XRT_LAUNCH_CHECK("linear (split reduce, q/k/v)");
        }
        return 0;
    }
    if (whole_norm) {
        if constexpr (sizeof(TO) == 4) {
            const long count = (long)M * N;
            if (norm->gain_dtype == XRT_F32)
                split_reduce_rmsnorm_kernel<float><<<M, 256, 0, s>>>(workspace, plan.splits, count, N, out, (const float*)norm->gain, norm->eps, (bf16*)norm->scaled_out);
            else
                split_reduce_rmsnorm_kernel<bf16><<<M, 256, 0, s>>>(workspace, plan.splits, count, N, out, (const bf16*)norm->gain, norm->eps, (bf16*)norm->scaled_out);
            XRT_LAUNCH_CHECK("linear (split reduce with the norm after it)");
        }
        return 0;
    }
    if (!scaled && !emits && mode != MODE_GATED && N % 4 == 0 && M > SPLIT_BM && (uintptr_t)out % 16 == 0) {
        const long count = (long)M * N;
        const unsigned wide_blocks = (unsigned)((count / 4 + 255) / 256);
        if (mode == MODE_STORE) split_reduce_wide_kernel<MODE_STORE, TO><<<wide_blocks, 256, 0, s>>>(workspace, plan.splits, count, out);
        else if constexpr (sizeof(TO) == 4) split_reduce_wide_kernel<MODE_ACCUMULATE, TO><<<wide_blocks, 256, 0, s>>>(workspace, plan.splits, count, out);
        else XRT_REQUIRE(false, "linear (mfma): accumulation needs a float32 output");
        XRT_LAUNCH_CHECK("linear (split reduce, four columns a thread)");
        return 0;
    }
#define XRT_REDUCE(MODE_, NORM_) split_reduce_kernel<MODE_, TO, NORM_><<<blocks, 256, 0, s>>>(workspace, plan.splits, M, N, out, around, activation)
    if (mode == MODE_STORE) { if (scaled) XRT_REDUCE(MODE_STORE, 1); else XRT_REDUCE(MODE_STORE, 0); }
    else if (mode == MODE_GATED) { if (scaled) XRT_REDUCE(MODE_GATED, 1); else XRT_REDUCE(MODE_GATED, 0); }
    else if (scaled) XRT_REDUCE(MODE_ACCUMULATE, 1);
    else if (emits) {
        XRT_REQUIRE(N % 16 == 0, "linear (mfma): sums of squares per 16 columns need N = %d to be a multiple of 16", N);
        XRT_REDUCE(MODE_ACCUMULATE, 2);
    } else XRT_REDUCE(MODE_ACCUMULATE, 0);
#undef XRT_REDUCE
    XRT_LAUNCH_CHECK("linear (split reduce)");
    return 0;
}

}  // namespace

bool xrt_linear_mfma_accepts(const void* a, const void* w, int M, int N, int K, int mode) {
    const long rows_w = mode == MODE_GATED ? 2L * N : N;     // operands are addressed with 32-bit element offsets
    return K % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 && (long)M * K < (1L << 31) && (rows_w + 15) * K < (1L << 31);
}

int xrt_linear_mfma(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                    const Packing& packing, hipStream_t s) {
    if (out_dtype == XRT_F32) return launch_shape<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, activation, packing, s);
    return launch_shape<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, activation, packing, s);
}

// Whether a product runs through the tiles of this section (17 to 64 rows of x, or more rows and few
// tiles), and the floats of workspace it then needs (0 where k is not split).
bool xrt_linear_split_takes(const void* a, const void* w, int M, int N, int K, int mode, long* workspace_floats) {
    *workspace_floats = 0;
    if (M <= 16 || K % 64 != 0 || K < 128 || !xrt_linear_mfma_accepts(a, w, M, N, K, mode)) return false;
    const SplitPlan plan = split_plan(M, N, K, mode);
    if (plan.splits == 1) return M <= SPLIT_BM;               // more rows and enough tiles without a split: the kernels above
    if (plan.rows_w * (long)M >= (1L << 31)) return false;
    *workspace_floats = (long)plan.splits * M * plan.rows_w;
    return true;
}

// Whether an accumulating product of many rows runs as large tiles that split k, so that its second kernel can do the
// RMSNorm that follows it outright; and the floats of workspace it then needs. (With the smaller tiles' few rows the
// kernel that takes a row per workgroup has too few workgroups: 5.75 against 5.65 ms a prompt of 128 tokens.)
bool xrt_linear_split_takes_whole_norm(const void* a, const void* w, int M, int N, int K, int mode, long* workspace_floats) {
    *workspace_floats = 0;
    if (mode != MODE_ACCUMULATE || M <= SPLIT_BM || K % 64 != 0 || N % 4 != 0 || N > NORM_QUADS * 256 * 4 ||
        !xrt_linear_mfma_accepts(a, w, M, N, K, mode))
        return false;
    const SplitPlan plan = split_plan(M, N, K, mode, true);
    if (plan.tile != 256 || plan.splits < 2 || (long)M * N >= (1L << 31)) return false;
    *workspace_floats = (long)plan.splits * M * N;
    return true;
}

// Whether a product of 17 to 64 rows can do its half of an RMSNorm: take rows that come without the
// division (any mode), or, accumulating and split along k, write what the norm after it needs, provided
// the product after the norm (same rows, N columns of a) will run through these tiles too.
bool xrt_linear_split_takes_norm(const void* a, const void* w, int M, int N, int K, int mode) {
    long unused = 0;
    if (M <= 16 || M > SPLIT_BM || !xrt_linear_split_takes(a, w, M, N, K, mode, &unused)) return false;
    if (mode != MODE_ACCUMULATE) return true;
    return split_plan(M, N, K, mode).splits > 1 && N % 64 == 0 && N >= 128;
}

int xrt_linear_split(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode, int activation,
                     const Packing& packing, float* workspace, const xrt_linear_norm* norm, hipStream_t s) {
    if (out_dtype == XRT_F32) return launch_split<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, activation, packing, workspace, norm, nullptr, s);
    return launch_split<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, activation, packing, workspace, norm, nullptr, s);
}

// Whether the q/k/v projection of a step of 17 to 64 tokens can also do what follows it (rotation over the
// whole head or none, no head norms, cache write) in the kernel that adds up its partial sums.
bool xrt_linear_split_takes_qkv(const void* a, const void* w, int M, int N, int K, const QkvAfter& after, long* workspace_floats) {
    *workspace_floats = 0;
    if (M > SPLIT_BM || after.head_dim % 2 != 0 || N != (after.n_heads + 2 * after.n_kv_heads) * after.head_dim) return false;
    if (after.rope_theta != nullptr && after.rope_dim != after.head_dim) return false;
    return xrt_linear_split_takes(a, w, M, N, K, MODE_STORE, workspace_floats) && *workspace_floats > 0;
}

int xrt_linear_split_qkv(const void* a, const void* w, void* qkv, int M, int N, int K, const Packing& packing, float* workspace,
                         const xrt_linear_norm* norm, const QkvAfter& after, hipStream_t s) {
    return launch_split<bf16>((const bf16*)a, (const bf16*)w, (bf16*)qkv, M, N, K, MODE_STORE, XRT_ACT_SILU, packing, workspace, norm, &after, s);
}
