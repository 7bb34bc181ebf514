// Matrix product for many rows (prefill), bfloat16 operands, float32 accumulation on the
// matrix cores: out[m, n] = sum_k a[m, k] * w[n, k]; both operands are contiguous along k.
//
// A workgroup computes a BM x BN tile of the output with v_mfma_f32_32x32x16_bf16. Tiles of
// a and w, 64 wide in k, are staged through LDS: while the matrix cores work on one buffer,
// the next tile is written into the other and the one after that is on its way from global
// memory into registers (one barrier per step). LDS
// rows are padded by 16 bytes so that the 16-byte operand reads of 16 consecutive rows fall
// into different banks. Each wavefront owns a (BM/WM) x (BN/WN) part of the tile and keeps
// its accumulators in registers for the whole K loop.
//
// Workgroup ids are remapped so that the workgroups that run on one XCD (ids are dealt
// round-robin to the 8 XCDs) work on neighbouring tiles and share their operands in that
// XCD's L2.
//
// Epilogues: store (bfloat16 or float32), accumulate into float32, or the gated pair
// silu(gate) * up: then the w tile holds BN/2 gate rows and the BN/2 up rows that belong to
// them (rows n and n + N of w), and the two halves meet through LDS after the K loop.
#include "common.h"
#include "xrt_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 64;
constexpr int PITCH = BK + 8;          // bf16 elements per LDS row
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };

__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

template <int BM, int BN, int WM, int WN, int MODE, typename TO>
__global__ void __launch_bounds__(WM * WN * XRT_WAVE) gemm_mfma_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    int tiles_m, int tiles_n) {
    constexpr int THREADS = WM * WN * XRT_WAVE;
    constexpr int WAVE_M = BM / WM, WAVE_N = BN / WN;        // part of the tile owned by one wavefront
    constexpr int TM = WAVE_M / 32, TN = WAVE_N / 32;        // 32x32 accumulator tiles of a wavefront
    constexpr int CHUNKS_A = BM * BK / 8 / THREADS;          // 16-byte chunks each thread moves per step
    constexpr int CHUNKS_B = BN * BK / 8 / THREADS;
    static_assert(BM * BK / 8 % THREADS == 0 && BN * BK / 8 % THREADS == 0, "tile does not divide among the threads");

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    bf16* lds_a = reinterpret_cast<bf16*>(lds_raw);                    // [2][BM][PITCH]
    bf16* lds_b = lds_a + 2 * BM * PITCH;                              // [2][BN][PITCH]

    // ---- which tile: ids are dealt to XCDs round-robin; give each XCD a contiguous run of tiles,
    // and walk a run m-fastest inside panels of 8 n-tiles so that concurrent tiles share w
    const int total = tiles_m * tiles_n;
    int id = blockIdx.x;
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
    const long n0 = (long)tile_n * BN_OUT;

    const int tid = threadIdx.x, lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    const int wave_m = wave / WN, wave_n = wave % WN;

    // Row of w behind row r of the tile. Rows beyond the operands are clamped to the last row:
    // loads then need no guard, and what such a row contributes lands in outputs that are not written.
    auto w_row = [&](int r) -> long {
        if constexpr (MODE == MODE_GATED) {
            return min(n0 + (r % BN_OUT), (long)N - 1) + (long)(r / BN_OUT) * N;
        } else {
            return min(n0 + r, (long)N - 1);
        }
    };
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
        off_b[i] = (unsigned)(w_row(chunk / 8) * K + (chunk % 8) * 8);
    }

    struct Stage { bf16x8 a[CHUNKS_A], b[CHUNKS_B]; };
    auto fetch = [&](Stage& stage, int k0) {                  // a whole tile of 64 along k, no guards
#pragma unroll
        for (int i = 0; i < CHUNKS_A; ++i) stage.a[i] = *reinterpret_cast<const bf16x8*>(a + (off_a[i] + (unsigned)k0));
#pragma unroll
        for (int i = 0; i < CHUNKS_B; ++i) stage.b[i] = *reinterpret_cast<const bf16x8*>(w + (off_b[i] + (unsigned)k0));
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
            stage.b[i] = k + 8 <= K ? *reinterpret_cast<const bf16x8*>(w + (off_b[i] + (unsigned)k0)) : bf16x8{};
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

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

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
    __syncthreads();                                          // the epilogue may reuse the LDS

    // ---- epilogue: accumulator element e of tile (i, j) is row (e/4)*8 + (lane/32)*4 + e%4, column lane%32
    if constexpr (MODE == MODE_GATED) {
        // wavefronts of the right half (up) hand their accumulators to the wavefront that holds
        // the gate values of the same rows and columns: wave_n and wave_n + WN/2
        static_assert(WN % 2 == 0, "a gated tile needs an even number of wavefront columns");
        float* exchange = reinterpret_cast<float*>(lds_raw);           // [pairs][TM*TN*16][64]
        const int pair = wave_m * (WN / 2) + wave_n % (WN / 2);
        float* mine = exchange + (long)pair * (TM * TN * 16) * XRT_WAVE;
        if (wave_n >= WN / 2) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) mine[((i * TN + j) * 16 + e) * XRT_WAVE + lane] = acc[i][j][e];
        }
        __syncthreads();
        if (wave_n < WN / 2) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const long m = m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4;
                        const long n = n0 + wave_n * WAVE_N + j * 32 + lane % 32;
                        const float up = mine[((i * TN + j) * 16 + e) * XRT_WAVE + lane];
                        if (m < M && n < N) out[m * (long)N + n] = from_float<TO>(silu(acc[i][j][e]) * up);
                    }
        }
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const long m = m0 + wave_m * WAVE_M + i * 32 + (e / 4) * 8 + (lane / 32) * 4 + e % 4;
                    const long n = n0 + wave_n * WAVE_N + j * 32 + lane % 32;
                    if (m < M && n < N) {
                        TO* dst = out + m * (long)N + n;
                        if constexpr (MODE == MODE_STORE) *dst = from_float<TO>(acc[i][j][e]);
                        else *dst = from_float<TO>(to_float(*dst) + acc[i][j][e]);
                    }
                }
    }
}

template <int BM, int BN, int WM, int WN, int MODE, typename TO>
int launch(const bf16* a, const bf16* w, TO* out, int M, int N, int K, hipStream_t s) {
    constexpr int BN_OUT = MODE == MODE_GATED ? BN / 2 : BN;
    constexpr int THREADS = WM * WN * XRT_WAVE;
    constexpr size_t staging = (size_t)2 * (BM + BN) * PITCH * sizeof(bf16);
    constexpr size_t exchange = MODE == MODE_GATED ? (size_t)(WM * WN / 2) * (BM / WM / 32) * (BN / WN / 32) * 16 * XRT_WAVE * sizeof(float) : 0;
    constexpr size_t lds = staging > exchange ? staging : exchange;
    static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a compute unit");
    auto kernel = gemm_mfma_kernel<BM, BN, WM, WN, MODE, TO>;
    static bool configured = false;          // per instantiation
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        XRT_REQUIRE(e == hipSuccess, "linear (mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN_OUT - 1) / BN_OUT;
    const int total = tiles_m * tiles_n;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);           // a whole number of rounds over the XCDs
    kernel<<<grid, THREADS, lds, s>>>(a, w, out, M, N, K, tiles_m, tiles_n);
    XRT_LAUNCH_CHECK("linear (mfma)");
    return 0;
}

template <typename TO>
int launch_shape(const bf16* a, const bf16* w, TO* out, int M, int N, int K, int mode, hipStream_t s) {
    // large tiles when they still fill the chip's 256 compute units, else smaller ones
    const long big_tiles = (long)((M + 255) / 256) * ((N + 255) / 256);
    const bool big = big_tiles >= 192;
    if (mode == MODE_STORE) return big ? launch<256, 256, 2, 4, MODE_STORE, TO>(a, w, out, M, N, K, s)
                                       : launch<128, 128, 2, 2, MODE_STORE, TO>(a, w, out, M, N, K, s);
    if (mode == MODE_ACCUMULATE) return big ? launch<256, 256, 2, 4, MODE_ACCUMULATE, TO>(a, w, out, M, N, K, s)
                                            : launch<128, 128, 2, 2, MODE_ACCUMULATE, TO>(a, w, out, M, N, K, s);
    const long big_gated = (long)((M + 255) / 256) * ((N + 127) / 128);
    return big_gated >= 192 ? launch<256, 256, 2, 4, MODE_GATED, TO>(a, w, out, M, N, K, s)
                            : launch<128, 128, 2, 2, MODE_GATED, TO>(a, w, out, M, N, K, s);
}

}  // namespace

bool xrt_linear_mfma_accepts(const void* a, const void* w, int M, int N, int K, int mode) {
    const long rows_w = mode == MODE_GATED ? 2L * N : N;     // operands are addressed with 32-bit element offsets
    return K % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 && (long)M * K < (1L << 31) && rows_w * K < (1L << 31);
}

int xrt_linear_mfma(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode,
                    hipStream_t s) {
    if (out_dtype == XRT_F32) return launch_shape<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, s);
    return launch_shape<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, s);
}
