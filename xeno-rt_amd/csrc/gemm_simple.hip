// Plain tiled matrix product out[m, n] = sum_k a[m, k] * w[n, k] with float32 accumulation
// on the vector ALUs (no matrix cores, no reduced precision): the product of the 32-bit
// path, and the fallback of the bfloat16 path for shapes its fast kernels refuse.
//
// Every output element is summed in the same order, whatever the number of rows, the tile
// it falls in or the batch around it, so a token's result does not depend on how a request
// was cut into steps: the products of 16 consecutive k are added up in order, and these
// sums are added up in order (a long k then loses less to rounding than one running sum:
// the error grows with the square root of k / 16 + 16 instead of k). Semantics of the reference's
// row-major matvec (crates/xrt-kernels/src/cpu/matmul.rs:153-167, 269-288): w is
// [out][in], no bias.
#include "common.h"
#include "xrt_hip.h"
#include "activation.h"

namespace {

constexpr int BN = 64, BK = 16, PAD = 4;
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };

template <typename T>
__device__ __forceinline__ void load4(const T* __restrict__ base, long row, int n_rows, int k, int K,
                                      bool vector_ok, float (&v)[4]) {
    if (row < n_rows && vector_ok && k + 3 < K) {
        const T* p = base + row * (long)K + k;
        if constexpr (sizeof(T) == 4) {
            const float4 q = *reinterpret_cast<const float4*>(p);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
            struct alignas(8) Four { T e[4]; };
            const Four q = *reinterpret_cast<const Four*>(p);
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = to_float(q.e[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            v[i] = (row < n_rows && k + i < K) ? to_float(base[row * (long)K + k + i]) : 0.f;
    }
}

// RM rows of the output per thread: a tile is 16 RM x 64. With few rows of a (a decode step) the
// small tile does a quarter of the arithmetic; an element's sum is the same either way.
template <typename TI, typename TO, int MODE, int RM>
__global__ void __launch_bounds__(256) gemm_simple_kernel(const TI* __restrict__ a, const TI* __restrict__ w,
                                                          TO* __restrict__ out, int M, int N, int K,
                                                          int vector_ok, int activation) {
    constexpr int BM = 16 * RM;
    __shared__ __attribute__((aligned(16))) float As[BK][BM + PAD];
    __shared__ __attribute__((aligned(16))) float Ws[BK][BN + PAD];
    __shared__ __attribute__((aligned(16))) float Us[MODE == MODE_GATED ? BK : 1][BN + PAD];

    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const long m0 = (long)blockIdx.y * BM, n0 = (long)blockIdx.x * BN;
    const int load_row = tid / 4, load_k = (tid % 4) * 4;

    float acc[RM][4] = {}, acc_up[MODE == MODE_GATED ? RM : 1][4] = {};

    // the tile after the one being multiplied is on its way from global memory meanwhile
    float va[4], vw[4], vu[4] = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int k0) {
        if (load_row < BM) load4(a, m0 + load_row, M, k0 + load_k, K, vector_ok, va);
        load4(w, n0 + load_row, N, k0 + load_k, K, vector_ok, vw);
        // rows of the "up" half follow the N rows of the "gate" half
        if constexpr (MODE == MODE_GATED) load4(w + (long)N * K, n0 + load_row, N, k0 + load_k, K, vector_ok, vu);
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (load_row < BM) As[load_k + i][load_row] = va[i];
            Ws[load_k + i][load_row] = vw[i];
            if constexpr (MODE == MODE_GATED) Us[load_k + i][load_row] = vu[i];
        }
        if (k0 + BK < K) fetch(k0 + BK);
        __syncthreads();
        float part[RM][4] = {}, part_up[MODE == MODE_GATED ? RM : 1][4] = {};      // this tile's sums
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float ar[RM];
#pragma unroll
            for (int i = 0; i < RM; ++i) ar[i] = As[kk][ty * RM + i];
            const float4 wv = *reinterpret_cast<const float4*>(&Ws[kk][tx * 4]);
            const float wr[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(ar[i], wr[j], part[i][j]);
            if constexpr (MODE == MODE_GATED) {
                const float4 uv = *reinterpret_cast<const float4*>(&Us[kk][tx * 4]);
                const float ur[4] = {uv.x, uv.y, uv.z, uv.w};
#pragma unroll
                for (int i = 0; i < RM; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) part_up[i][j] = fmaf(ar[i], ur[j], part_up[i][j]);
            }
        }
#pragma unroll
        for (int i = 0; i < RM; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[i][j] += part[i][j];
                if constexpr (MODE == MODE_GATED) acc_up[i][j] += part_up[i][j];
            }
        __syncthreads();
    }

    // when accumulating, the old values are read in one go (from addresses clamped into
    // the matrix) before any is written: guarded one by one, each read would wait for the last
    float before[RM][4] = {};
    if constexpr (MODE == MODE_ACCUMULATE) {
#pragma unroll
        for (int i = 0; i < RM; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                before[i][j] = to_float(out[min(m0 + ty * RM + i, (long)M - 1) * N + min(n0 + tx * 4 + j, (long)N - 1)]);
    }
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        const long m = m0 + ty * RM + i;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long n = n0 + tx * 4 + j;
            if (m >= M || n >= N) continue;
            TO* dst = out + m * (long)N + n;
            if constexpr (MODE == MODE_STORE) *dst = from_float<TO>(acc[i][j]);
            if constexpr (MODE == MODE_ACCUMULATE) *dst = from_float<TO>(before[i][j] + acc[i][j]);
            if constexpr (MODE == MODE_GATED) *dst = from_float<TO>(gate_activation<sizeof(TO) == 2>(acc[i][j], activation) * acc_up[i][j]);
        }
    }
}

// ---- few rows of a (a decode step), float32: the product is bound by reading w once, and the tile kernel above, which
// multiplies a 16 x 64 tile through LDS in steps of 16 along k, reads it at a tenth of what the memory gives. Here a
// workgroup of four wavefronts takes ROWS rows of w (gated: ROWS / 2 gate rows and the up rows of the same outputs) and
// walks k in segments of 64 tiles of 16. In a segment lane t of every wavefront owns tile t: it loads 64 contiguous
// bytes of each of its wavefront's rows (a wavefront's load is four contiguous kilobytes of a row), takes the rows of a,
// eight at a time, from LDS, where their segment was put once for all, and works out the tile's sum for every row of a:
// the products of 16 consecutive k, added up in order. The tiles' sums then go through LDS to one thread per output,
// which adds them to its running sum in the order of k. That is the order of the kernel above, term for term, so an
// output has the same bits whichever kernel made it, and a token's result does not depend on the step it came in.
constexpr int STREAM_ROWS = 16, STREAM_WAVES = 4, STREAM_TILES = 64, STREAM_HALF = 8;
constexpr int STREAM_PITCH = STREAM_TILES + 1;        // of the tiles' sums of one output: the threads that add them up read down a column

template <int MODE>
__global__ void __launch_bounds__(STREAM_WAVES * XRT_WAVE) gemm_stream_kernel(
    const float* __restrict__ a, const float* __restrict__ w, float* __restrict__ out, int M, int N, int K, int activation) {
    constexpr int PER_WAVE = STREAM_ROWS / STREAM_WAVES;
    constexpr int SEGMENT = STREAM_TILES * BK;                               // columns of k per segment
    extern __shared__ __attribute__((aligned(16))) float stream_lds[];
    float* a_segment = stream_lds;                                           // [STREAM_HALF rows of a][SEGMENT]
    float* sums = stream_lds + (long)STREAM_HALF * SEGMENT;                  // [STREAM_ROWS][STREAM_HALF][STREAM_PITCH]
    const int tid = threadIdx.x, lane = tid % XRT_WAVE, wave = tid / XRT_WAVE;
    constexpr int OUTPUTS = MODE == MODE_GATED ? STREAM_ROWS / 2 : STREAM_ROWS;   // outputs per workgroup
    const long n0 = (long)blockIdx.x * OUTPUTS;
    // row of w behind row r of the workgroup's rows (gated: the gate rows of the outputs, then their up rows); clamped
    // into the matrix, and what a clamped row makes is not written
    auto w_row = [&](int r) -> long {
        if constexpr (MODE == MODE_GATED) return min(n0 + r % OUTPUTS, (long)N - 1) + (long)(r / OUTPUTS) * N;
        return min(n0 + r, (long)N - 1);
    };
    const float* rows[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) rows[i] = w + w_row(wave * PER_WAVE + i) * K;
    // the thread that adds up the sums of output row `mine_r`, row `mine_m` of a half of a's rows
    const int mine_r = tid / STREAM_HALF, mine_m = tid % STREAM_HALF;
    const bool adds = mine_r < STREAM_ROWS;
    float running[2] = {0.f, 0.f};                                           // one per half of a's rows
    typedef float floatx4 __attribute__((ext_vector_type(4)));

    // this lane's tile of each of its wavefront's rows of w in a segment: zeros beyond K, as the kernel above pads its
    // last tile. The next segment's tiles are asked for before this segment's sums are worked out.
    floatx4 ahead[PER_WAVE][BK / 4];
    auto ask = [&](int k0) {
        const int columns = min(SEGMENT, K - k0);
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i)
#pragma unroll
            for (int q = 0; q < BK / 4; ++q) {
                const int k = lane * BK + q * 4;
                ahead[i][q] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (k < columns) ahead[i][q] = *reinterpret_cast<const floatx4*>(rows[i] + k0 + k);
            }
    };
    ask(0);
    for (int k0 = 0; k0 < K; k0 += SEGMENT) {
        const int columns = min(SEGMENT, K - k0);                            // a multiple of 4: the launcher checks
        const int tiles = (columns + BK - 1) / BK;
        float wv[PER_WAVE][BK];
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i)
#pragma unroll
            for (int q = 0; q < BK / 4; ++q) {
                const floatx4 v = ahead[i][q];
                wv[i][q * 4] = v[0]; wv[i][q * 4 + 1] = v[1]; wv[i][q * 4 + 2] = v[2]; wv[i][q * 4 + 3] = v[3];
            }
        if (k0 + SEGMENT < K) ask(k0 + SEGMENT);
        for (int half = 0; half * STREAM_HALF < M; ++half) {
            const int m_count = min(STREAM_HALF, M - half * STREAM_HALF);
            // the segment of this half of a's rows, for all wavefronts: the q-th 16 bytes of tile t of row m lie at [m][q][t],
            // so that the lanes of a wavefront, which read the same q of neighbouring tiles, read neighbouring places
            for (int piece = tid; piece < m_count * (SEGMENT / 4); piece += STREAM_WAVES * XRT_WAVE) {
                const int m = piece / (SEGMENT / 4), within = piece % (SEGMENT / 4), k = within * 4;
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (k < columns) v = *reinterpret_cast<const floatx4*>(a + (long)(half * STREAM_HALF + m) * K + k0 + k);
                *reinterpret_cast<floatx4*>(a_segment + (((long)m * (BK / 4) + within % (BK / 4)) * STREAM_TILES + within / (BK / 4)) * 4) = v;
            }
            __syncthreads();
            // the tile's sums: the products of its 16 columns in order, from zero (fmaf as in the kernel above)
            // (two rows of a at a time, so that eight chains of products run side by side; an odd last row is done twice)
            for (int m0 = 0; m0 < m_count; m0 += 2) {
                float av[2][BK];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const float* am = a_segment + (long)min(m0 + u, m_count - 1) * SEGMENT + lane * 4;
#pragma unroll
                    for (int q = 0; q < BK / 4; ++q) {
                        const floatx4 v = *reinterpret_cast<const floatx4*>(am + q * STREAM_TILES * 4);
                        av[u][q * 4] = v[0]; av[u][q * 4 + 1] = v[1]; av[u][q * 4 + 2] = v[2]; av[u][q * 4 + 3] = v[3];
                    }
                }
                float part[2][PER_WAVE];
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < PER_WAVE; ++i) part[u][i] = 0.f;
#pragma unroll
                for (int kk = 0; kk < BK; ++kk)
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int i = 0; i < PER_WAVE; ++i) part[u][i] = fmaf(av[u][kk], wv[i][kk], part[u][i]);
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < PER_WAVE; ++i)
                        sums[((wave * PER_WAVE + i) * STREAM_HALF + min(m0 + u, m_count - 1)) * STREAM_PITCH + lane] = part[u][i];
            }
            __syncthreads();
            if (adds && mine_m < m_count) {
                // all tiles' sums are asked for at once, then added in the order of k (those beyond K are not)
                const float* mine = sums + (mine_r * STREAM_HALF + mine_m) * STREAM_PITCH;
                float of_tile[STREAM_TILES];
#pragma unroll
                for (int t = 0; t < STREAM_TILES; ++t) of_tile[t] = mine[t];
                float sum = running[half];
#pragma unroll
                for (int t = 0; t < STREAM_TILES; ++t) sum = t < tiles ? sum + of_tile[t] : sum;
                running[half] = sum;
            }
            __syncthreads();
        }
    }
    // ---- epilogue: thread (mine_r, mine_m) holds output row mine_r for rows mine_m and mine_m + 8 of a
    if constexpr (MODE == MODE_GATED) {
        // the up sums go to the threads that hold the gate sums of the same outputs
        if (adds && mine_r >= OUTPUTS) { sums[(mine_r * STREAM_HALF + mine_m) * 2] = running[0]; sums[(mine_r * STREAM_HALF + mine_m) * 2 + 1] = running[1]; }
        __syncthreads();
    }
    if (!adds || mine_r >= OUTPUTS || n0 + mine_r >= N) return;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int m = half * STREAM_HALF + mine_m;
        if (m >= M) continue;
        float* dst = out + (long)m * N + n0 + mine_r;
        if constexpr (MODE == MODE_STORE) *dst = running[half];
        if constexpr (MODE == MODE_ACCUMULATE) *dst = *dst + running[half];
        if constexpr (MODE == MODE_GATED) *dst = gate_activation(running[half], activation) * sums[((mine_r + OUTPUTS) * STREAM_HALF + mine_m) * 2 + half];
    }
}

// Whether the kernel above takes the product: float32, up to 16 rows of a, whole pieces of 16 bytes.
bool stream_takes(const void* a, const void* w, int M, int K) {
    return M >= 1 && M <= 2 * STREAM_HALF && K % 4 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
}

int launch_stream(const float* a, const float* w, float* out, int M, int N, int K, int mode, int activation, hipStream_t s) {
    const int outputs = mode == MODE_GATED ? STREAM_ROWS / 2 : STREAM_ROWS;
    const unsigned grid = (unsigned)((N + outputs - 1) / outputs);
    const size_t lds = ((size_t)STREAM_HALF * STREAM_TILES * BK + (size_t)STREAM_ROWS * STREAM_HALF * STREAM_PITCH) * sizeof(float);
#define XRT_STREAM(MODE_)                                                                                                    \
    do {                                                                                                                     \
        static bool configured = false;                                                                                      \
        if (!configured) {                                                                                                   \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_stream_kernel<MODE_>),                     \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                      \
            XRT_REQUIRE(e == hipSuccess, "linear (plain, few rows): cannot reserve LDS: %s", hipGetErrorString(e));          \
            configured = true;                                                                                               \
        }                                                                                                                    \
        gemm_stream_kernel<MODE_><<<grid, STREAM_WAVES * XRT_WAVE, lds, s>>>(a, w, out, M, N, K, activation);                \
    } while (0)
    if (mode == MODE_STORE) XRT_STREAM(MODE_STORE);
    else if (mode == MODE_ACCUMULATE) XRT_STREAM(MODE_ACCUMULATE);
    else XRT_STREAM(MODE_GATED);
#undef XRT_STREAM
    XRT_LAUNCH_CHECK("linear (plain, few rows)");
    return 0;
}

template <typename TI, typename TO, int RM>
void launch_rows(const void* a, const void* w, void* out, int M, int N, int K, int mode, int activation, hipStream_t s) {
    constexpr int BM = 16 * RM;
    const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    const int vector_ok = (K % 4 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
    if (mode == MODE_STORE)
        gemm_simple_kernel<TI, TO, MODE_STORE, RM><<<grid, 256, 0, s>>>((const TI*)a, (const TI*)w, (TO*)out, M, N, K, vector_ok, activation);
    else if (mode == MODE_ACCUMULATE)
        gemm_simple_kernel<TI, TO, MODE_ACCUMULATE, RM><<<grid, 256, 0, s>>>((const TI*)a, (const TI*)w, (TO*)out, M, N, K, vector_ok, activation);
    else
        gemm_simple_kernel<TI, TO, MODE_GATED, RM><<<grid, 256, 0, s>>>((const TI*)a, (const TI*)w, (TO*)out, M, N, K, vector_ok, activation);
}

template <typename TI, typename TO>
int launch(const void* a, const void* w, void* out, int M, int N, int K, int mode, int activation, hipStream_t s) {
    if (M <= 16) launch_rows<TI, TO, 1>(a, w, out, M, N, K, mode, activation, s);
    else launch_rows<TI, TO, 4>(a, w, out, M, N, K, mode, activation, s);
    XRT_LAUNCH_CHECK("linear (plain)");
    return 0;
}

}  // namespace

int xrt_linear_plain(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
                     int mode, int activation, hipStream_t s) {
    if (dtype == XRT_F32 && out_dtype == XRT_F32 && stream_takes(a, w, M, K))
        return launch_stream((const float*)a, (const float*)w, (float*)out, M, N, K, mode, activation, s);
    if (dtype == XRT_F32 && out_dtype == XRT_F32) return launch<float, float>(a, w, out, M, N, K, mode, activation, s);
    if (dtype == XRT_BF16 && out_dtype == XRT_F32) return launch<bf16, float>(a, w, out, M, N, K, mode, activation, s);
    if (dtype == XRT_BF16 && out_dtype == XRT_BF16) return launch<bf16, bf16>(a, w, out, M, N, K, mode, activation, s);
    xrt_set_error("linear: unsupported dtypes in=%d out=%d", dtype, out_dtype);
    return 1;
}
