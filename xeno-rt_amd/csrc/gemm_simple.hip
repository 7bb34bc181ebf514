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
            if constexpr (MODE == MODE_GATED) *dst = from_float<TO>(gate_activation(acc[i][j], activation) * acc_up[i][j]);
        }
    }
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
    if (dtype == XRT_F32 && out_dtype == XRT_F32) return launch<float, float>(a, w, out, M, N, K, mode, activation, s);
    if (dtype == XRT_BF16 && out_dtype == XRT_F32) return launch<bf16, float>(a, w, out, M, N, K, mode, activation, s);
    if (dtype == XRT_BF16 && out_dtype == XRT_BF16) return launch<bf16, bf16>(a, w, out, M, N, K, mode, activation, s);
    xrt_set_error("linear: unsupported dtypes in=%d out=%d", dtype, out_dtype);
    return 1;
}
