// Matrix product for few rows (M <= 64: decode steps and short prompts), bfloat16 operands,
// float32 accumulation on the matrix cores: out[m, n] = sum_k x[m, k] * w[n, k].
//
// Such a product is bound by reading w once from HBM, so the kernel is built around that
// stream. A workgroup of 8 wavefronts owns 16 (or 32) rows of w. Each wavefront takes one
// eighth of K and streams its part of those rows straight from global memory into the A
// operand of v_mfma_f32_16x16x32_bf16: a 128-wide K step is four load instructions, and in each
// the four lanes (r, 0..3) of a row read 64 contiguous bytes of it, so that one instruction
// asks for 16 half cache lines and a row is read in 256-byte runs. The B operand holds the
// activations x (16 rows of m per tile), read with the same K permutation. Loads carry no
// branches (addresses are clamped into the operands instead), run one step ahead of the
// matrix cores, and the products of a step go to accumulators that do not wait on each other:
// all three matter, because a wavefront that stalls stops issuing its next loads.
// The eight partial sums are added in wavefront order through LDS, so the result does not
// depend on timing. Epilogues: store (bfloat16 or float32), accumulate into float32, or the
// gated pair silu(gate) * up with the two halves of w (rows n and n + N).
#include "common.h"
#include "xrt_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVES = 8;
constexpr int KSTEP = 128;       // K covered by one step of a wavefront: 4 lane groups x 32
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };

__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

// MT: tiles of 16 rows of x; RT: tiles of 16 rows of w per wavefront; GATED doubles the w tiles.
// With one tile of x (the common decode case) the kernel is held to 128 registers, so that at
// least two workgroups fit a compute unit: the stream from HBM needs the wavefronts in flight.
template <int MT, int RT, int MODE, typename TO>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, (MT == 1 ? 4 : 2)) gemm_skinny_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K) {
    constexpr int WT = RT * (MODE == MODE_GATED ? 2 : 1);       // w tiles per wavefront
    __shared__ floatx4 partial[2][WAVES][XRT_WAVE];

    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int r = lane % 16, c = lane / 16;
    const long n0 = (long)blockIdx.x * (16 * RT);

    const int steps = (K + KSTEP - 1) / KSTEP;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int k_begin = wave * steps_per_wave * KSTEP;
    const int k_end = min(K, k_begin + steps_per_wave * KSTEP);

    // CHAINS accumulators per output tile, used in turn and added at the end
    constexpr int CHAINS = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
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
        const long n = min(n0 + rt * 16 + r, (long)N - 1);
        w_ptr[t] = w + (n + (long)half * N) * K + c * 8;
    }
    const bf16* x_ptr[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) x_ptr[m] = x + (long)min(m * 16 + r, M - 1) * K + c * 8;

    auto load_w = [&](bf16x8 (&regs)[WT][4], int kb) {
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) regs[t][j] = *reinterpret_cast<const bf16x8*>(w_ptr[t] + kb + j * 32);
    };
    auto load_x = [&](bf16x8 (&regs)[MT][4], int kb) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j) regs[m][j] = *reinterpret_cast<const bf16x8*>(x_ptr[m] + kb + j * 32);
    };
    auto multiply = [&](const bf16x8 (&wregs)[WT][4], const bf16x8 (&xregs)[MT][4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < WT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    chain[j % CHAINS][t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wregs[t][j], xregs[m][j], chain[j % CHAINS][t][m], 0, 0, 0);
    };

    // Whole steps of 128 along k run through a pipeline of two register sets: while the matrix
    // cores consume one step, the loads of the next are in flight. The steady-state loop body has
    // no branch; the last one or two steps are peeled off.
    const int full = max(0, (min(k_end, K / KSTEP * KSTEP) - k_begin) / KSTEP);     // whole steps of this wavefront
    if (full > 0) {
        bf16x8 w_a[WT][4], w_b[WT][4];
        bf16x8 x_a[MT][4], x_b[MT][4];
        load_x(x_a, k_begin);
        load_w(w_a, k_begin);
        int i = 0;
        for (; i + 2 < full; i += 2) {
            load_x(x_b, k_begin + (i + 1) * KSTEP);
            load_w(w_b, k_begin + (i + 1) * KSTEP);
            multiply(w_a, x_a);
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
    }
    // what is left of K when it is no multiple of 128: one guarded step, in the wavefront that owns it
    const int tail_begin = k_begin + full * KSTEP;
    if (tail_begin < k_end) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
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
        const int slot = tile & 1;
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
            if (mm < M) {
                const float g[4] = {gate_sum.x, gate_sum.y, gate_sum.z, gate_sum.w};
                const float u[4] = {up_sum.x, up_sum.y, up_sum.z, up_sum.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (nn + i >= N) continue;
                    TO* dst = out + (long)mm * N + nn + i;
                    if constexpr (MODE == MODE_STORE) *dst = from_float<TO>(g[i]);
                    if constexpr (MODE == MODE_ACCUMULATE) *dst = from_float<TO>(to_float(*dst) + g[i]);
                    if constexpr (MODE == MODE_GATED) *dst = from_float<TO>(silu(g[i]) * u[i]);
                }
            }
        }
        // slots alternate, and a slot is rewritten only two tiles later, after this tile's barrier
    }
}

template <int MT, int RT, typename TO>
int launch_mode(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, hipStream_t s) {
    const unsigned grid = (unsigned)((N + 16 * RT - 1) / (16 * RT));
    const dim3 block(WAVES * XRT_WAVE);
    if (mode == MODE_STORE)
        gemm_skinny_kernel<MT, RT, MODE_STORE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K);
    else if (mode == MODE_ACCUMULATE)
        gemm_skinny_kernel<MT, RT, MODE_ACCUMULATE, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K);
    else if constexpr (RT == 1)
        gemm_skinny_kernel<MT, RT, MODE_GATED, TO><<<grid, block, 0, s>>>(x, w, out, M, N, K);
    else {
        xrt_set_error("linear (skinny): a gated product takes one row tile per wavefront");
        return 1;
    }
    XRT_LAUNCH_CHECK("linear (skinny)");
    return 0;
}

template <typename TO>
int launch_tiles(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int mode, hipStream_t s) {
    const int mt = (M + 15) / 16;
    // two row tiles per wavefront keep more loads in flight and halve the reads of x, if enough
    // workgroups remain to fill the chip
    // (with three or four tiles of x the reads of x from L2 outweigh those of w from HBM: then
    // the wider tile pays as soon as it leaves most compute units a workgroup)
    const bool wide = mode != MODE_GATED && (N / 32) >= (mt >= 3 ? 160 : 1024);
#define XRT_SKINNY(MT_) (wide ? launch_mode<MT_, 2, TO>(x, w, out, M, N, K, mode, s) : launch_mode<MT_, 1, TO>(x, w, out, M, N, K, mode, s))
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

int xrt_linear_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode,
                      hipStream_t s) {
    if (out_dtype == XRT_F32) return launch_tiles<float>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, s);
    return launch_tiles<bf16>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, s);
}
