// Matrix product for few rows (M <= 64: decode steps and short prompts), bfloat16 operands,
// float32 accumulation on the matrix cores: out[m, n] = sum_k x[m, k] * w[n, k].
//
// Such a product is bound by reading w once from HBM, so the kernel is built around that
// stream. A workgroup of 8 wavefronts owns 16 (or 32) rows of w. Each wavefront takes one
// eighth of K and streams its part of those rows straight from global memory into the A
// operand of v_mfma_f32_16x16x32_bf16: lane (r, c) reads 64 contiguous bytes of row r per
// 128-wide K step (four 16-byte loads in flight), so a row is read in 256-byte runs. The B
// operand holds the activations x (16 rows of m per tile), read with the same K permutation.
// The eight partial sums are added in wavefront order through LDS, so the result does not
// depend on timing. Epilogues: store (bfloat16 or float32), accumulate into float32, or the
// gated pair silu(gate) * up with the two halves of w (rows n and n + N).
//
// The product can take the RMSNorm before it along: x is then the float32 residual stream
// (optionally only some of its rows), the B operand is x[m, k] * weight[k] rounded to bfloat16,
// every lane adds up the squares of what it reads, and since the wavefronts of a workgroup
// cover all of K between them, their sums give 1/sqrt(mean(x^2) + eps) of every row, which
// scales the accumulators in the epilogue. (rmsnorm.rs:26-43 of the reference: the factor is
// a scalar per row, so it commutes with the product.)
#include <type_traits>

#include "common.h"
#include "xrt_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVES = 8;
constexpr int KSTEP = 128;       // K covered by one step of a wavefront: 4 lane groups x 32
enum { MODE_STORE = 0, MODE_ACCUMULATE = 1, MODE_GATED = 2 };

__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

struct NoNorm {};

// MT: tiles of 16 rows of x; RT: tiles of 16 rows of w per wavefront; GATED doubles the w tiles.
// TX = bf16: x is the product's operand as it is. TX = float: x is the residual stream and the
// RMSNorm with weights `gamma` (of type TG) and `eps` is applied on the way; `rows` (optional)
// picks the rows of x.
// With one tile of x (the common decode case) the kernel is held to 128 registers, so that two
// workgroups fit a compute unit: the stream from HBM needs that many wavefronts in flight.
template <int MT, int RT, int MODE, typename TO, typename TX, typename TG>
__global__ void __launch_bounds__(WAVES * XRT_WAVE, (MT == 1 ? 4 : 2)) gemm_skinny_kernel(
    const TX* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out, int M, int N, int K,
    const TG* __restrict__ gamma, float eps, const int* __restrict__ rows) {
    constexpr int WT = RT * (MODE == MODE_GATED ? 2 : 1);       // w tiles per wavefront
    constexpr bool NORM = sizeof(TX) == 4;
    __shared__ floatx4 partial[2][WAVES][XRT_WAVE];
    __shared__ float squares[NORM ? WAVES : 1][MT][16];

    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int r = lane % 16, c = lane / 16;
    const long n0 = (long)blockIdx.x * (16 * RT);

    const int steps = (K + KSTEP - 1) / KSTEP;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int k_begin = wave * steps_per_wave * KSTEP;
    const int k_end = min(K, k_begin + steps_per_wave * KSTEP);

    // CHAINS accumulators per output tile, used in turn and added at the end: products that do
    // not wait on each other keep the wavefront issuing (its next loads above all)
    constexpr int CHAINS = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    floatx4 chain[CHAINS][WT][MT];
#pragma unroll
    for (int h = 0; h < CHAINS; ++h)
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m) chain[h][t][m] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Addresses are clamped into the operands instead of guarding every load: a row of w beyond
    // N (or of x beyond M) reads the last row, and what it contributes lands in outputs that are
    // never written. Loads without branches around them can all be in flight together.
    const bf16* w_ptr[WT];
#pragma unroll
    for (int t = 0; t < WT; ++t) {
        const int rt = t % RT, half = t / RT;                   // half 1: the "up" rows of a gated product
        const long n = min(n0 + rt * 16 + r, (long)N - 1);
        w_ptr[t] = w + (n + (long)half * N) * K + c * 32;
    }
    const TX* x_ptr[MT];
    float sum_sq[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        long row = min(m * 16 + r, M - 1);
        if constexpr (NORM) { if (rows != nullptr) row = rows[row]; }
        x_ptr[m] = x + row * (long)K + c * 32;
        sum_sq[m] = 0.f;
    }

    struct XRaw { float4 lo, hi; };                              // eight float32 of x, before the norm's weight
    typedef typename std::conditional<NORM, XRaw, bf16x8>::type XReg;

    auto load_w = [&](bf16x8 (&regs)[WT][4], int kb) {
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) regs[t][j] = *reinterpret_cast<const bf16x8*>(w_ptr[t] + kb + j * 8);
    };
    auto load_x = [&](XReg (&regs)[MT][4], int kb) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (NORM) {
                    const float* src = reinterpret_cast<const float*>(x_ptr[m]) + kb + j * 8;
                    regs[m][j].lo = *reinterpret_cast<const float4*>(src);
                    regs[m][j].hi = *reinterpret_cast<const float4*>(src + 4);
                } else {
                    regs[m][j] = *reinterpret_cast<const bf16x8*>(x_ptr[m] + kb + j * 8);
                }
            }
    };
    // the B operand from what was loaded of x: as it is, or times the norm's weight (and the
    // squares are added up on the way)
    auto operand = [&](const XReg& raw, int m, int k) -> bf16x8 {
        if constexpr (!NORM) {
            return raw;
        } else {
            struct alignas(sizeof(TG) * 8) Eight { TG e[8]; };
            const Eight g = *reinterpret_cast<const Eight*>(gamma + k);
            const float v[8] = {raw.lo.x, raw.lo.y, raw.lo.z, raw.lo.w, raw.hi.x, raw.hi.y, raw.hi.z, raw.hi.w};
            bf16x8 value;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sum_sq[m] = fmaf(v[e], v[e], sum_sq[m]);
                value[e] = (bf16)(v[e] * to_float(g.e[e]));
            }
            return value;
        }
    };
    auto multiply = [&](const bf16x8 (&wregs)[WT][4], const XReg (&xregs)[MT][4], int kb) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bf16x8 b[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) b[m] = operand(xregs[m][j], m, kb + c * 32 + j * 8);
#pragma unroll
            for (int t = 0; t < WT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    chain[j % CHAINS][t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wregs[t][j], b[m], chain[j % CHAINS][t][m], 0, 0, 0);
        }
    };

    // Whole steps of 128 along k run through a pipeline of two register sets: while the matrix
    // cores consume one step, the loads of the next are in flight. The steady-state loop body has
    // no branch; the last one or two steps are peeled off.
    const int full = max(0, (min(k_end, K / KSTEP * KSTEP) - k_begin) / KSTEP);     // whole steps of this wavefront
    if (full > 0) {
        bf16x8 w_a[WT][4], w_b[WT][4];
        XReg x_a[MT][4], x_b[MT][4];
        load_x(x_a, k_begin);
        load_w(w_a, k_begin);
        int i = 0;
        for (; i + 2 < full; i += 2) {
            load_x(x_b, k_begin + (i + 1) * KSTEP);
            load_w(w_b, k_begin + (i + 1) * KSTEP);
            multiply(w_a, x_a, k_begin + i * KSTEP);
            load_x(x_a, k_begin + (i + 2) * KSTEP);
            load_w(w_a, k_begin + (i + 2) * KSTEP);
            multiply(w_b, x_b, k_begin + (i + 1) * KSTEP);
        }
        if (full - i == 2) {
            load_x(x_b, k_begin + (i + 1) * KSTEP);
            load_w(w_b, k_begin + (i + 1) * KSTEP);
            multiply(w_a, x_a, k_begin + i * KSTEP);
            multiply(w_b, x_b, k_begin + (i + 1) * KSTEP);
        } else {
            multiply(w_a, x_a, k_begin + i * KSTEP);
        }
    }
    // what is left of K when it is no multiple of 128: one guarded step, in the wavefront that owns it
    const int tail_begin = k_begin + full * KSTEP;
    if (tail_begin < k_end) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = tail_begin + c * 32 + j * 8;
            const bool inside = k + 8 <= K;                      // K is a multiple of 8
            bf16x8 b[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                XReg raw{};
                if (inside) {
                    if constexpr (NORM) {
                        const float* src = reinterpret_cast<const float*>(x_ptr[m]) + tail_begin + j * 8;
                        raw.lo = *reinterpret_cast<const float4*>(src);
                        raw.hi = *reinterpret_cast<const float4*>(src + 4);
                    } else {
                        raw = *reinterpret_cast<const bf16x8*>(x_ptr[m] + tail_begin + j * 8);
                    }
                }
                b[m] = inside ? operand(raw, m, k) : bf16x8{};
            }
#pragma unroll
            for (int t = 0; t < WT; ++t) {
                const bf16x8 a = inside ? *reinterpret_cast<const bf16x8*>(w_ptr[t] + tail_begin + j * 8) : bf16x8{};
#pragma unroll
                for (int m = 0; m < MT; ++m) chain[0][t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[m], chain[0][t][m], 0, 0, 0);
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

    if constexpr (NORM) {
        // squares of every row: over the four lanes that share a row, then (below) over the wavefronts
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = sum_sq[m];
            v += __shfl_xor(v, 16, XRT_WAVE);
            v += __shfl_xor(v, 32, XRT_WAVE);
            if (c == 0) squares[wave][m][r] = v;
        }
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
                float inv_rms = 1.0f;
                if constexpr (NORM) {
                    float total = 0.f;
#pragma unroll
                    for (int other = 0; other < WAVES; ++other) total += squares[other][m][r];
                    inv_rms = 1.0f / sqrtf(total / (float)K + eps);
                }
                const float g[4] = {gate_sum.x * inv_rms, gate_sum.y * inv_rms, gate_sum.z * inv_rms, gate_sum.w * inv_rms};
                const float u[4] = {up_sum.x * inv_rms, up_sum.y * inv_rms, up_sum.z * inv_rms, up_sum.w * inv_rms};
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

template <int MT, int RT, typename TO, typename TX, typename TG>
int launch_mode(const TX* x, const bf16* w, TO* out, int M, int N, int K, int mode, const TG* gamma, float eps,
                const int* rows, hipStream_t s) {
    const unsigned grid = (unsigned)((N + 16 * RT - 1) / (16 * RT));
    const dim3 block(WAVES * XRT_WAVE);
    constexpr bool NORM = sizeof(TX) == 4;
    if (mode == MODE_STORE)
        gemm_skinny_kernel<MT, RT, MODE_STORE, TO, TX, TG><<<grid, block, 0, s>>>(x, w, out, M, N, K, gamma, eps, rows);
    else if (mode == MODE_GATED) {
        if constexpr (RT == 1)
            gemm_skinny_kernel<MT, RT, MODE_GATED, TO, TX, TG><<<grid, block, 0, s>>>(x, w, out, M, N, K, gamma, eps, rows);
        else { xrt_set_error("linear (skinny): a gated product takes one row tile per wavefront"); return 1; }
    } else {
        if constexpr (!NORM)
            gemm_skinny_kernel<MT, RT, MODE_ACCUMULATE, TO, TX, TG><<<grid, block, 0, s>>>(x, w, out, M, N, K, gamma, eps, rows);
        else { xrt_set_error("linear (skinny): a product with a norm does not accumulate"); return 1; }
    }
    XRT_LAUNCH_CHECK("linear (skinny)");
    return 0;
}

template <typename TO, typename TX, typename TG>
int launch_tiles(const TX* x, const bf16* w, TO* out, int M, int N, int K, int mode, const TG* gamma, float eps,
                 const int* rows, hipStream_t s) {
    const int mt = (M + 15) / 16;
    // two row tiles per wavefront keep more loads in flight and halve the reads of x, if enough
    // workgroups remain to fill the chip
    const bool wide = (N / 32) >= 1024 && mode != MODE_GATED;
#define XRT_SKINNY(MT_) (wide ? launch_mode<MT_, 2, TO, TX, TG>(x, w, out, M, N, K, mode, gamma, eps, rows, s) \
                              : launch_mode<MT_, 1, TO, TX, TG>(x, w, out, M, N, K, mode, gamma, eps, rows, s))
    constexpr bool NORM = sizeof(TX) == 4;
    if (mt == 1) return XRT_SKINNY(1);
    if (mt == 2) return XRT_SKINNY(2);
    if constexpr (!NORM) {                       // with a norm, float32 x for more rows would not fit the registers
        if (mt == 3) return XRT_SKINNY(3);
        return XRT_SKINNY(4);
    } else {
        xrt_set_error("linear (skinny): a product with a norm takes at most 32 rows, found %d", M);
        return 1;
    }
#undef XRT_SKINNY
}

}  // namespace

// Whether the skinny kernel takes this product (bfloat16 weights assumed by the caller).
bool xrt_linear_skinny_accepts(const void* a, const void* w, int M, int K) {
    return M >= 1 && M <= 64 && K % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
}

int xrt_linear_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int mode,
                      hipStream_t s) {
    const NoNorm* none = nullptr;
    if (out_dtype == XRT_F32)
        return launch_tiles<float, bf16, NoNorm>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K, mode, none, 0.f, nullptr, s);
    return launch_tiles<bf16, bf16, NoNorm>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K, mode, none, 0.f, nullptr, s);
}

// out = rmsnorm(x[rows], gamma, eps) . w^T, x float32 [*, K]; mode store or gated
int xrt_norm_linear_skinny(const float* x, const int* rows, const void* gamma, int gamma_dtype, float eps, const void* w,
                           void* out, int out_dtype, int M, int N, int K, int mode, hipStream_t s) {
    if (gamma_dtype == XRT_F32) {
        if (out_dtype == XRT_F32)
            return launch_tiles<float, float, float>(x, (const bf16*)w, (float*)out, M, N, K, mode, (const float*)gamma, eps, rows, s);
        return launch_tiles<bf16, float, float>(x, (const bf16*)w, (bf16*)out, M, N, K, mode, (const float*)gamma, eps, rows, s);
    }
    if (out_dtype == XRT_F32)
        return launch_tiles<float, float, bf16>(x, (const bf16*)w, (float*)out, M, N, K, mode, (const bf16*)gamma, eps, rows, s);
    return launch_tiles<bf16, float, bf16>(x, (const bf16*)w, (bf16*)out, M, N, K, mode, (const bf16*)gamma, eps, rows, s);
}
