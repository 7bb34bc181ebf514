// Embedding gather, residual add and RMSNorm.
//
// RMSNorm: y = (x * r) * w, r = 1/sqrt(mean(x^2) + eps), all in float32
// (reference: crates/xrt-kernels/src/cpu/rmsnorm.rs:26-43). One workgroup per row;
// the order of the sum depends only on the row length, so a row's result is the
// same in any batch.
#include "common.h"
#include "xrt_hip.h"
#include "packing.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int hidden) {
    const long token = blockIdx.x;
    const T* row = table + (long)ids[token] * hidden;
    float* dst = out + token * hidden;
    if constexpr (sizeof(T) == 2) {
        if (hidden % 8 == 0) {              // 16 bytes of the row a lane and step (a row then starts at a multiple of 16 bytes)
            for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
                const bf16x8 eight = *reinterpret_cast<const bf16x8*>(row + i);
                float4 low, high;
                low.x = (float)eight[0]; low.y = (float)eight[1]; low.z = (float)eight[2]; low.w = (float)eight[3];
                high.x = (float)eight[4]; high.y = (float)eight[5]; high.z = (float)eight[6]; high.w = (float)eight[7];
                *reinterpret_cast<float4*>(dst + i) = low;
                *reinterpret_cast<float4*>(dst + i + 4) = high;
            }
            return;
        }
    }
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(row[i]);
}

// the same from a table kept in tiles (a table that is also the output head's weight)
__global__ void embed_packed_kernel(const bf16* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, const Packing packing) {
    const long token = blockIdx.x;
    const long row = packed_row(packing, ids[token]);
    float* dst = out + token * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(table[packed_offset(row, i / 8 * 8, hidden) + i % 8]);
}

template <typename T>
__global__ void add_kernel(float* __restrict__ residual, const T* __restrict__ delta, long count) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) residual[i] += to_float(delta[i]);
}

template <typename T> struct alignas(sizeof(T) * 4) Vec4 { T e[4]; };

// Rows whose length is a multiple of 4 are read once, 16 bytes per lane and all loads in flight
// together, and kept in registers between the sum and the scaling (up to CACHED * 1024 elements;
// the rest of a longer row is read twice). Other rows take the scalar path. The order of the sum
// depends only on the row length.
template <typename TW, typename TO>
__global__ void __launch_bounds__(256) rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ weight,
                                                      float eps, TO* __restrict__ out,
                                                      const int* __restrict__ rows, int hidden) {
    constexpr int CACHED = 8;
    __shared__ float scratch[32];
    const long src = rows ? rows[blockIdx.x] : blockIdx.x;
    const float* row = x + src * hidden;
    TO* dst = out + (long)blockIdx.x * hidden;
    if (hidden % 4 == 0) {
        const int quads = hidden / 4;
        const float4* row4 = reinterpret_cast<const float4*>(row);
        float4 kept[CACHED];
        Vec4<TW> gain[CACHED];                                  // asked for now, so that they arrive under the sum
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < CACHED; ++i) {
            const int q = threadIdx.x + i * 256;
            kept[i] = q < quads ? row4[q] : make_float4(0.f, 0.f, 0.f, 0.f);
            gain[i] = q < quads ? *reinterpret_cast<const Vec4<TW>*>(weight + 4 * q) : Vec4<TW>{};
        }
#pragma unroll
        for (int i = 0; i < CACHED; ++i)
            sum = fmaf(kept[i].x, kept[i].x, fmaf(kept[i].y, kept[i].y, fmaf(kept[i].z, kept[i].z, fmaf(kept[i].w, kept[i].w, sum))));
        for (int q = threadIdx.x + CACHED * 256; q < quads; q += 256) {
            const float4 v = row4[q];
            sum = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, sum))));
        }
        sum = block_sum(sum, scratch);
        const float inv_rms = 1.0f / sqrtf(sum / (float)hidden + eps);
        auto emit = [&](int q, const float4& v, const Vec4<TW>& w) {
            Vec4<TO> r;
            r.e[0] = from_float<TO>((v.x * inv_rms) * to_float(w.e[0]));
            r.e[1] = from_float<TO>((v.y * inv_rms) * to_float(w.e[1]));
            r.e[2] = from_float<TO>((v.z * inv_rms) * to_float(w.e[2]));
            r.e[3] = from_float<TO>((v.w * inv_rms) * to_float(w.e[3]));
            *reinterpret_cast<Vec4<TO>*>(dst + 4 * q) = r;
        };
#pragma unroll
        for (int i = 0; i < CACHED; ++i) {
            const int q = threadIdx.x + i * 256;
            if (q < quads) emit(q, kept[i], gain[i]);
        }
        for (int q = threadIdx.x + CACHED * 256; q < quads; q += 256) emit(q, row4[q], *reinterpret_cast<const Vec4<TW>*>(weight + 4 * q));
        return;
    }
    float sum = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) sum = fmaf(row[i], row[i], sum);
    sum = block_sum(sum, scratch);
    const float inv_rms = 1.0f / sqrtf(sum / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x)
        dst[i] = from_float<TO>((row[i] * inv_rms) * to_float(weight[i]));
}

extern "C" int xrt_embed(const void* table, int table_dtype, const xrt_packing* packing, const int* ids, float* out, int tokens,
                         int hidden, int vocab, void* stream) {
    XRT_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes tokens=%d hidden=%d vocab=%d", tokens, hidden, vocab);
    XRT_REQUIRE(table_dtype == XRT_F32 || table_dtype == XRT_BF16, "embed: unknown dtype %d", table_dtype);
    if (tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (packing && is_packed(*packing)) {
        XRT_REQUIRE(packing->kind == XRT_PACK_TILES && table_dtype == XRT_BF16 && hidden % 32 == 0,
                    "embed: a packed table is bfloat16 in plain tiles with a width that is a multiple of 32");
        embed_packed_kernel<<<tokens, 256, 0, s>>>((const bf16*)table, ids, out, hidden, *packing);
        XRT_LAUNCH_CHECK("embed (packed)");
        return 0;
    }
    if (table_dtype == XRT_F32)
        embed_kernel<float><<<tokens, 256, 0, s>>>((const float*)table, ids, out, hidden);
    else
        embed_kernel<bf16><<<tokens, 256, 0, s>>>((const bf16*)table, ids, out, hidden);
    XRT_LAUNCH_CHECK("embed");
    return 0;
}

extern "C" int xrt_add(float* residual, const void* delta, int delta_dtype, long count, void* stream) {
    XRT_REQUIRE(count >= 0, "add: negative count");
    XRT_REQUIRE(delta_dtype == XRT_F32 || delta_dtype == XRT_BF16, "add: unknown dtype %d", delta_dtype);
    if (count == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (delta_dtype == XRT_F32)
        add_kernel<float><<<blocks, 256, 0, s>>>(residual, (const float*)delta, count);
    else
        add_kernel<bf16><<<blocks, 256, 0, s>>>(residual, (const bf16*)delta, count);
    XRT_LAUNCH_CHECK("add");
    return 0;
}

extern "C" int xrt_rmsnorm(const float* x, const void* weight, int weight_dtype, float eps, void* out,
                           int out_dtype, const int* rows, int n_rows, int hidden, void* stream) {
    XRT_REQUIRE(n_rows >= 0 && hidden > 0, "rmsnorm: bad sizes rows=%d hidden=%d", n_rows, hidden);
    XRT_REQUIRE((weight_dtype == XRT_F32 || weight_dtype == XRT_BF16) && (out_dtype == XRT_F32 || out_dtype == XRT_BF16),
                "rmsnorm: unknown dtype weight=%d out=%d", weight_dtype, out_dtype);
    if (n_rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define XRT_RMS(TW, TO) rmsnorm_kernel<TW, TO><<<n_rows, 256, 0, s>>>(x, (const TW*)weight, eps, (TO*)out, rows, hidden)
    if (weight_dtype == XRT_F32 && out_dtype == XRT_F32) XRT_RMS(float, float);
    else if (weight_dtype == XRT_F32) XRT_RMS(float, bf16);
    else if (out_dtype == XRT_F32) XRT_RMS(bf16, float);
    else XRT_RMS(bf16, bf16);
#undef XRT_RMS
    XRT_LAUNCH_CHECK("rmsnorm");
    return 0;
}
