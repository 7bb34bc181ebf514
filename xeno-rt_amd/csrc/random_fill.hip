// Random weights on the device: element i of a tensor's stream, as the host-side generator of the
// random-weights mode makes it (weights/random_init.py), bit for bit.
//   words:  mix(key + 2i*G), mix(key + (2i+1)*G)   (mix: one splitmix64 step, G its increment)
//   sum:    twelve 10-bit fields, six of each word
//   value:  float(2*sum - 12*1023) * scale + offset, rounded to the stored type to nearest even
// Integer arithmetic and one float32 multiplication (and one addition): nothing that two machines round differently.
#include "common.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ unsigned long long mix(unsigned long long v) {
    v += 0x9E3779B97F4A7C15ull;
    v = (v ^ (v >> 30)) * 0xBF58476D1CE4E5B9ull;
    v = (v ^ (v >> 27)) * 0x94D049BB133111EBull;
    return v ^ (v >> 31);
}

__device__ __forceinline__ int fields(unsigned long long word) {
    int sum = 0;
#pragma unroll
    for (int f = 0; f < 6; ++f) sum += (int)((word >> (10 * f)) & 1023ull);
    return sum;
}

template <typename T>
__global__ void __launch_bounds__(256) random_normal_kernel(T* __restrict__ out, long count, unsigned long long key,
                                                             float scale, float offset) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const unsigned long long base = key + (unsigned long long)(2 * i) * 0x9E3779B97F4A7C15ull;
        const int sum = fields(mix(base)) + fields(mix(base + 0x9E3779B97F4A7C15ull));
        const float centred = (float)(2 * sum - 12 * 1023);
        float value, product;
        {
#pragma clang fp contract(off)                              // two roundings, as on the host: never one fused operation
            product = centred * scale;
            value = product + offset;
        }
        if (offset == 0.f) value = product;
        out[i] = from_float<T>(value);
    }
}

}  // namespace

extern "C" int xrt_random_normal(void* out, int dtype, long count, unsigned long long key, float scale, float offset,
                                 void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "random_normal: unknown dtype %d", dtype);
    XRT_REQUIRE(count >= 0 && out != nullptr, "random_normal: bad operands");
    if (count == 0) return 0;
    const long blocks_wanted = (count + 255) / 256;
    const unsigned blocks = (unsigned)(blocks_wanted < 16384 ? blocks_wanted : 16384);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == XRT_F32) random_normal_kernel<float><<<blocks, 256, 0, s>>>((float*)out, count, key, scale, offset);
    else random_normal_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, count, key, scale, offset);
    XRT_LAUNCH_CHECK("random_normal");
    return 0;
}
