// Two probes of the machine, for the benchmark's "measured ceiling" columns: how fast a kernel that does
// nothing else reads device memory, and how fast the matrix cores multiply tiles that never leave the
// registers. Nothing of the model runs through them.
#include "common.h"
#include "xrt_hip.h"

namespace {

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Every workgroup owns a contiguous slice; a wavefront reads 1 KB per instruction, eight instructions in flight.
template <bool NONTEMPORAL>
__global__ void __launch_bounds__(256) probe_read_kernel(const uint4v* __restrict__ p, long per_group, unsigned* sink) {
    const uint4v* base = p + (long)blockIdx.x * per_group;
    const int wave = threadIdx.x / XRT_WAVE, lane = threadIdx.x % XRT_WAVE;
    unsigned acc = 0;
    for (long i = (long)wave * XRT_WAVE * 8; i + XRT_WAVE * 8 <= per_group; i += 4L * XRT_WAVE * 8) {
        uint4v v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            v[u] = NONTEMPORAL ? __builtin_nontemporal_load(base + i + u * XRT_WAVE + lane) : base[i + u * XRT_WAVE + lane];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].w;
    }
    if (acc == 0x12345678u) sink[0] = acc;          // never true for the probe's buffer of ones: keeps the loads alive
}

// Four independent chains of 32x32x16 products per wavefront, operands and sums in registers.
// The operands are small whole numbers, or (random_operands) numbers of either sign in [1, 2) with random mantissas:
// the matrix cores draw more power on those, and the clock that the chip then holds is lower.
__global__ void __launch_bounds__(256) probe_mfma_kernel(long iterations, int random_operands, float* sink) {
    bf16x8 a, b;
    unsigned state = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (bf16)(float)((threadIdx.x + e) % 3);
        b[e] = (bf16)(float)((threadIdx.x + 2 * e) % 5);
        if (random_operands) {
            state = state * 1664525u + 1013904223u;
            a[e] = __builtin_bit_cast(bf16, (unsigned short)(((state >> 16) & 0x807fu) | 0x3f80u));
            b[e] = __builtin_bit_cast(bf16, (unsigned short)((state & 0x807fu) | 0x3f80u));
        }
    }
    floatx16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
    for (long it = 0; it < iterations; ++it) {
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) total += acc[c][0] + acc[c][15];
    if (total == -1.5f && iterations < 0) sink[0] = total;             // never true
}

}  // namespace

extern "C" int xrt_probe_read(const void* buffer, long bytes, int nontemporal, void* sink, void* stream) {
    XRT_REQUIRE(buffer && sink && bytes > 0 && (uintptr_t)buffer % 16 == 0, "probe_read: bad operands");
    const int groups = 2048;
    const long per_group = bytes / 16 / groups / (4L * XRT_WAVE * 8) * (4L * XRT_WAVE * 8);    // 16-byte words, whole rounds
    XRT_REQUIRE(per_group > 0, "probe_read: %ld bytes are too few for %d workgroups", bytes, groups);
    hipStream_t s = (hipStream_t)stream;
    if (nontemporal) probe_read_kernel<true><<<groups, 256, 0, s>>>((const uint4v*)buffer, per_group, (unsigned*)sink);
    else probe_read_kernel<false><<<groups, 256, 0, s>>>((const uint4v*)buffer, per_group, (unsigned*)sink);
    XRT_LAUNCH_CHECK("probe_read");
    return 0;
}

extern "C" long xrt_probe_read_bytes(long bytes) {
    const long per_group = bytes / 16 / 2048 / (4L * XRT_WAVE * 8) * (4L * XRT_WAVE * 8);
    return per_group * 16 * 2048;
}

extern "C" int xrt_probe_mfma(long iterations, int random_operands, void* sink, void* stream) {
    XRT_REQUIRE(sink && iterations > 0, "probe_mfma: bad operands");
    probe_mfma_kernel<<<XRT_PROBE_MFMA_GROUPS, 256, 0, (hipStream_t)stream>>>(iterations, random_operands, (float*)sink);
    XRT_LAUNCH_CHECK("probe_mfma");
    return 0;
}
