// Shared device and host helpers of the kernel library (gfx950, 64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16;

// element type codes of the C interface
enum { XRT_F32 = 0, XRT_BF16 = 1 };

// tokens per cache block; keys are [kv_head][token][dim], values [kv_head][dim][token] inside a block
#define XRT_BLOCK_TOKENS 64
#define XRT_WAVE 64
// compute units of the chip: what the launchers count in when they deal work out in rounds
#define XRT_COMPUTE_UNITS 256

// ---- error reporting -------------------------------------------------------
void xrt_set_error(const char* format, ...);

#define XRT_REQUIRE(condition, ...)            \
    do {                                       \
        if (!(condition)) {                    \
            xrt_set_error(__VA_ARGS__);        \
            return 1;                          \
        }                                      \
    } while (0)

#define XRT_LAUNCH_CHECK(name)                                                      \
    do {                                                                            \
        hipError_t launch_error_ = hipGetLastError();                               \
        if (launch_error_ != hipSuccess) {                                          \
            xrt_set_error("%s: launch failed: %s", name, hipGetErrorString(launch_error_)); \
            return 1;                                                               \
        }                                                                           \
    } while (0)

// ---- conversions -----------------------------------------------------------
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return (bf16)v; }   // round to nearest even

// The value that the lane 8 places away in this lane's row of 16 lanes holds (lane ^ 8): one instruction of the vector
// unit (a rotation of the row by half), where a shuffle goes through the LDS hardware.
__device__ __forceinline__ float from_eight_lanes_away(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
}

// ---- wave reductions (fixed butterfly order: results do not depend on the launch) ----
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, XRT_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = XRT_WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, XRT_WAVE));
    return v;
}

// Orders the LDS accesses of the lanes of one wavefront: what any lane wrote before is
// seen by every lane after. (A wavefront's LDS operations execute in order; the fences keep
// the compiler from moving accesses across.)
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// sum over a block of up to 1024 threads; every thread gets the result. `scratch` holds 32 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int waves = (blockDim.x + XRT_WAVE - 1) / XRT_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}
// ---- the cache ---------------------------------------------------------------------------
// Element offset of the cache block that holds `pos` of sequence `slot`, for one key/value head;
// -1 if there is none (padding, or a table entry that names no block).
__device__ __forceinline__ long cache_block_base(const int* block_table, int table_stride, int n_blocks, int slot,
                                                 int pos, int n_kv_heads, int kv_head, int head_dim) {
    if (slot < 0) return -1;
    const int block = block_table[(long)slot * table_stride + pos / XRT_BLOCK_TOKENS];
    if (block < 0 || block >= n_blocks) return -1;
    return ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
}

// ---- global memory -> LDS without passing registers (gfx950) ----------------------------------
// 16 bytes per lane from global memory into LDS without passing registers: lane l of the
// wavefront writes LDS byte address lds_base + 16 * l (lds_base is the same for the whole
// wavefront and travels in M0) with the 16 bytes at base + byte_offset (of that lane). Written
// as assembly so that the waits for these loads are the explicit ones in the kernel: the
// compiler, when it knows of such a load, waits for all of them at every barrier.
__device__ __forceinline__ void load_to_lds(const void* base, unsigned byte_offset, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(byte_offset), "s"(base) : "memory", "m0");
}
// The same with 4 bytes per lane: lane l writes LDS byte address lds_base + 4 * l.
__device__ __forceinline__ void load_dword_to_lds(const void* base, unsigned byte_offset, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(byte_offset), "s"(base) : "memory", "m0");
}
// Waits until at most `pending` of this wavefront's loads (the newest ones) are outstanding and
// its LDS reads are done, then meets the workgroup's other wavefronts. __syncthreads() cannot
// stand here: its release fence waits for every load, also those meant to stay in flight.
template <int pending>
__device__ __forceinline__ void wait_loads_and_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(pending) : "memory");
}
__device__ __forceinline__ unsigned lds_address(const void* p) {
    return (unsigned)(unsigned long)(const __attribute__((address_space(3))) void*)p;
}


