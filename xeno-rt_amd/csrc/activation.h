// The activation of a gated product, out = act(a . w_gate) * (a . w_up): one code, one formula, here.
// A product's mode carries the code in its bits from 8 up (mode 2 alone is the gated product with SiLU).
// Another activation is another code and another case below; every kernel with a gated epilogue
// takes the code as an argument and calls gate_activation.
#pragma once
#include "common.h"

#include "xrt_hip.h"

enum { XRT_ACT_COUNT = 1 };          // codes XRT_ACT_* of xrt_hip.h below this are known

inline int mode_of(int mode) { return mode & 255; }
inline int activation_of(int mode) { return mode >> 8; }

// QUICK: the exponential and the division by the hardware's own instructions (a few units in the last place of a
// float32), for results that are rounded to bfloat16 anyway: five instructions where the exact ones take some thirty,
// which a tile of a prefill's gate/up product pays 64 times a lane.
template <bool QUICK = false>
__device__ __forceinline__ float gate_activation(float z, int activation) {
    switch (activation) {
        case XRT_ACT_SILU:
        default:                                    // silu(z) = z / (1 + exp(-z)): crates/xrt-kernels/src/cpu/silu.rs:1-3 of the reference
            if constexpr (QUICK) return z * __frcp_rn(1.0f + __expf(-z));
            else return z / (1.0f + expf(-z));
    }
}
