// Weight matrices in tiles, for products that are bound by reading w.
//
// A matrix w[rows][K] (bfloat16) may be kept "packed": in tiles of 16 rows x 32 columns, 1 KB each, the
// tiles of a group of 16 rows one after another along k, groups one after another. Inside a tile the 16-byte
// pieces (8 columns of one row) lie in the order in which the lanes of a wavefront hold the A operand of
// v_mfma_f32_16x16x32_bf16: piece (row r, columns 8c .. 8c + 7) at place r + 16 c. One load instruction of
// a wavefront then reads a whole contiguous tile, and any eight rows of one quarter are one cache line.
// Rows beyond the matrix (it is padded to a multiple of 16) hold zeros.
//
// The rows may also stand in another order than the outputs they make, so that outputs which an epilogue
// combines lie in one tile:
//   XRT_PACK_TILES   packed row p is row p of w;
//   XRT_PACK_GATED   w is [gate rows 0 .. n-1 | up rows n .. 2n-1] (n a multiple of 8): a group of 16 packed
//                    rows holds gate rows 8g .. 8g + 7, then the up rows of the same outputs;
//   XRT_PACK_ROTARY  w is [heads][head_dim] rows; in each of the first `rotated_heads` heads a group of 16
//                    holds dims 8s .. 8s + 7, then dims head_dim / 2 + 8s .. + 7: the pairs of a rotation
//                    over the whole head. The other heads keep their order.
#pragma once
#include "common.h"
#include "xrt_hip.h"

typedef xrt_packing Packing;

__host__ __device__ inline bool is_packed(const Packing& p) { return p.kind != XRT_PACK_NONE; }

// the row of w (in the order of the outputs) that packed row `r` holds
__host__ __device__ inline long logical_row(const Packing& p, long r) {
    if (p.kind == XRT_PACK_GATED) {
        const long group = r / 16, within = r % 16;
        return within < 8 ? group * 8 + within : (long)p.gated_n + group * 8 + (within - 8);
    }
    if (p.kind == XRT_PACK_ROTARY) {
        const long head = r / p.head_dim, within = r % p.head_dim;
        if (head >= p.rotated_heads) return r;
        const long s = within / 16, half = within % 16 / 8, j = within % 8;
        return head * p.head_dim + half * (p.head_dim / 2) + s * 8 + j;
    }
    return r;
}

// the packed row that holds row `l` of w
__host__ __device__ inline long packed_row(const Packing& p, long l) {
    if (p.kind == XRT_PACK_GATED) {
        const bool up = l >= p.gated_n;
        const long j = up ? l - p.gated_n : l;
        return j / 8 * 16 + (up ? 8 : 0) + j % 8;
    }
    if (p.kind == XRT_PACK_ROTARY) {
        const long head = l / p.head_dim, d = l % p.head_dim;
        if (head >= p.rotated_heads) return l;
        const long half = d / (p.head_dim / 2), within = d % (p.head_dim / 2);
        return head * p.head_dim + within / 8 * 16 + half * 8 + within % 8;
    }
    return l;
}

// element offset of the 8 columns from k (a multiple of 8) of packed row r; K a multiple of 32
__host__ __device__ inline long packed_offset(long r, int k, int K) {
    return ((r / 16) * (long)(K / 32) + k / 32) * 512 + ((k % 32 / 8) * 16 + r % 16) * 8;
}

// element offset of the 8 columns from k of the row of w that makes output row `l`, in either form
__host__ __device__ inline long weight_offset(const Packing& p, long l, int k, int K) {
    return is_packed(p) ? packed_offset(packed_row(p, l), k, K) : l * K + k;
}
