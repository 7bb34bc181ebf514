// Where a key or a value lies inside its cache block.
//
// A block holds XRT_BLOCK_TOKENS (64) keys and values of one key/value head: 64 * head_dim elements each.
// Decode attention is bound by reading them, and it reads fastest when every load instruction of a
// wavefront takes one contiguous kilobyte that nobody else reads (such loads can pass the caches by).
// So, when head_dim is a multiple of 32, a block lies in the order in which the wavefront of the decode
// kernel holds it: in tiles of 64 pieces, a piece being 8 elements that one lane feeds to the matrix
// cores (v_mfma_f32_16x16x32: lane (r, c), r = lane % 16, c = lane / 16, holds row r, columns 8c .. 8c + 7
// of a 16 x 32 operand), piece (r, c) at place r + 16 c of its tile.
//   keys:   a piece is 8 consecutive dims of one key. Tile ((g * 2 + t) * head_dim / 32 + s) holds dims
//           32 s .. 32 s + 31 of the 16 keys 32 g + 8 (r / 4) + 4 t + r % 4: the keys of a score tile are
//           picked so that, after the product, a lane holds the scores of eight consecutive keys, which is
//           the operand of the product with the values.
//   values: a piece is 8 consecutive tokens of one dim (values are kept transposed). Tile
//           (g * head_dim / 16 + u) holds tokens 32 g .. 32 g + 31 of dims 16 u .. 16 u + 15.
// Other head sizes keep the plain order: keys [token][dim], values [dim][token].
// Every kernel that writes or reads the cache goes through the two functions below; pieces stay whole,
// so 8 (4, 2) elements from a multiple of 8 (4, 2) are contiguous in either order.
#pragma once
#include "common.h"

__host__ __device__ constexpr bool cache_in_tiles(int head_dim) { return head_dim % 32 == 0; }

// element offset, within the block of one key/value head, of dim `dim` of the key of token `token` (0 .. 63)
__host__ __device__ constexpr int cache_key_offset(int token, int dim, int head_dim) {
    if (!cache_in_tiles(head_dim)) return token * head_dim + dim;
    const int within = token % 32;
    const int tile = ((token / 32) * 2 + within % 8 / 4) * (head_dim / 32) + dim / 32;
    const int place = within / 8 * 4 + within % 4 + 16 * (dim % 32 / 8);
    return (tile * 64 + place) * 8 + dim % 8;
}

// the same of dim `dim` of the value of token `token`
__host__ __device__ constexpr int cache_value_offset(int dim, int token, int head_dim) {
    if (!cache_in_tiles(head_dim)) return dim * XRT_BLOCK_TOKENS + token;
    const int tile = (token / 32) * (head_dim / 16) + dim / 16;
    const int place = dim % 16 + 16 * (token % 32 / 8);
    return (tile * 64 + place) * 8 + token % 8;
}
