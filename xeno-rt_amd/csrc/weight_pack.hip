// Packs a weight matrix into the tiled layout of packing.h.
#include "packing.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// one thread per 16-byte piece of the packed matrix
__global__ void __launch_bounds__(256) pack_weight_kernel(const bf16* __restrict__ w, bf16* __restrict__ packed, int rows,
                                                          long padded_rows, int K, const Packing packing) {
    const long pieces = padded_rows * (K / 8);
    for (long piece = (long)blockIdx.x * blockDim.x + threadIdx.x; piece < pieces; piece += (long)gridDim.x * blockDim.x) {
        // pieces in the order of the packed matrix, so that the stores are contiguous
        const long tile = piece / 64;
        const int place = (int)(piece % 64);
        const long group = tile / (K / 32);
        const int k = (int)(tile % (K / 32)) * 32 + place / 16 * 8;
        const long row = logical_row(packing, group * 16 + place % 16);
        bf16x8 value = {};
        if (row < rows) value = *reinterpret_cast<const bf16x8*>(w + row * K + k);
        *reinterpret_cast<bf16x8*>(packed + piece * 8) = value;
    }
}

}  // namespace

extern "C" int xrt_pack_weight(const void* w, void* packed, int rows, int K, const xrt_packing* packing, void* stream) {
    XRT_REQUIRE(w && packed && packing, "pack_weight: null operand");
    XRT_REQUIRE(rows > 0 && K > 0 && K % 32 == 0, "pack_weight: K = %d must be a positive multiple of 32", K);
    XRT_REQUIRE((uintptr_t)w % 16 == 0 && (uintptr_t)packed % 16 == 0, "pack_weight: operands must be aligned to 16 bytes");
    XRT_REQUIRE(packing->kind == XRT_PACK_TILES || packing->kind == XRT_PACK_GATED || packing->kind == XRT_PACK_ROTARY,
                "pack_weight: unknown packing %d", packing->kind);
    if (packing->kind == XRT_PACK_GATED)
        XRT_REQUIRE(packing->gated_n > 0 && packing->gated_n % 8 == 0 && rows == 2 * packing->gated_n,
                    "pack_weight: gate/up pairs need 2 x %d rows with that a multiple of 8, found %d rows", packing->gated_n, rows);
    if (packing->kind == XRT_PACK_ROTARY)
        XRT_REQUIRE(packing->head_dim > 0 && packing->head_dim % 16 == 0 && rows % packing->head_dim == 0 &&
                        packing->rotated_heads >= 0 && packing->rotated_heads <= rows / packing->head_dim,
                    "pack_weight: rotary pairs need rows = heads x head_dim (a multiple of 16), found %d rows of heads of %d",
                    rows, packing->head_dim);
    const long padded = ((long)rows + 15) / 16 * 16;
    const long pieces = padded * (K / 8);
    const unsigned blocks = (unsigned)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
    pack_weight_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const bf16*)w, (bf16*)packed, rows, padded, K, *packing);
    XRT_LAUNCH_CHECK("pack_weight");
    return 0;
}

// A product that streams w takes as long as the compute unit with the most rows of it. Packed, w is dealt
// out in groups of 16 rows, which stream about 1.35 times as fast as rows contiguous along k; those can be
// dealt out in tiles of 8 to 16 rows that divide evenly among the 256 compute units. So packing pays where
// the fullest compute unit gets less than 1.35 times its share of the groups. Matrices of few groups are
// bound by other things; they are packed too, so that small models meet the same kernels as large ones.
extern "C" int xrt_packing_suits(int rows, int K) {
    if (rows <= 0 || K <= 0 || K % 32 != 0) return 0;
    const long groups = ((long)rows + 15) / 16;
    const long rounds = (groups + XRT_COMPUTE_UNITS - 1) / XRT_COMPUTE_UNITS;
    return groups <= 64 || rounds * XRT_COMPUTE_UNITS * 100 <= groups * 135;
}
