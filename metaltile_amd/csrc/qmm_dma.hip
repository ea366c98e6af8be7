// Instances of the tile kernel whose activation tile is brought in by load-to-LDS instructions (4-bit codes here, 8-bit
// ones in qmm_dma_b8.hip;
// f16 / bf16, 2 K-groups x 4 column waves): replaces the same reference kernels as qmm_direct.hip (mt_qmm_mma and
// its _m16 form, crates/metaltile-std/src/mlx/quantized.rs:2106-2405, 2408) with the same arithmetic, on 64 x 128,
// 128 x 128 and 256 x 128 tiles. A translation unit of its own so that it compiles beside qmm_direct.hip.
#include "qmm_dma_picks.h"

namespace mtq {

// LDS of one workgroup: the ring of tiles and the scales / biases window, or the epilogue's partial sums and
// element tile (at most 128 rows at a time).
size_t qmm_dma_lds_bytes(uint32_t rows, uint32_t gpr, bool windowed, bool shallow) {
    // `shallow`: 64-row tiles with a ring of two, so that two workgroups share a compute unit (64 KB each at 64
    // groups per row): for launches of more tiles than compute units, where one workgroup's prologue and epilogue
    // then run beside the other's loop (8 x 14336 x 4096 grouped by expert, 100 rows each: 199 -> 187 us; one
    // round of tiles is faster on the ring of three: 4096 x 4096, 512 rows 24.9 against 26.3 us)
    const uint32_t mb = rows / 32, nbuf = (mb == 8 || (mb == 2 && shallow)) ? 2 : 3, dbn = 128, kg = 2;
    // scales and biases: the tile's whole rows, or two windows of 32 groups
    const size_t sb = windowed ? 32768 : (size_t)2 * dbn * (gpr + (nbuf != 3 ? 0 : 2)) * 2;
    const size_t main_loop = (size_t)nbuf * mb * kg * 4096 + sb;
    const uint32_t epb = mb == 8 ? 4 : mb;
    const size_t epilogue = (size_t)(kg - 1) * 4 * epb * 16 * 64 * 4 + (size_t)epb * 32 * dbn * 2;
    return main_loop > epilogue ? main_loop : epilogue;
}

const void* qmm_dma_pick_b8(int dtype, uint32_t rows, bool grouped, bool windowed, bool shallow);
const void* qmm_dma_split_pick_b8(int dtype, uint32_t rows);
const void* qmm_dma4_pick_b8(int dtype, uint32_t rows, bool split, bool grouped);

const void* qmm_dma_pick(int bits, int dtype, uint32_t rows, bool grouped, bool windowed, bool shallow) {
    return bits == 8 ? qmm_dma_pick_b8(dtype, rows, grouped, windowed, shallow) : qmm_dma_pick_t<4>(dtype, rows, grouped, windowed, shallow);
}

// K-split instances on 2 K-groups: `groups` = the most groups of scales one split's share of a row spans (whole
// 8-group vectors, or whole dwords where a row is not whole vectors)
size_t qmm_dma_split_lds_bytes(uint32_t rows, uint32_t groups) {
    const uint32_t mb = rows / 32, dbn = 128, kg = 2;
    const size_t main_loop = (size_t)3 * mb * kg * 4096 + (size_t)2 * dbn * (((groups + 3) & ~3u) + 2) * 2;
    const size_t epilogue = (size_t)(kg - 1) * 4 * mb * 16 * 64 * 4;
    return main_loop > epilogue ? main_loop : epilogue;
}

const void* qmm_dma_split_pick(int bits, int dtype, uint32_t rows) {
    return bits == 8 ? qmm_dma_split_pick_b8(dtype, rows) : qmm_dma_split_pick_t<4>(dtype, rows);
}

// 4 K-groups x 2 column waves (32 x 64 and 64 x 64 tiles, 256 k per iteration): the tilings of few rows, also as
// K-split instances that write f32 partial tiles.
size_t qmm_dma4_lds_bytes(uint32_t rows, uint32_t gpr) {
    const uint32_t mb = rows / 32, dbn = 64, kg = 4;
    const size_t main_loop = (size_t)3 * mb * kg * 4096 + (size_t)2 * dbn * (gpr + 2) * 2;
    const size_t epilogue = (size_t)(kg - 1) * 2 * mb * 16 * 64 * 4 + (size_t)mb * 32 * dbn * 2;
    return main_loop > epilogue ? main_loop : epilogue;
}

const void* qmm_dma4_pick(int bits, int dtype, uint32_t rows, bool split, bool grouped) {
    return bits == 8 ? qmm_dma4_pick_b8(dtype, rows, split, grouped) : qmm_dma4_pick_t<4>(dtype, rows, split, grouped);
}

}  // namespace mtq
