// The load-to-LDS tile kernel's instances for 8-bit codes (see qmm_dma.hip; replaces mt_qmm_mma_int8 and its _m16 form,
// crates/metaltile-std/src/mlx/quantized.rs:2731, 2990): a translation unit of its own so that it compiles beside the
// 4-bit one.
#include "qmm_dma_picks.h"

namespace mtq {

const void* qmm_dma_pick_b8(int dtype, uint32_t rows, bool grouped, bool windowed, bool shallow) {
    return qmm_dma_pick_t<8>(dtype, rows, grouped, windowed, shallow);
}
const void* qmm_dma_split_pick_b8(int dtype, uint32_t rows) { return qmm_dma_split_pick_t<8>(dtype, rows); }
const void* qmm_dma4_pick_b8(int dtype, uint32_t rows, bool split, bool grouped) { return qmm_dma4_pick_t<8>(dtype, rows, split, grouped); }

}  // namespace mtq
