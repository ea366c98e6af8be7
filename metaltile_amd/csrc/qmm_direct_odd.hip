// Instances of the register-operand tile kernel for the bit-stream code widths (3, 5, 6, 7 bits):
// replaces mt_qmm_mma_b3 / _b5 / _b6 (crates/metaltile-std/src/mlx/quantized.rs:3560-3900) and, grouped
// by expert, mt_moe_gather_qmm_mma_b3 / _b5 / _b6 (crates/metaltile-std/src/ffai/moe.rs:2552-2835).
// A lane's 32 codes of a 64-k slice are `bits` whole words at any width, so the kernel is the same;
// only the extraction differs (constant shifts, a code may straddle two words). Fewer tilings than the
// 2-, 4-, 8-bit set are built: 128-row tiles on 1 K-group, 64-row tiles on 2 and 4 K-groups, 32-row tiles
// on 4 K-groups, and the grouped 64-row forms.
#include "qmm_direct_impl.h"

namespace mtq {

template <int DT, int B> static const void* pick_b(uint32_t kgroups, uint32_t tile_rows, bool sbl, bool grouped, bool split) {
#define QO(MBv, KGv, GRv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, MBv, true, KGv, GRv> : (const void*)qmm_direct_kernel<DT, B, 2, MBv, false, KGv, GRv>)
    if (grouped) {
        if (tile_rows != 64) return nullptr;
        return kgroups == 4 ? QO(2, 4, true) : kgroups == 2 ? QO(2, 2, true) : nullptr;
    }
    if (split) {  // K-split instances (f32 partial tiles, no store of their own)
#define QS(MBv, KGv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, MBv, true, KGv, false, true> : (const void*)qmm_direct_kernel<DT, B, 2, MBv, false, KGv, false, true>)
        if (tile_rows == 128 && kgroups == 1) return QS(4, 1);
        if (tile_rows == 64 && kgroups == 4) return QS(2, 4);
        if (tile_rows == 32 && kgroups == 4) return QS(1, 4);
        return nullptr;
#undef QS
    }
    if (tile_rows == 128 && kgroups == 1) return QO(4, 1, false);
    if (tile_rows == 64 && kgroups == 2) return QO(2, 2, false);
    if (tile_rows == 64 && kgroups == 4) return QO(2, 4, false);
    if (tile_rows == 64 && kgroups == 1) return QO(2, 1, false);
    if (tile_rows == 32 && kgroups == 4) return QO(1, 4, false);
    return nullptr;
#undef QO
}

template <int DT> static const void* pick_dt(int bits, uint32_t kgroups, uint32_t tile_rows, bool sbl, bool grouped, bool split) {
    switch (bits) {
        case 3: return pick_b<DT, 3>(kgroups, tile_rows, sbl, grouped, split);
        case 5: return pick_b<DT, 5>(kgroups, tile_rows, sbl, grouped, split);
        case 6: return pick_b<DT, 6>(kgroups, tile_rows, sbl, grouped, split);
        case 7: return pick_b<DT, 7>(kgroups, tile_rows, sbl, grouped, split);
        default: return nullptr;
    }
}

const void* qmm_direct_pick_odd(int dtype, int bits, uint32_t kgroups, uint32_t tile_rows, bool sbl, bool grouped, bool split) {
    return dtype == DT_BF16 ? pick_dt<DT_BF16>(bits, kgroups, tile_rows, sbl, grouped, split)
         : dtype == DT_F16 ? pick_dt<DT_F16>(bits, kgroups, tile_rows, sbl, grouped, split) : nullptr;
}

}  // namespace mtq
