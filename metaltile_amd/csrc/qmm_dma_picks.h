// The instances of the load-to-LDS tile kernel by tiling, as templates over the code width, so that each width is
// built in a translation unit of its own (qmm_dma.hip: 4 bits, qmm_dma_b8.hip: 8 bits).
#pragma once
#include "qmm_dma_impl.h"

namespace mtq {

template <int BITS> const void* qmm_dma_pick_t(int dtype, uint32_t rows, bool grouped, bool windowed, bool shallow) {
    if (!grouped && rows == 64 && !shallow) {
        if (windowed)
            return dtype == DT_BF16 ? (const void*)qmm_dma_kernel<DT_BF16, 2, 2, 8, 0, false, false, true, BITS>
                 : dtype == DT_F16 ? (const void*)qmm_dma_kernel<DT_F16, 2, 2, 8, 0, false, false, true, BITS> : nullptr;
        return dtype == DT_BF16 ? (const void*)qmm_dma_kernel<DT_BF16, 2, 2, 8, 0, false, false, false, BITS> : dtype == DT_F16 ? (const void*)qmm_dma_kernel<DT_F16, 2, 2, 8, 0, false, false, false, BITS> : nullptr;
    }
    if (grouped) {  // rows routed to experts: 64-row tiles cut from each expert's rows
        if (rows != 64) return nullptr;
        if (windowed)
            return dtype == DT_BF16 ? (const void*)qmm_dma_kernel<DT_BF16, 2, 2, 8, 2, true, false, true, BITS>
                 : dtype == DT_F16 ? (const void*)qmm_dma_kernel<DT_F16, 2, 2, 8, 2, true, false, true, BITS> : nullptr;
        return dtype == DT_BF16 ? (const void*)qmm_dma_kernel<DT_BF16, 2, 2, 8, 2, true, false, false, BITS>
             : dtype == DT_F16 ? (const void*)qmm_dma_kernel<DT_F16, 2, 2, 8, 2, true, false, false, BITS> : nullptr;
    }
    if (windowed) {
#define QDMAW(DTv) (rows == 64 ? (const void*)qmm_dma_kernel<DTv, 2, 2, 8, 2, false, false, true, BITS>                                \
                    : rows == 128 ? (const void*)qmm_dma_kernel<DTv, 4, 2, 8, 0, false, false, true, BITS>                              \
                    : rows == 256 && BITS == 4 ? (const void*)qmm_dma_kernel<DTv, 8, 2, 8, 0, false, false, true, 4> : nullptr)
        return dtype == DT_BF16 ? QDMAW(DT_BF16) : dtype == DT_F16 ? QDMAW(DT_F16) : nullptr;
#undef QDMAW
    }
#define QDMA(DTv) (rows == 64 ? (const void*)qmm_dma_kernel<DTv, 2, 2, 8, 2, false, false, false, BITS> : rows == 128 ? (const void*)qmm_dma_kernel<DTv, 4, 2, 8, 0, false, false, false, BITS> \
                   : rows == 256 ? (const void*)qmm_dma_kernel<DTv, 8, 2, 8, 0, false, false, false, BITS> : nullptr)
    return dtype == DT_BF16 ? QDMA(DT_BF16) : dtype == DT_F16 ? QDMA(DT_F16) : nullptr;
#undef QDMA
}


// K-split instances of the 64 x 128 and 128 x 128 tiles (f32 partial tiles, a ring of three, whole groups of the split's
// share of the rows in LDS)
template <int BITS> const void* qmm_dma_split_pick_t(int dtype, uint32_t rows) {
    if (rows != 64 && rows != 128) return nullptr;
    if (dtype == DT_BF16) return rows == 64 ? (const void*)qmm_dma_kernel<DT_BF16, 2, 2, 8, 0, false, true, false, BITS> : (const void*)qmm_dma_kernel<DT_BF16, 4, 2, 8, 0, false, true, false, BITS>;
    if (dtype == DT_F16) return rows == 64 ? (const void*)qmm_dma_kernel<DT_F16, 2, 2, 8, 0, false, true, false, BITS> : (const void*)qmm_dma_kernel<DT_F16, 4, 2, 8, 0, false, true, false, BITS>;
    return nullptr;
}

template <int BITS> const void* qmm_dma4_pick_t(int dtype, uint32_t rows, bool split, bool grouped) {
    if (grouped) {
        if (split || (rows != 32 && rows != 64)) return nullptr;
        if (dtype == DT_BF16) return rows == 32 ? (const void*)qmm_dma_kernel<DT_BF16, 1, 4, 8, 0, true, false, false, BITS> : (const void*)qmm_dma_kernel<DT_BF16, 2, 4, 8, 0, true, false, false, BITS>;
        if (dtype == DT_F16) return rows == 32 ? (const void*)qmm_dma_kernel<DT_F16, 1, 4, 8, 0, true, false, false, BITS> : (const void*)qmm_dma_kernel<DT_F16, 2, 4, 8, 0, true, false, false, BITS>;
        return nullptr;
    }
#define QDMA4(DTv) (split ? (rows == 32 ? (const void*)qmm_dma_kernel<DTv, 1, 4, 8, 0, false, true, false, BITS> : (const void*)qmm_dma_kernel<DTv, 2, 4, 8, 0, false, true, false, BITS>) \
                          : (rows == 32 ? (const void*)qmm_dma_kernel<DTv, 1, 4, 8, 0, false, false, false, BITS> : (const void*)qmm_dma_kernel<DTv, 2, 4, 8, 0, false, false, false, BITS>))
    if (rows != 32 && rows != 64) return nullptr;
    return dtype == DT_BF16 ? QDMA4(DT_BF16) : dtype == DT_F16 ? QDMA4(DT_F16) : nullptr;
#undef QDMA4
}


}  // namespace mtq
