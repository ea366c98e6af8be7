// Host side of the GEMV kernel for two to four activation rows (qmv_rows_few_impl.h): which shapes it takes, its launch.
#include <hip/hip_runtime.h>

#include "../../include/mtq.h"
#include "mtq_device.h"
#include "mtq_internal.h"
#include "qmv_rows_few_impl.h"

namespace mtq {

// chunks per lane and row of the instance that takes the shape, or 0
static int rows_few_t(const QmvParams& p) {
    if (p.bits != 2 && p.bits != 4) return 0;
    const uint32_t G = p.group_size;
    if (G != 32 && G != 64 && G != 128) return 0;
    if (p.bits == 4) return p.K == 4096 ? 8 : p.K == 8192 ? 16 : 0;
    return p.K == 8192 ? 8 : 0;   // (16384 2-bit codes: four rows of activations in operand order no longer fit in LDS)
}

bool qmv_rows_few_takes(const QmvParams& p) {
    if (p.gather != GATHER_NONE || p.M < 2 || p.M > 4 || (p.dtype != DT_F16 && p.dtype != DT_BF16) || p.N == 0) return false;
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16 || (uintptr_t)p.out % 2) return false;
    return rows_few_t(p) != 0;
}

// Where this kernel is ahead of the matrix-core GEMV that served these shapes before (same run, f16, 8192 x 8192, us,
// four / two rows of x): 2-bit g32 13.4 -> 9.3 / 12.0 -> 8.5, g64 11.5 -> 8.6 / 10.3 -> 7.8, g128 10.2 -> 8.4 / 8.6 -> 7.6;
// 4-bit g32 13.8 -> 12.0 / 12.5 -> 11.0, g64 11.4 -> 11.1 / 10.3 -> 10.4, g128 11.2 -> 10.8 / 10.0 -> 10.1. Behind: fewer
// weight rows (a workgroup is 32 rows and fills a compute unit: 4096 x 8192 8.2 -> 9.7, 2048 x 8192 7.4 -> 9.2) and
// rows of 4096 codes (14336 x 4096 10.4 -> 10.9); those stay where they were.
bool qmv_rows_few_preferred(const QmvParams& p) {
    if (!qmv_rows_few_takes(p) || p.N < 8192 || p.K != 8192) return false;
    return p.bits == 2 || p.group_size == 32 || p.M >= 3;
}

template <int DT, int LOG2G> static const void* rows_few_fn_g(int bits, int t, size_t* lds) {
    if (bits == 4 && t == 8) { *lds = RowsFewGeom<4, 8, LOG2G>::TOTAL; return (const void*)qmv_rows_few_kernel<DT, 4, 8, LOG2G>; }
    if (bits == 4 && t == 16) { *lds = RowsFewGeom<4, 16, LOG2G>::TOTAL; return (const void*)qmv_rows_few_kernel<DT, 4, 16, LOG2G>; }
    if (bits == 2 && t == 8) { *lds = RowsFewGeom<2, 8, LOG2G>::TOTAL; return (const void*)qmv_rows_few_kernel<DT, 2, 8, LOG2G>; }
    return nullptr;
}
template <int DT> static const void* rows_few_fn(int bits, int t, uint32_t G, size_t* lds) {
    return G == 32 ? rows_few_fn_g<DT, 5>(bits, t, lds) : G == 64 ? rows_few_fn_g<DT, 6>(bits, t, lds) : rows_few_fn_g<DT, 7>(bits, t, lds);
}

int launch_qmv_rows_few(const QmvParams& p, const LaunchCtx& lc) {
    if (!qmv_rows_few_takes(p))
        return fail(ERR_UNSUPPORTED, "qmv few-rows kernel: 2..4 activation rows, f16 / bf16, 4096 or 8192 4-bit codes or 8192 2-bit codes per row");
    const int t = rows_few_t(p);
    size_t lds = 0;
    const void* fn = p.dtype == DT_BF16 ? rows_few_fn<DT_BF16>(p.bits, t, p.group_size, &lds) : rows_few_fn<DT_F16>(p.bits, t, p.group_size, &lds);
    if (!fn) return fail(ERR_UNSUPPORTED, "qmv few-rows kernel: no instance for this row length and group size");
    hipError_t e = set_max_dynamic_lds(fn, lds);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    QmvRowsFArgs a{(const rp_u32x4*)p.w, (const uint16_t*)p.scales, (const uint16_t*)p.biases, (const uint16_t*)p.x, (uint16_t*)p.out, p.N, p.M, nullptr};
    void* args[] = {&a};
    e = launch_kernel(fn, dim3((p.N + 31u) / 32u), dim3(1024), args, lds, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv few-rows kernel launch");
    return ERR_OK;
}

}  // namespace mtq
