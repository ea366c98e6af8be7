// The 16-row matrix-core GEMV's instances for expert-routed rows (groups of 64 codes; see qmv_wide.hip): a translation
// unit of its own so that it compiles beside the plain ones.
#include "qmv_wide_impl.h"

namespace mtq {

const void* qmv_wide_gather_pick(int dtype, int mode, uint32_t nb, uint32_t sets) {
#define QWG3(DTv, MODEv, NBv) (sets == 1 ? (const void*)qmv_wide_kernel<DTv, 64, NBv, 1, MODEv> : sets == 2 ? (const void*)qmv_wide_kernel<DTv, 64, NBv, 2, MODEv> \
                               : NBv == 1 ? (const void*)qmv_wide_kernel<DTv, 64, 1, 3, MODEv> : nullptr)
#define QWG2(DTv, MODEv) (nb == 2 ? QWG3(DTv, MODEv, 2) : QWG3(DTv, MODEv, 1))
#define QWG(DTv) (mode == GATHER_CSR ? QWG2(DTv, GATHER_CSR) : QWG2(DTv, GATHER_INDICES))
    return dtype == DT_BF16 ? QWG(DT_BF16) : dtype == DT_F16 ? QWG(DT_F16) : nullptr;
#undef QWG
#undef QWG2
#undef QWG3
}

}  // namespace mtq
