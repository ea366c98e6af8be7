// Instantiates the matrix-core qmv kernel family for element dtype bf16, code widths 3, 5 and 6
// (see qmv_mfma_impl.h).
#include "qmv_mfma_impl.h"

namespace mtq {
template int qmv_mfma_launch_dtype_odd<DT_BF16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);
}
