// Instantiates the matrix-core qmv kernel family for element dtype bf16 (see qmv_mfma_impl.h).
#include "qmv_mfma_impl.h"

namespace mtq {
template int qmv_mfma_launch_dtype<DT_BF16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);
}
