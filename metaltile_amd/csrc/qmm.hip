// placeholder, replaced below
#include "mtq_internal.h"
namespace mtq {
int launch_qmm_mfma(const QmmParams&, const LaunchCtx&) { return fail(ERR_UNSUPPORTED, "qmm mfma not built"); }
}
