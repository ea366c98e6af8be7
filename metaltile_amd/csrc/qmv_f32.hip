// Instantiates the qmv kernel family for element dtype f32 (see qmv_impl.h).
#include "qmv_impl.h"

namespace mtq {
template int qmv_launch_dtype<DT_F32>(QmvKArgs&, int, int, const QmvGeom&, const LaunchCtx&);
template int qmv_stream_launch_dtype<DT_F32>(QmvSArgs&, int, int, const QmvSGeom&, const LaunchCtx&);
template int qmv_stream_norm_launch_dtype<DT_F32>(QmvSArgs&, int, const QmvSGeom&, const LaunchCtx&);
}
