"""MI355X-native affine-quantized matmul (qmv / qmm / gather_qmv).

Host-side Python mirror of the reference's runtime surface for this path
(`Context.dispatch_with_grid`, `GpuRunner`, `pack_f32`, `BenchStats`,
`mt_qmm_for`) on top of the C-ABI in ``include/mtq.h``. All compute happens in
hand-written HIP kernels inside ``libmtq_hip.so``; there is no CPU fallback.
"""
from .dtypes import DType, pack_f32, unpack_f32, dtype_label  # noqa: F401
from .errors import MtqError  # noqa: F401
from .stats import BenchStats, to_gbps, to_gflops  # noqa: F401
from .selector import mt_qmm_for  # noqa: F401
from . import dynamic_m  # noqa: F401
from .runtime import Context, DispatchResult, GpuRunner, GpuBuffer  # noqa: F401
from . import ops  # noqa: F401

__all__ = [
    "DType", "pack_f32", "unpack_f32", "dtype_label", "MtqError", "BenchStats", "to_gbps",
    "to_gflops", "mt_qmm_for", "Context", "DispatchResult", "GpuRunner", "GpuBuffer", "ops",
]
