"""Kernel routing by M for prefill.

Mirrors ``mt_qmm_for`` (crates/metaltile-std/src/mlx/quantized.rs:5040-5065):
returns the name of the reference kernel its selector picks. The HIP backend
accepts every one of these names; internally it runs the MFMA tile kernel for
the `mma` names and the GEMV family for the others.
"""
from .dtypes import DType


def mt_qmm_for(dtype: DType, m: int) -> str:
    del dtype  # the choice does not depend on dtype (only the reference's LDS skew does)
    if m >= 32 and m % 32 == 0:
        return "mt_qmm_mma"
    if m == 16:
        return "mt_qmm_mma_m16"
    if m >= 4 and m % 4 == 0:
        return "mt_qmm_bm4"
    if m >= 2 and m % 2 == 0:
        return "mt_qmm_bm2"
    return "mt_qmm"
