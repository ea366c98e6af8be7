"""Host-side driver for prefill with an arbitrary token count.

Mirrors crates/metaltile-std/src/mlx/quantized_mma_dynamic_m.rs:48-110: the reference pads
the activation rows to a multiple of its 32-row tile, dispatches `mt_qmm_mma` over the padded
shape and lets the caller drop the padding rows. The HIP tile kernel guards its row tail
itself, so `qmm_dynamic_m` below needs no padding; the reference's helpers are kept with
their names and values for callers that size buffers or grids the reference's way.
"""
from __future__ import annotations

from . import ops
from .dtypes import DType

BM_TILE = 32
BN_TILE = 32
BK_TILE = 32
TPG = 128


def pad_t_to_bm(t: int) -> int:
    """Round `t` up to the next multiple of 32 (quantized_mma_dynamic_m.rs:68-71)."""
    return -(-t // BM_TILE) * BM_TILE


def pad_x_rows_bytes(x_bytes: bytes, t: int, k: int, bytes_per_elem: int) -> bytes:
    """Append zero rows up to pad_t_to_bm(t) (quantized_mma_dynamic_m.rs:80-88)."""
    row = k * bytes_per_elem
    if len(x_bytes) != t * row:
        raise ValueError("x_bytes must be t * k * bytes_per_elem")
    return bytes(x_bytes) + bytes((pad_t_to_bm(t) - t) * row)


def dispatch_grid(t: int, n: int):
    """Threadgroup grid [N/32, m_padded/32, 1] of the reference's dispatch (quantized_mma_dynamic_m.rs:105-109)."""
    if n % BN_TILE:
        raise ValueError(f"n must be multiple of {BN_TILE} (BN tile)")
    return [n // BN_TILE, pad_t_to_bm(t) // BM_TILE, 1]


def kernel_name_for(dtype: DType) -> str:
    """The kernel the reference's dynamic-M path dispatches for every dtype."""
    del dtype
    return "mt_qmm_mma"


def qmm_dynamic_m(dtype: DType, bits: int, group_size: int, w, scales, biases, x, out, t: int, n: int, k: int):
    """out[t, n] = x[t, k] @ w_hat.T for any token count t >= 0 in one call; x and out hold exactly t rows."""
    if t == 0:
        return
    ops.qmm(dtype, bits, group_size, w, scales, biases, x, out, t, n, k)
