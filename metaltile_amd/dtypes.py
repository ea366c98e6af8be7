"""Element dtypes and the byte packers of the test/bench setups.

Mirrors ``pack_f32`` / ``unpack_f32`` (crates/metaltile-std/src/utils.rs:26-65)
and ``dtype_label`` (crates/metaltile-std/src/bench_types.rs:20-32). f16 goes
through IEEE round-to-nearest-even including subnormals (what the `half` crate
does); bf16 is round-to-nearest-even on the raw f32 bits
(crates/metaltile-std/src/runner.rs:521-525).
"""
from __future__ import annotations

import enum

import numpy as np


class DType(enum.IntEnum):
    F32 = 0
    F16 = 1
    BF16 = 2
    U32 = 3

    @property
    def size_bytes(self) -> int:
        return 2 if self in (DType.F16, DType.BF16) else 4


def dtype_label(dt: DType) -> str:
    return {DType.F32: "f32", DType.F16: "f16", DType.BF16: "bf16", DType.U32: "u32"}.get(dt, "?")


def f32_to_bf16_bits(vals: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(vals, dtype=np.float32).view(np.uint32)
    r = (u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16
    out = r.astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    if nan.any():
        out = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), out)
    return out


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_f32(vals, dt: DType) -> bytes:
    """f32 values -> little-endian bytes of dtype `dt`."""
    v = np.ascontiguousarray(vals, dtype=np.float32).ravel()
    if dt == DType.F16:
        with np.errstate(over="ignore"):
            return v.astype("<f2").tobytes()
    if dt == DType.BF16:
        return f32_to_bf16_bits(v).astype("<u2").tobytes()
    if dt == DType.U32:
        return v.astype("<u4").tobytes()  # value cast, not a bit reinterpret
    return v.astype("<f4").tobytes()


def unpack_f32(data: bytes, dt: DType) -> np.ndarray:
    """Inverse of pack_f32; a trailing partial element is dropped."""
    sz = dt.size_bytes
    n = len(data) // sz
    buf = memoryview(data)[: n * sz]
    if dt == DType.F16:
        return np.frombuffer(buf, dtype="<f2").astype(np.float32)
    if dt == DType.BF16:
        return bf16_bits_to_f32(np.frombuffer(buf, dtype="<u2"))
    if dt == DType.U32:
        return np.frombuffer(buf, dtype="<u4").astype(np.float32)
    return np.frombuffer(buf, dtype="<f4").astype(np.float32)


def round_through(vals, dt: DType) -> np.ndarray:
    """`unpack_f32(pack_f32(v, dt), dt)`: the values a kernel sees after its load cast."""
    return unpack_f32(pack_f32(vals, dt), dt)
