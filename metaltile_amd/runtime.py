"""Host-side mirror of the reference runtime surface, on the HIP C-ABI.

`Context.dispatch_with_grid` follows
crates/metaltile-runtime/src/context.rs:269-283 (named byte buffers in, named
output bytes out, copy-in / copy-out per call); `GpuRunner` follows
crates/metaltile-std/src/runner.rs (resident buffers, `measure`, `flush_slc`).
A kernel is identified by the reference kernel's name plus the element dtype.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Sequence

import numpy as np

from . import _lib
from .dtypes import DType
from .errors import MtqError
from .signatures import KERNEL_SIGNATURES, KernelSignature

_initialised_device: Optional[int] = None


def _ensure_init(device: int = 0):
    global _initialised_device
    lib = _lib.load()
    if _initialised_device != device:
        _lib.check(lib.mtq_init(device))
        _initialised_device = device
    return lib


@dataclass
class DispatchResult:
    """crates/metaltile-runtime/src/context.rs:49-56."""
    elapsed_us: float
    gflops: float = 0.0
    outputs: Dict[str, bytes] = field(default_factory=dict)


class GpuBuffer:
    """A resident device allocation (crates/metaltile-std/src/runner.rs:168-181)."""

    def __init__(self, nbytes: int, device: int = 0):
        self._lib = _ensure_init(device)
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _lib.check(self._lib.mtq_alloc(self.nbytes, C.byref(p)))
        self.ptr = p.value

    @classmethod
    def from_bytes(cls, data, device: int = 0) -> "GpuBuffer":
        arr = np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes, device)
        buf.upload(arr)
        return buf

    def upload(self, data) -> None:
        arr = np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data
        arr = np.ascontiguousarray(arr)
        if arr.nbytes > self.nbytes:
            raise MtqError(-4, f"upload of {arr.nbytes} bytes into a {self.nbytes}-byte buffer")
        _lib.check(self._lib.mtq_upload(self.ptr, arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def read_bytes(self, n: Optional[int] = None) -> bytes:
        n = self.nbytes if n is None else int(n)
        out = np.empty(n, dtype=np.uint8)
        _lib.check(self._lib.mtq_download(out.ctypes.data_as(C.c_void_p), self.ptr, n))
        return out.tobytes()

    def read_array(self, dtype, count: Optional[int] = None) -> np.ndarray:
        dtype = np.dtype(dtype)
        n = self.nbytes // dtype.itemsize if count is None else int(count)
        out = np.empty(n, dtype=dtype)
        _lib.check(self._lib.mtq_download(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes))
        return out

    def zero(self) -> None:
        _lib.check(self._lib.mtq_memset(self.ptr, 0, self.nbytes))

    def free(self) -> None:
        if getattr(self, "ptr", None):
            self._lib.mtq_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _bind(sig: KernelSignature, bufs: Mapping[str, GpuBuffer], consts: Mapping[str, int]):
    missing = [p for p in sig.params if p not in bufs] + [c for c in sig.constexprs if c not in consts]
    if missing:
        raise MtqError(-2, f"{sig.name}: missing bindings {missing}")
    barr = (_lib.MtqBuf * len(sig.params))()
    for i, p in enumerate(sig.params):
        barr[i].ptr = bufs[p].ptr
        barr[i].bytes = bufs[p].nbytes
    carr = (C.c_uint32 * len(sig.constexprs))(*[int(consts[c]) for c in sig.constexprs])
    return barr, carr


def _u3(v: Sequence[int]):
    return (C.c_uint32 * 3)(*[int(x) for x in v])


class Context:
    """crates/metaltile-runtime/src/context.rs:174-298, HIP flavour."""

    def __init__(self, device: int = 0):
        self._lib = _ensure_init(device)
        self.device = device

    def device_name(self) -> str:
        out = C.create_string_buffer(128)
        _lib.check(self._lib.mtq_device_name(out, 128))
        return out.value.decode()

    def dispatch_with_grid(self, kernel: str, dtype: DType, buffers: Mapping[str, bytes],
                           fn_consts: Optional[Mapping[str, int]] = None,
                           grid_groups: Sequence[int] = (1, 1, 1),
                           threads_per_group: Sequence[int] = (64, 1, 1)) -> DispatchResult:
        """Upload `buffers`, run `kernel`, read back its output parameters.

        As in the reference's test harness (crates/metaltile-std/src/run_kernel.rs:101-107)
        constexprs may be given inside `buffers` as 4-byte little-endian values
        or separately in `fn_consts`.
        """
        sig = KERNEL_SIGNATURES.get(kernel)
        if sig is None:
            raise MtqError(-5, f"unknown kernel '{kernel}'")
        consts = dict(fn_consts or {})
        for c in sig.constexprs:
            if c not in consts and c in buffers:
                raw = bytes(buffers[c])
                if len(raw) < 4:
                    raise MtqError(-4, f"constexpr '{c}' needs 4 bytes, got {len(raw)}")
                consts[c] = int.from_bytes(raw[:4], "little")
        dev: Dict[str, GpuBuffer] = {}
        try:
            for p in sig.params:
                if p not in buffers:
                    raise MtqError(-2, f"{kernel}: buffer '{p}' not bound")
                dev[p] = GpuBuffer.from_bytes(bytes(buffers[p]), self.device)
            barr, carr = _bind(sig, dev, consts)
            us = C.c_double(0.0)
            _lib.check(self._lib.mtq_dispatch(kernel.encode(), int(dtype), barr, len(sig.params), carr,
                                              len(sig.constexprs), _u3(grid_groups),
                                              _u3(threads_per_group), C.byref(us)))
            outs = {p: dev[p].read_bytes(len(buffers[p])) for p in sig.outputs}
            return DispatchResult(elapsed_us=us.value, gflops=0.0, outputs=outs)
        finally:
            for b in dev.values():
                b.free()


class GpuRunner:
    """crates/metaltile-std/src/runner.rs:253-475, HIP flavour (resident buffers)."""

    def __init__(self, device: int = 0):
        self._lib = _ensure_init(device)
        self.device = device

    def device_name(self) -> str:
        return Context(self.device).device_name()

    def device_info(self) -> dict:
        info = _lib.MtqDeviceInfo()
        _lib.check(self._lib.mtq_get_device_info(C.byref(info)))
        return {k: (getattr(info, k).decode() if isinstance(getattr(info, k), bytes) else getattr(info, k))
                for k, _ in info._fields_}

    def buffer_bytes(self, data) -> GpuBuffer:
        return GpuBuffer.from_bytes(data, self.device)

    def buffer_zeros(self, nbytes: int) -> GpuBuffer:
        return GpuBuffer(nbytes, self.device)

    def read_bytes(self, buf: GpuBuffer, n: int) -> bytes:
        return buf.read_bytes(n)

    def dispatch(self, kernel: str, dtype: DType, bufs: Mapping[str, GpuBuffer],
                 consts: Mapping[str, int]) -> float:
        sig = KERNEL_SIGNATURES[kernel]
        barr, carr = _bind(sig, bufs, consts)
        us = C.c_double(0.0)
        _lib.check(self._lib.mtq_dispatch(kernel.encode(), int(dtype), barr, len(sig.params), carr,
                                          len(sig.constexprs), _u3((1, 1, 1)), _u3((64, 1, 1)),
                                          C.byref(us)))
        return us.value

    def measure(self, kernel: str, dtype: DType, bufs: Mapping[str, GpuBuffer],
                consts: Mapping[str, int], warmup: int, iters: int) -> List[float]:
        sig = KERNEL_SIGNATURES[kernel]
        barr, carr = _bind(sig, bufs, consts)
        samples = (C.c_double * max(iters, 1))()
        _lib.check(self._lib.mtq_measure(kernel.encode(), int(dtype), barr, len(sig.params), carr,
                                         len(sig.constexprs), _u3((1, 1, 1)), _u3((64, 1, 1)),
                                         int(warmup), int(iters), samples))
        return [samples[i] for i in range(iters)]

    def dispatch_chain(self, specs, repeat: int = 1, per_kernel: bool = True, stream_events: bool = False):
        """Enqueue `specs` = [(kernel, dtype, bufs, consts), ...] back to back,
        `repeat` times, with no host wait in between (the reference's
        `Context::dispatch_chain` over resident buffers,
        crates/metaltile-runtime/src/context.rs:363-401). Returns
        (per-dispatch GPU durations in us or None, wall-clock us, time between
        two events bracketing the chain on the stream in us or None)."""
        n = len(specs)
        arr = (_lib.MtqDispatchSpec * max(n, 1))()
        keep = []
        for i, (kernel, dtype, bufs, consts) in enumerate(specs):
            sig = KERNEL_SIGNATURES[kernel]
            barr, carr = _bind(sig, bufs, consts)
            name = kernel.encode()
            keep.append((barr, carr, name))
            arr[i].kernel_name = name
            arr[i].dtype = int(dtype)
            arr[i].bufs = barr
            arr[i].n_bufs = len(sig.params)
            arr[i].consts = carr
            arr[i].n_consts = len(sig.constexprs)
        total = n * repeat
        per = (C.c_double * max(total, 1))() if per_kernel else None
        wall = C.c_double(0.0)
        sus = C.c_double(0.0)
        _lib.check(self._lib.mtq_dispatch_chain(arr, n, int(repeat), per, C.byref(wall),
                                                C.byref(sus) if stream_events else None))
        return ([per[i] for i in range(total)] if per_kernel else None), wall.value, (sus.value if stream_events else None)

    def copy_kernel(self, dst: GpuBuffer, src: GpuBuffer, nbytes: int, repeat: int = 1) -> float:
        us = C.c_double(0.0)
        _lib.check(self._lib.mtq_copy_kernel(dst.ptr, src.ptr, int(nbytes), int(repeat), C.byref(us)))
        return us.value

    def read_kernel(self, srcs, nbytes: int, repeat: int = 1, workgroups: int = 0, in_flight: int = 8, nontemporal: bool = False) -> float:
        """Average duration (us) of a launch that only reads `nbytes` of each buffer in `srcs`, enqueued back to back."""
        us = C.c_double(0.0)
        arr = (C.c_void_p * len(srcs))(*[s.ptr for s in srcs])
        sink = GpuBuffer(16)
        try:
            _lib.check(self._lib.mtq_read_kernel(arr, len(srcs), int(nbytes), int(repeat), int(workgroups), int(in_flight), int(bool(nontemporal)),
                                                 sink.ptr, C.byref(us)))
        finally:
            sink.free()
        return us.value

    def flush_slc(self) -> None:
        _lib.check(self._lib.mtq_flush_cache())

    def wake_clocks(self, min_gpu_ms: float = 40.0):
        """Sustained full-grid load for at least `min_gpu_ms` of GPU time (the reference's `wake_dvfs`,
        crates/metaltile-std/src/runner.rs:280-284, sized by time). Returns (GPU ms spent, dispatches)."""
        ms, n = C.c_double(0.0), C.c_int(0)
        _lib.check(self._lib.mtq_wake_clocks(float(min_gpu_ms), C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def clock_probe(self) -> dict:
        """One reading of the shader clock behind whatever is queued on the library's stream."""
        s = _lib.MtqClockSample()
        _lib.check(self._lib.mtq_clock_probe(C.byref(s)))
        return {"sclk_mhz": s.sclk_mhz, "counter_mhz": s.counter_mhz, "probe_us": s.probe_us,
                "wall_clock_mhz": s.wall_clock_mhz, "valu_ops": int(s.valu_ops)}

    def probe_qmv_rows(self, sets, N: int, mode: int = 0, repeat: int = 1, stamps: Optional[GpuBuffer] = None) -> float:
        """Average launch duration (us) of the wave-per-four-rows make of the 4-bit g64 bf16 GEMV (K = 4096) over
        `sets` = [(w, scales, biases, x, out) GpuBuffers, ...], enqueued back to back `repeat` times."""
        flat = [b.ptr for s in sets for b in s]
        arr = (C.c_void_p * len(flat))(*flat)
        us = C.c_double(0.0)
        _lib.check(self._lib.mtq_probe_qmv_rows(arr, len(sets), int(N), int(mode), int(repeat), stamps.ptr if stamps else None, C.byref(us)))
        return us.value

    def sync(self) -> None:
        _lib.check(self._lib.mtq_sync())
