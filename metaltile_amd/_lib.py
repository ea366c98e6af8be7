"""ctypes binding of libmtq_hip.so (the C-ABI declared in include/mtq.h).

The library is looked up in-tree (metaltile_amd/libmtq_hip.so). If it is
missing, or no GPU is usable, callers get an exception: there is no fallback
implementation behind this module.
"""
from __future__ import annotations

import ctypes as C
import os

from .errors import MtqError

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmtq_hip.so")


class MtqBuf(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("bytes", C.c_size_t)]


class MtqDispatchSpec(C.Structure):
    _fields_ = [("kernel_name", C.c_char_p), ("dtype", C.c_int), ("bufs", C.POINTER(MtqBuf)),
                ("n_bufs", C.c_int), ("consts", C.POINTER(C.c_uint32)), ("n_consts", C.c_int)]


class MtqDeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128), ("arch", C.c_char * 32), ("compute_units", C.c_int),
        ("clock_khz", C.c_int), ("memory_clock_khz", C.c_int), ("memory_bus_bits", C.c_int),
        ("total_memory", C.c_size_t), ("l2_bytes", C.c_int), ("lds_per_cu_bytes", C.c_int),
    ]


PLAN_MAX_LAUNCHES = 8


class MtqClockSample(C.Structure):
    _fields_ = [("sclk_mhz", C.c_double), ("counter_mhz", C.c_double), ("probe_us", C.c_double),
                ("wall_clock_mhz", C.c_double), ("valu_ops", C.c_uint64)]


class MtqPlanLaunch(C.Structure):
    _fields_ = [("kernel", C.c_char * 192), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3), ("lds_bytes", C.c_size_t)]


class MtqPlanInfo(C.Structure):
    _fields_ = [("n_launches", C.c_int), ("launch", MtqPlanLaunch * PLAN_MAX_LAUNCHES), ("scratch_bytes", C.c_size_t)]


_u32 = C.c_uint32
_vp = C.c_void_p
_u32p = C.POINTER(C.c_uint32)
_dblp = C.POINTER(C.c_double)
_bufp = C.POINTER(MtqBuf)

# name -> (restype, argtypes); every symbol include/mtq.h and include/mtq_measure.h declare
SIGNATURES = {
    "mtq_init": (C.c_int, [C.c_int]),
    "mtq_shutdown": (C.c_int, []),
    "mtq_last_error": (C.c_char_p, []),
    "mtq_device_name": (C.c_int, [C.c_char_p, C.c_size_t]),
    "mtq_get_device_info": (C.c_int, [C.POINTER(MtqDeviceInfo)]),
    "mtq_set_stream": (C.c_int, [_vp]),
    "mtq_alloc": (C.c_int, [C.c_size_t, C.POINTER(_vp)]),
    "mtq_free": (C.c_int, [_vp]),
    "mtq_upload": (C.c_int, [_vp, _vp, C.c_size_t]),
    "mtq_download": (C.c_int, [_vp, _vp, C.c_size_t]),
    "mtq_memset": (C.c_int, [_vp, C.c_int, C.c_size_t]),
    "mtq_sync": (C.c_int, []),
    "mtq_qmv": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_qmm": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_gather_qmv_csr": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "mtq_gather_qmv_indices": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "mtq_gather_qmv_single": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_qvm": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_qvm_noalloc": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_qmv_batched": (C.c_int, [C.c_int, C.c_int, _u32, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                  C.POINTER(C.c_void_p), _vp, C.POINTER(C.c_void_p), _u32p, _u32]),
    "mtq_dequant_gather": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_qmm_batched": (C.c_int, [C.c_int, C.c_int, _u32, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                  C.POINTER(C.c_void_p), _vp, C.POINTER(C.c_void_p), _u32p, _u32, _u32]),
    "mtq_rms_norm_qmv": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32]),
    "mtq_gated_rms_norm_qmv": (C.c_int, [C.c_int, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_moe_router_topk": (C.c_int, [C.c_int, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "mtq_moe_sort_by_expert": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _vp]),
    "mtq_moe_permute": (C.c_int, [C.c_int, _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_moe_unpermute": (C.c_int, [C.c_int, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "mtq_moe_down_swiglu_accum": (C.c_int, [C.c_int, _u32, _u32, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), _vp, _vp, _vp,
                                            _vp, _vp, _vp, _u32, _u32, _u32]),
    "mtq_affine_quantize": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, C.c_size_t]),
    "mtq_affine_dequantize": (C.c_int, [C.c_int, C.c_int, _u32, _vp, _vp, _vp, _vp, C.c_size_t]),
    "mtq_dispatch": (C.c_int, [C.c_char_p, C.c_int, _bufp, C.c_int, _u32p, C.c_int, _u32p, _u32p, _dblp]),
    "mtq_measure": (C.c_int, [C.c_char_p, C.c_int, _bufp, C.c_int, _u32p, C.c_int, _u32p, _u32p, C.c_int, C.c_int, _dblp]),
    "mtq_dispatch_chain": (C.c_int, [C.POINTER(MtqDispatchSpec), C.c_int, C.c_int, _dblp, _dblp, _dblp]),
    "mtq_copy_kernel": (C.c_int, [_vp, _vp, C.c_size_t, C.c_int, _dblp]),
    "mtq_plan": (C.c_int, [C.c_int, C.c_int, C.c_int, _u32, _u32, _u32, _u32, _u32, _u32, C.POINTER(MtqPlanInfo)]),
    "mtq_read_kernel": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _dblp]),
    "mtq_kernel_supported": (C.c_int, [C.c_char_p]),
    "mtq_kernel_count": (C.c_int, []),
    "mtq_kernel_name": (C.c_char_p, [C.c_int]),
    "mtq_qmm_for": (C.c_char_p, [C.c_int, _u32]),
    "mtq_flush_cache": (C.c_int, []),
    "mtq_wake_clocks": (C.c_int, [C.c_double, _dblp, C.POINTER(C.c_int)]),
    "mtq_clock_probe": (C.c_int, [C.POINTER(MtqClockSample)]),
    "mtq_probe_qmv_rows": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, _u32, C.c_int, C.c_int, _vp, _dblp]),
    "mtq_set_option": (C.c_int, [C.c_char_p, C.c_int]),
    "mtq_timed_begin": (C.c_int, []),
    "mtq_timed_last_us": (C.c_int, [_dblp]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MtqError(-1, f"{LIB_PATH} is not built; run `python -m metaltile_amd.build` "
                           "(there is no fallback implementation)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().mtq_last_error()
        raise MtqError(rc, msg.decode("utf-8", "replace") if msg else "")
