"""Stacked expert weights larger than 4 GiB: the routed expert's slab starts beyond the 32-bit
byte range of the weight buffer, so any 32-bit offset arithmetic on the way to it would read the
wrong slab. Only that expert's slab (and its scales / biases) holds real data; the rest of the
stack is a constant fill. Checked against the oracle's plain qmm on the expert's own matrix,
1e-2 on max|a-e| / max(|e|, 1) (the bf16 bound of the gather configuration)."""
import ctypes as C

import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, _lib, ops, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu


def _upload_at(buf, offset, data):
    lib = _lib.load()
    arr = np.ascontiguousarray(np.frombuffer(data, dtype=np.uint8))
    assert offset + arr.nbytes <= buf.nbytes
    _lib.check(lib.mtq_upload(C.c_void_p(buf.ptr + offset), arr.ctypes.data_as(C.c_void_p), arr.nbytes))


def test_expert_slab_beyond_4gib(oracle):
    dt, bits, G = DType.BF16, 4, 64
    E, N, K, T = 140, 8192, 8192, 5           # 32 MiB of codes per expert, 4.4 GiB in all
    e = E - 1
    wpe, spe = N * K // 2, N * (K // G) * 2   # bytes per expert: codes, scales (= biases)
    assert e * wpe >= 1 << 32
    c = make_case(6100, dt, bits, G, T, N, K)
    print(f"[case] gather into expert {e} of {E}, slab offset {e * wpe / 2**30:.2f} GiB", flush=True)
    lib = _lib.load()
    w, s, b = GpuBuffer(E * wpe), GpuBuffer(E * spe), GpuBuffer(E * spe)
    _lib.check(lib.mtq_memset(C.c_void_p(w.ptr), 0x5A, w.nbytes))
    _lib.check(lib.mtq_memset(C.c_void_p(s.ptr), 0, s.nbytes))
    _lib.check(lib.mtq_memset(C.c_void_p(b.ptr), 0, b.nbytes))
    _upload_at(w, e * wpe, c.w.tobytes())
    _upload_at(s, e * spe, c.scales_bytes)
    _upload_at(b, e * spe, c.biases_bytes)
    x = GpuBuffer.from_bytes(c.x_bytes)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, T, N, K, bits, G, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), 2)

    offsets = np.zeros(E + 1, "<u4")
    offsets[e + 1:] = T                        # every row belongs to the last expert
    indices = np.full(T, e, "<u4")
    for view, route, fn in (("csr", offsets, ops.gather_qmv_csr), ("indices", indices, ops.gather_qmv_indices)):
        out = GpuBuffer(T * N * 2)
        r = GpuBuffer.from_bytes(route.tobytes())
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), dt)
        out.free(); r.free()
        assert rel_err(got, exp) <= 1e-2, view
    # one row, expert id read on the device
    out = GpuBuffer(N * 2)
    r = GpuBuffer.from_bytes(np.array([e], "<u4").tobytes())
    x1 = GpuBuffer.from_bytes(c.x_bytes[:K * 2])
    ops.gather_qmv_single(dt, bits, G, w, s, b, x1, r, out, N, K, E)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, exp[:N]) <= 1e-2
    for buf in (w, s, b, x, x1, r, out):
        buf.free()


@pytest.mark.parametrize("M", [1, 4, 32])
def test_single_matrix_beyond_4gib(oracle, M):
    """One weight matrix of 4.5 GiB: the last rows lie beyond the 32-bit byte range. Real data in the
    first and the last 32 rows (checked against the oracle on those rows), constant fill between."""
    dt, bits, G = DType.BF16, 4, 64
    N, K, R = 589824, 16384, 32
    rb, sb_row = K // 2, (K // G) * 2             # bytes per row: codes, scales (= biases)
    assert (N - R) * rb >= 1 << 32
    print(f"[case] qmv on a {N * rb / 2**30:.2f} GiB matrix, M={M}", flush=True)
    lib = _lib.load()
    w, s, b = GpuBuffer(N * rb), GpuBuffer(N * sb_row), GpuBuffer(N * sb_row)
    _lib.check(lib.mtq_memset(C.c_void_p(w.ptr), 0x33, w.nbytes))
    _lib.check(lib.mtq_memset(C.c_void_p(s.ptr), 0, s.nbytes))
    _lib.check(lib.mtq_memset(C.c_void_p(b.ptr), 0, b.nbytes))
    cases = {}
    for tag, row0 in (("first", 0), ("last", N - R)):
        c = make_case(6200 + row0 % 97 + M, dt, bits, G, M, R, K)
        cases[tag] = (row0, c)
        _upload_at(w, row0 * rb, c.w.tobytes())
        _upload_at(s, row0 * sb_row, c.scales_bytes)
        _upload_at(b, row0 * sb_row, c.biases_bytes)
    x_case = cases["first"][1]                     # one activation batch for the whole matrix
    x = GpuBuffer.from_bytes(x_case.x_bytes)
    out = GpuBuffer(M * N * 2)
    (ops.qmm if M >= 32 else ops.qmv)(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt).reshape(M, N)
    for tag, (row0, c) in cases.items():
        exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, x_case.x_f, M, R, K, bits, G, threads=8)
        exp = oracle.round_through(exp.astype(np.float32), 2).reshape(M, R)
        # 32 rows may take the tile kernel, which rounds the weights to bf16 first: the reference's 5e-2 bound
        assert rel_err(got[:, row0:row0 + R].reshape(-1), exp.reshape(-1)) <= (5e-2 if M >= 32 else 1e-2), tag
    # rows of the constant fill have zero scale and bias
    assert not np.any(got[:, R:N - R])
    for buf in (w, s, b, x, out):
        buf.free()
