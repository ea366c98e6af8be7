"""Every code width 2..8 on shapes that take the tiled kernels (rows of whole
512-code segments), batches of 1..17 rows and both gather views, against the
f64-accumulated oracle. Tolerance on max|a-e|/max(|e|,1): 1e-2 for f16/bf16
(the benchmark configurations' bound), 1e-4 for f32."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}


def _expected(oracle, c, x=None, M=None):
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f if x is None else x, c.M if M is None else M, c.N, c.K,
                         c.bits, c.group_size, threads=8)
    return oracle.round_through(exp.astype(np.float32), ODT[c.dtype])


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16, DType.F32], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("M,N,K,G", [(1, 200, 1024, 64), (4, 72, 2048, 32), (9, 40, 1024, 128), (17, 36, 512, 64)])
def test_batched_rows_all_widths(oracle, bits, M, N, K, G, dt):
    c = make_case(500 + bits * 10 + M, dt, bits, G, M, N, K, bias_rule="midpoint")
    print(f"[case] qmv {dt.name} b{bits} g{G} M{M} N{N} K{K}", flush=True)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmv(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, _expected(oracle, c)) <= TOL[dt]
    for buf in (w, s, b, x, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_gather_all_widths(oracle, bits, dt):
    """5 experts, 23 rows with one empty expert and one with 11 rows (more than one pass), both routing views."""
    E, N, K, G = 5, 44, 1024, 64
    counts = [3, 0, 11, 1, 8]
    T = sum(counts)
    c = make_case(700 + bits, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype("<u4")
    indices = np.repeat(np.arange(E), counts).astype("<u4")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=indices, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    for view, route, fn in (("csr", offsets, ops.gather_qmv_csr), ("indices", indices, ops.gather_qmv_indices)):
        print(f"[case] gather {view} {dt.name} b{bits}", flush=True)
        out = GpuBuffer(T * N * dt.size_bytes)
        r = GpuBuffer.from_bytes(route.tobytes())
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), dt)
        assert rel_err(got, exp) <= TOL[dt], view
        out.free(); r.free()
    # unsorted per-row indices: a permutation of the rows permutes the outputs
    perm = np.random.default_rng(bits).permutation(T)
    xp = c.x_f.reshape(T, K)[perm].reshape(-1)
    xb = GpuBuffer.from_bytes(pack_f32(xp, dt))
    r = GpuBuffer.from_bytes(indices[perm].astype("<u4").tobytes())
    out = GpuBuffer(T * N * dt.size_bytes)
    ops.gather_qmv_indices(dt, bits, G, xb, w, s, b, r, out, T, N, K, E)
    got = unpack_f32(out.read_bytes(), dt).reshape(T, N)
    assert rel_err(got.reshape(-1), exp.reshape(T, N)[perm].reshape(-1)) <= TOL[dt]
    for buf in (w, s, b, x, xb, r, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("G", [256, 512, 1024, 2048])
@pytest.mark.parametrize("M", [1, 4, 8])
def test_large_groups(oracle, M, G, bits, dt):
    """Groups of 256..2048 codes: wider than one wave-wide step of the matrix-core GEMV for the
    larger ones, which then hands the request to the other kernels of the family."""
    N, K = 136, 4096
    c = make_case(900 + bits + G + M, dt, bits, G, M, N, K, bias_rule="midpoint")
    print(f"[case] large group {dt.name} b{bits} g{G} M{M}", flush=True)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmv(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, _expected(oracle, c)) <= TOL[dt]
    for buf in (w, s, b, x, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("K", [768, 896, 1152, 1280, 2880, 3584, 11008, 18944])
@pytest.mark.parametrize("M", [1, 3, 8])
def test_rows_that_are_not_whole_steps(oracle, M, K, bits, dt):
    """Row lengths of real models that are not a whole number of the kernels' wave-wide steps
    (768, 1280, 11008: the last step is partial) or whose step count has no small divisor
    (3584 = 7 steps, 18944 = 37: K parts of unequal length), or whose rows of scales are not whole
    8-byte vectors (896, 1152, 2880: 14, 18, 45 groups)."""
    N, G = 52, 64
    c = make_case(1100 + bits + K % 97 + M, dt, bits, G, M, N, K, bias_rule="midpoint")
    print(f"[case] row length {K} {dt.name} b{bits} M{M}", flush=True)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmv(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, _expected(oracle, c)) <= TOL[dt]
    for buf in (w, s, b, x, out):
        buf.free()


@pytest.mark.parametrize("K", [768, 11008])
def test_gather_rows_that_are_not_whole_steps(oracle, K):
    E, N, G, bits, dt = 4, 44, 64, 4, DType.BF16
    counts = [5, 0, 2, 9]
    T = sum(counts)
    c = make_case(1200 + K % 89, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype("<u4")
    indices = np.repeat(np.arange(E), counts).astype("<u4")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=indices, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    for view, route, fn in (("csr", offsets, ops.gather_qmv_csr), ("indices", indices, ops.gather_qmv_indices)):
        print(f"[case] gather {view} row length {K}", flush=True)
        out = GpuBuffer(T * N * dt.size_bytes)
        r = GpuBuffer.from_bytes(route.tobytes())
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), dt)
        assert rel_err(got, exp) <= TOL[dt], view
        out.free(); r.free()
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,N,K", [(2, 100, 1024), (3, 64, 2080), (4, 256, 8192), (8, 40, 1024), (6, 33, 544)])
def test_2bit_groups_of_32_on_the_matrix_core_kernel(oracle, M, N, K, dt):
    """2-bit codes with groups of 32: a 16-byte lane chunk holds 64 codes (two groups), so the matrix-core
    kernel takes them 32 codes (8 bytes) per lane; rows that are not whole 512-code steps included. Batches
    and both gather views against the f64-accumulated oracle, 1e-2 as above."""
    bits, G = 2, 32
    c = make_case(900 + M + K, dt, bits, G, M, N, K, bias_rule="midpoint")
    print(f"[case] qmv {dt.name} b2 g32 M{M} N{N} K{K}", flush=True)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
    ops.qmv(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, _expected(oracle, c)) <= TOL[dt]
    for buf in (w, s, b, x, out):
        buf.free()
    # the same rows routed to 3 experts (one empty)
    E = 3
    counts = [M - 1, 0, 1]
    cg = make_case(950 + M + K, dt, bits, G, M, N, K, E=E, bias_rule="midpoint")
    indices = np.repeat(np.arange(E), counts).astype("<u4")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype("<u4")
    exp = oracle.gather_qmm(cg.x_f, cg.w, cg.scales_f, cg.biases_f, M, K, N, E, bits, G, indices=indices, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(cg.w.tobytes()), GpuBuffer.from_bytes(cg.scales_bytes),
                  GpuBuffer.from_bytes(cg.biases_bytes), GpuBuffer.from_bytes(cg.x_bytes))
    for view, route, fn in (("csr", offsets, ops.gather_qmv_csr), ("indices", indices, ops.gather_qmv_indices)):
        r = GpuBuffer.from_bytes(route.tobytes())
        out = GpuBuffer(M * N * dt.size_bytes)
        fn(dt, bits, G, x, w, s, b, r, out, M, N, K, E)
        assert rel_err(unpack_f32(out.read_bytes(), dt), exp) <= TOL[dt], view
        out.free(); r.free()
    for buf in (w, s, b, x):
        buf.free()
