"""The GEMV kernel for two to four activation rows (one wave per four weight rows, metaltile_amd/csrc/qmv_rows_few.hip)
against the f64 oracle: every width / group / row-length instance, both 16-bit types, 2, 3 and 4 rows of x, weight-row
counts that leave the last workgroup and the last wave ragged, behind a cache flush, with guard elements after each
output row block."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


CASES = [  # bits, G, K
    (4, 32, 4096), (4, 64, 4096), (4, 128, 4096),
    (4, 32, 8192), (4, 64, 8192), (4, 128, 8192),
    (2, 32, 8192), (2, 64, 8192), (2, 128, 8192),
]


@pytest.mark.parametrize("dt_name", ["F16", "BF16"])
@pytest.mark.parametrize("bits,G,K", CASES)
@pytest.mark.parametrize("M,N", [(2, 1), (3, 37), (4, 1030), (4, 64)])
def test_few_rows_kernel_matches_oracle(oracle, dt_name, bits, G, K, M, N):
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    dt = getattr(DType, dt_name)
    c = make_case(4400 + bits * 11 + G + N + K + M, dt, bits, G, M, N, K, bias_rule="midpoint")
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    out = GpuBuffer.from_bytes(np.full(M * N + 8, 0xABAB, np.uint16).tobytes())
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        rc, launches, _, _ = ops.plan("qmv", dt, bits, G, M, N, K)
        assert rc == 0 and "qmv_rows_few_kernel" in launches[0][0], launches
        assert launches[0][1][0] == (N + 31) // 32 and launches[0][2][0] == 1024, launches[0]
        m.GpuRunner(0).flush_slc()
        ops.qmv(dt, bits, G, bw, bs, bb, bx, out, M, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_array(np.uint16)
    assert np.all(raw[M * N:] == 0xABAB)
    got = m.unpack_f32(raw[:M * N].tobytes(), dt)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G)
    assert rel_err(got, exp) <= 1e-2   # 16-bit output rounding dominates
    for b in (bw, bs, bb, bx, out):
        b.free()


def test_rows_are_independent(oracle):
    """Each activation row's result does not depend on what the other rows hold: four rows at once equal the same rows
    run two at a time, bit for bit (rows the call does not bind enter the matrix instruction as zeros)."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    dt, bits, G, N, K = DType.BF16, 4, 64, 96, 8192
    c = make_case(4501, dt, bits, G, 4, N, K, bias_rule="midpoint")
    bw, bs, bb = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes))
    xb = c.x_bytes
    row = K * 2
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        bx = GpuBuffer.from_bytes(xb)
        out4 = GpuBuffer.from_bytes(bytes(4 * N * 2))
        ops.qmv(dt, bits, G, bw, bs, bb, bx, out4, 4, N, K)
        all4 = out4.read_array(np.uint16).reshape(4, N)
        for lo in (0, 2):
            bx2 = GpuBuffer.from_bytes(xb[lo * row:(lo + 2) * row])
            out2 = GpuBuffer.from_bytes(bytes(2 * N * 2))
            ops.qmv(dt, bits, G, bw, bs, bb, bx2, out2, 2, N, K)
            assert np.array_equal(out2.read_array(np.uint16).reshape(2, N), all4[lo:lo + 2])
            bx2.free(); out2.free()
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    for b in (bw, bs, bb, bx, out4):
        b.free()


def test_shapes_the_few_rows_kernel_refuses():
    """One row, more than four rows, other widths and row lengths stay on the kernels that served them before, also when
    the option asks for the wave-per-row kernels."""
    from metaltile_amd import DType, ops, _lib
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        for bits, G, M, K in ((4, 64, 1, 8192), (4, 64, 5, 8192), (8, 64, 4, 8192), (2, 64, 4, 16384), (4, 64, 4, 14336), (4, 16, 4, 8192),
                              (2, 64, 4, 4096)):
            rc, launches, _, _ = ops.plan("qmv", DType.F16, bits, G, M, 4096, K)
            assert rc == 0 and "qmv_rows_few" not in launches[0][0], (bits, G, M, K, launches[0][0])
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
