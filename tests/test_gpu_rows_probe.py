"""The wave-per-four-rows measurement kernel (include/mtq_measure.h: mtq_probe_qmv_rows) computes the same product as
the reference's mt_qmv (crates/metaltile-std/src/mlx/quantized.rs:8-308): checked against the f64 oracle through the
C-ABI, so that its timings describe a kernel that does the whole job."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("N,K", [(4, 4096), (20, 4096), (1028, 4096), (14336, 4096), (1, 14336), (19, 14336), (1030, 14336), (4096, 14336)])
def test_rows_kernel_through_mtq_qmv(oracle, dt_name, N, K):
    """The same kernel as the product path of mtq_qmv (forced with qmv.kernel = 3 below its automatic size), ragged last
    workgroups included, behind a cache flush, against the f64 oracle and bit for bit against the streaming kernel's
    neighbour rows that it must not touch."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    dt = getattr(DType, dt_name)
    c = make_case(3200 + N + K, dt, 4, 64, 1, N, K)
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    out = GpuBuffer.from_bytes(np.full(N + 8, 0xABAB, np.uint16).tobytes())
    from metaltile_amd import _lib
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        assert ("qmv_rows_kernel" if K == 4096 else "qmv_rows_long_kernel") in ops.plan("qmv", dt, 4, 64, 1, N, K)[1][0][0]
        m.GpuRunner(0).flush_slc()
        ops.qmv(dt, 4, 64, bw, bs, bb, bx, out, 1, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_array(np.uint16)
    assert np.all(raw[N:] == 0xABAB)                       # nothing past the last row
    got = m.unpack_f32(raw[:N].tobytes(), dt)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 4, 64)
    assert rel_err(got, exp) <= 1e-2
    for b in (bw, bs, bb, bx, out):
        b.free()


@pytest.mark.parametrize("N", [16, 4096, 14336])
def test_rows_probe_matches_oracle(oracle, N):
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    K = 4096
    c = make_case(3100 + N, DType.BF16, 4, 64, 1, N, K)
    bufs = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes),
            GpuBuffer.from_bytes(c.x_bytes), GpuBuffer.from_bytes(np.full(N, 0xABAB, np.uint16).tobytes()))
    runner = m.GpuRunner(0)
    runner.flush_slc()
    us = runner.probe_qmv_rows([bufs], N, mode=0, repeat=1)
    assert us > 0
    got = m.unpack_f32(bufs[4].read_bytes(), DType.BF16)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 4, 64)
    assert rel_err(got, exp) <= 1e-2   # the headline configuration's bound (bf16 output rounding dominates)
    # the knocked-out modes run and are refused arguments are refused
    runner.probe_qmv_rows([bufs], N, mode=1, repeat=2)
    runner.probe_qmv_rows([bufs], N, mode=2, repeat=2)
    with pytest.raises(m.MtqError):
        runner.probe_qmv_rows([bufs], N + 4, mode=0)
    with pytest.raises(m.MtqError):
        runner.probe_qmv_rows([bufs], N, mode=3)
    for b in bufs:
        b.free()


@pytest.mark.parametrize("dt_name", ["F16", "BF16"])
@pytest.mark.parametrize("bits,G,N,K", [(2, 32, 50, 8192), (2, 64, 1, 8192), (2, 128, 8192, 8192), (2, 64, 33, 16384), (2, 32, 8192, 8192),
                                        (4, 32, 50, 8192), (4, 64, 8192, 8192), (4, 128, 17, 8192), (4, 128, 40, 14336),
                                        (4, 64, 33, 28672), (4, 128, 1030, 28672),
                                        # the row lengths of other models: whole groups of 64 chunks (10240, 12288, 18432 codes)
                                        # and the last group partly filled (11008: 24 of 64, 13824: 48, 18944: 16, 27648: 32)
                                        (4, 64, 1030, 10240), (4, 128, 33, 12288), (4, 64, 515, 18432), (4, 64, 4100, 11008), (4, 128, 19, 11008),
                                        (4, 64, 5120, 13824), (4, 128, 1, 13824), (4, 64, 3584, 18944), (4, 128, 50, 18944), (4, 64, 1027, 27648),
                                        (4, 128, 16, 27648)])
def test_one_row_per_wave_kernel_other_widths_and_groups(oracle, dt_name, bits, G, N, K):
    """The one-row-per-wave kernel on the shapes it takes beyond the two of the headline: 2-bit codes (made operands in
    place, with an offset that depends on the crumb's position) and 4-bit codes in groups of 32 / 64 / 128 on rows of
    8192, 14336, 16384 (2-bit) and 28672 codes (the last with eight groups of the bias term per lane), and 4-bit codes in
    groups of 64 / 128 on the row lengths of other models, forced with qmv.kernel = 3, ragged last workgroups, behind a
    cache flush, against the f64 oracle on full-range codes."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    dt = getattr(DType, dt_name)
    c = make_case(3300 + bits * 7 + G + N + K, dt, bits, G, 1, N, K, bias_rule="midpoint")
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    out = GpuBuffer.from_bytes(np.full(N + 8, 0xABAB, np.uint16).tobytes())
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        name = ops.plan("qmv", dt, bits, G, 1, N, K)[1][0][0]
        assert "qmv_rows_long_kernel" in name or "qmv_rows_long_ragged_kernel" in name, name
        m.GpuRunner(0).flush_slc()
        ops.qmv(dt, bits, G, bw, bs, bb, bx, out, 1, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_array(np.uint16)
    assert np.all(raw[N:] == 0xABAB)
    got = m.unpack_f32(raw[:N].tobytes(), dt)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, bits, G)
    assert rel_err(got, exp) <= 1e-2
    for b in (bw, bs, bb, bx, out):
        b.free()


def test_shapes_the_one_row_per_wave_kernel_refuses():
    """Rows whose groups do not fit its bias-term ownership (more than 256 groups per row), other widths and other row
    lengths fall through to the kernels that served them before, also when the option asks for it."""
    from metaltile_amd import DType, ops, _lib
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        for bits, G, K in ((4, 32, 14336), (8, 64, 8192), (4, 32, 11008), (4, 64, 9216), (2, 16, 8192), (4, 64, 2048), (3, 64, 8192), (4, 32, 28672), (2, 32, 16384), (4, 64, 16384),
                           (4, 64, 57344)):
            rc, launches, _, _ = ops.plan("qmv", DType.F16, bits, G, 1, 4096, K)
            assert rc == 0 and "qmv_rows" not in launches[0][0], (bits, G, K, launches[0][0])
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
