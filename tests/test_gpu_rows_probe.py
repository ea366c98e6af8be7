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
