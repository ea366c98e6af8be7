"""The GEMV whose waves walk the rows (qmv_rows_walk_kernel: the activations put into operand order once per workgroup,
each wave taking rows g, g + G, ... with the next row's loads in flight) computes the reference's affine_qmv product
(crates/metaltile-std/src/mlx/quantized.rs:8-308; crates/metaltile-std/src/ffai/dequant_gemv.rs:52-100 for the other
group sizes): every instance through the C-ABI against the f64 oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# Rows per launch chosen for the ways a wave's share can end: one workgroup of sixteen rows per 16 rows up to 4096 rows
# (every wave one row or none), 4096 waves beyond (8192: two rows each; 12289: three, and one wave a fourth; 20481: five
# or six), ragged last workgroups, a single row. From 16384 rows of 4096 codes in groups of 64 a turn's rows are dealt to
# the waves slot by slot instead of workgroup by workgroup (16384: the first such size, four rows each; 20481).
ROWS = [1, 5, 16, 1030, 4096, 4100, 8192, 12289, 16384, 20481]


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("G", [32, 64, 128])
@pytest.mark.parametrize("K", [2048, 3072, 3584, 4096, 5120, 6144, 7168, 8192])
@pytest.mark.parametrize("N", ROWS)
def test_rows_walk_kernel_against_the_oracle(oracle, dt_name, G, K, N):
    """Forced with qmv.kernel = 4 (its automatic sizes start at 1536 rows), behind a cache flush, guard elements after
    the output, full-range codes, at the bound of the headline configuration."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    if N > 8192 and (G != 64 or K != 4096) and not (G == 32 and K == 8192 and dt_name == "F16") and not (G == 64 and K not in (4096, 8192) and dt_name == "BF16"):
        pytest.skip("the long walks run on the headline instance and on one instance of each other row length")
    dt = getattr(DType, dt_name)
    print(f"[case] rows walk {dt_name} g{G} N{N} K{K}", flush=True)
    c = make_case(5100 + N + K + G, dt, 4, G, 1, N, K, bias_rule="midpoint")
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    out = GpuBuffer.from_bytes(np.full(N + 8, 0xABAB, np.uint16).tobytes())
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 4) == 0
    try:
        rc, launches, _, n = ops.plan("qmv", dt, 4, G, 1, N, K)
        name = "qmv_rows_walk_kernel" if K % 2048 == 0 else "qmv_rows_walk_ragged_kernel"   # (rows that end inside a group of 64 chunks)
        assert rc == 0 and n == 1 and name in launches[0][0], launches
        m.GpuRunner(0).flush_slc()
        ops.qmv(dt, 4, G, bw, bs, bb, bx, out, 1, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_array(np.uint16)
    assert np.all(raw[N:] == 0xABAB)                       # nothing past the last row
    got = m.unpack_f32(raw[:N].tobytes(), dt)
    assert np.isfinite(got).all()
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 4, G)
    assert rel_err(got, exp) <= 1e-2
    for b in (bw, bs, bb, bx, out):
        b.free()


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("G", [32, 64, 128])
@pytest.mark.parametrize("N", [1, 50, 4096, 8192, 12289, 16390])
def test_rows_walk_kernel_two_bit_codes(oracle, dt_name, G, N):
    """2-bit codes on rows of 8192 (made operands in place, with an offset that depends on the crumb's position; groups
    of 32 span half a chunk, so a chunk's halves are scaled apart): forced with qmv.kernel = 4, full-range codes, behind
    a cache flush, guard elements, against the f64 oracle. (16390 rows: dealt to the waves slot by slot in groups of 32 / 64.)"""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    dt, K = getattr(DType, dt_name), 8192
    print(f"[case] rows walk 2-bit {dt_name} g{G} N{N}", flush=True)
    c = make_case(5300 + N + G, dt, 2, G, 1, N, K, bias_rule="midpoint")
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    out = GpuBuffer.from_bytes(np.full(N + 8, 0xABAB, np.uint16).tobytes())
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 4) == 0
    try:
        rc, launches, _, n = ops.plan("qmv", dt, 2, G, 1, N, K)
        assert rc == 0 and n == 1 and "qmv_rows_walk2_kernel" in launches[0][0], launches
        m.GpuRunner(0).flush_slc()
        ops.qmv(dt, 2, G, bw, bs, bb, bx, out, 1, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_array(np.uint16)
    assert np.all(raw[N:] == 0xABAB)
    got = m.unpack_f32(raw[:N].tobytes(), dt)
    assert np.isfinite(got).all()
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 2, G)
    assert rel_err(got, exp) <= 1e-2
    for b in (bw, bs, bb, bx, out):
        b.free()


def test_rows_walk_kernel_is_the_automatic_route_of_the_headline_shapes(oracle):
    """With no option set, the gate / up shape of the headline and a vocabulary projection take this kernel, and the
    result equals the forced wave-per-four-rows kernel's to the rounding of the output type."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, ops, _lib
    from metaltile_amd.synth import make_case
    from tests.parity import rel_err
    lib = _lib.load()
    dt, N, K = DType.BF16, 14336, 4096
    assert "qmv_rows_walk_kernel" in ops.plan("qmv", dt, 4, 64, 1, N, K)[1][0][0]
    c = make_case(5200, dt, 4, 64, 1, N, K)
    bw, bs, bb, bx = (GpuBuffer.from_bytes(v) for v in (c.w.tobytes(), c.scales_bytes, c.biases_bytes, c.x_bytes))
    outs = []
    for opt in (0, 3):
        out = GpuBuffer.from_bytes(np.full(N, 0xABAB, np.uint16).tobytes())
        assert lib.mtq_set_option(b"qmv.kernel", opt) == 0
        try:
            ops.qmv(dt, 4, 64, bw, bs, bb, bx, out, 1, N, K)
        finally:
            lib.mtq_set_option(b"qmv.kernel", 0)
        outs.append(m.unpack_f32(out.read_bytes(), dt))
        out.free()
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 4, 64)
    assert rel_err(outs[0], exp) <= 1e-2 and rel_err(outs[1], exp) <= 1e-2
    assert rel_err(outs[0], outs[1]) <= 2.0 ** -7          # two summation orders, each rounded to bf16 once
    for b in (bw, bs, bb, bx):
        b.free()
