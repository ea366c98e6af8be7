"""Every tiling of the direct matrix-core qmm kernel (K-groups 1, 2, 4 x tile heights 64,
128, and 32 with 4 K-groups), forced through the library's options on one ragged shape, against the oracle's
restatement of the reference's mma semantics (weights rounded to the element dtype
before the multiply, crates/metaltile-std/src/mlx/quantized.rs:2267-2274).
Tolerance: 2e-2 on max|a-e| / max(|e|, 1), the bound of the bf16 prefill configuration;
bit-equal results between tilings are not required (partial sums meet in a different order)."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, _lib, ops, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu

ODT = {DType.F16: 1, DType.BF16: 2}


def cold():
    """Empties the caches: the kernels whose loads are issued and waited for by hand must not depend on data
    arriving early (a wait that is one load short passes on warm caches)."""
    assert _lib.load().mtq_flush_cache() == 0


@pytest.fixture
def options():
    lib = _lib.load()

    def set_(name, value):
        assert lib.mtq_set_option(name.encode(), value) == 0, name

    yield set_
    for name in ("qmm.kernel", "qmm.kgroups", "qmm.tile_rows", "qmm.by_m", "qmm.ksplit", "qmm.dma"):
        lib.mtq_set_option(name.encode(), 0)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16])
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_direct_qmm_every_tiling(oracle, options, bits, dt):
    M, N, K, G = 200, 256, 1024, 64          # last 128-row and 64-row tiles are ragged
    c = make_case(5100 + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    for kg in (1, 2, 4):
        for rows in ((32, 64, 128) if kg == 4 else (64, 128)):
            print(f"[case] direct qmm {dt.name} b{bits} kgroups={kg} tile_rows={rows}", flush=True)
            options("qmm.kgroups", kg)
            options("qmm.tile_rows", rows)
            # both orders of walking the tiles; 4-bit codes on 2 K-groups also with and without the instances
            # that bring the activation tile in by load-to-LDS instructions
            for by_m, dma in ((1, 0), (2, 0), (1, 1)):
                options("qmm.by_m", by_m)
                options("qmm.dma", dma)
                out = GpuBuffer(M * N * dt.size_bytes)
                ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
                got = unpack_f32(out.read_bytes(), dt)
                out.free()
                err = rel_err(got, exp)
                assert err <= 2e-2, f"kgroups={kg} rows={rows} by_m={by_m} dma={dma}: rel err {err:.3e}"
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("N", [256, 8192])
@pytest.mark.parametrize("M", [9, 16, 17, 31])
def test_qmm_routing_between_8_and_32_rows(oracle, M, N):
    """9..31 activation rows go to the GEMV family (exact dequantisation) or to the tile kernel
    (weights rounded to bf16 first) depending on M and N; either way the result stays within the
    reference's bf16 bound against exact dequantisation, 5e-2 on max|a-e| / max(|e|, 1)
    (crates/metaltile-std/tests/qmm_gpu_correctness.rs:2085-2106)."""
    K, G, bits, dt = 1024, 64, 4, DType.BF16
    print(f"[case] qmm routing M={M} N={N}", flush=True)
    c = make_case(5200 + M + N, dt, bits, G, M, N, K)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    for buf in (w, s, b, x, out):
        buf.free()
    assert rel_err(got, exp) <= 5e-2


@pytest.mark.parametrize("K", [320, 768, 1152, 11008])
@pytest.mark.parametrize("M", [40, 300])
def test_tile_kernel_on_rows_of_whole_64s(oracle, M, K):
    """Row lengths that are multiples of 64 but not of 512 (768 and 11008 are down-projection widths
    of real models) run on the tile kernel, with fewer K-groups per workgroup or an odd number of iterations. Against the mma-semantics
    oracle, 2e-2 as for the prefill configuration."""
    N, G, bits, dt = 256, 64, 4, DType.BF16
    print(f"[case] qmm M={M} K={K}", flush=True)
    c = make_case(5300 + M + K % 101, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    for buf in (w, s, b, x, out):
        buf.free()
    assert rel_err(got, exp) <= 2e-2


@pytest.mark.parametrize("N", [8, 64, 192, 1000, 1001, 2880])
@pytest.mark.parametrize("tiling", [(0, 0), (128, 1), (128, 2), (64, 2), (64, 4), (32, 4)])
def test_tile_kernel_on_ragged_n(oracle, options, N, tiling):
    """Matrices whose row count is not a multiple of the tile width (2880 and odd vocabulary sizes in
    real models): the last column tile hangs over N, works its missing rows on row N - 1 and stores
    none of their columns. The output buffer carries a guard band after the last row that must stay
    untouched. Against the mma-semantics oracle, 2e-2 as for the prefill configuration."""
    rows, kg = tiling
    M, K, G, bits, dt = 70, 512, 64, 4, DType.BF16
    print(f"[case] qmm ragged N={N} tile_rows={rows} kgroups={kg}", flush=True)
    c = make_case(5600 + N + rows + kg, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    guard = 4096
    out = GpuBuffer.from_bytes(np.full(M * N + guard, 0x7B7B, np.uint16).tobytes())
    options("qmm.tile_rows", rows)
    options("qmm.kgroups", kg)
    options("qmm.kernel", 2)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    raw = np.frombuffer(out.read_bytes(), np.uint16)
    for buf in (w, s, b, x, out):
        buf.free()
    assert np.all(raw[M * N:] == 0x7B7B)
    got = unpack_f32(raw[:M * N].tobytes(), dt)
    assert rel_err(got, exp) <= 2e-2


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [3, 5, 6, 7])
def test_direct_qmm_bit_stream_widths(oracle, options, bits, dt):
    """3-, 5-, 6- and 7-bit codes on the register-operand tile kernel, every tiling built for them,
    ragged M and N. Against the mma-semantics oracle, 2e-2 as for the prefill configuration."""
    M, N, K, G = 200, 200, 1024, 64
    c = make_case(5700 + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    for rows, kg in ((0, 0), (128, 1), (64, 1), (64, 2), (64, 4), (32, 4)):
        print(f"[case] direct qmm {dt.name} b{bits} kgroups={kg} tile_rows={rows}", flush=True)
        options("qmm.kgroups", kg)
        options("qmm.tile_rows", rows)
        out = GpuBuffer.from_bytes(np.full(M * N + 512, 0x7B7B, np.uint16).tobytes())
        ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
        raw = np.frombuffer(out.read_bytes(), np.uint16)
        out.free()
        assert np.all(raw[M * N:] == 0x7B7B)
        err = rel_err(unpack_f32(raw[:M * N].tobytes(), dt), exp)
        assert err <= 2e-2, f"kgroups={kg} rows={rows}: rel err {err:.3e}"
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("M", [512, 2048])
def test_bit_stream_widths_route_to_tiles(oracle, bits, M):
    """The default routing at prefill sizes (128-row tiles from 2048 rows at N = 1024)."""
    N, K, G, dt = 1024, 512, 64, DType.BF16
    print(f"[case] qmm b{bits} M={M}", flush=True)
    c = make_case(5800 + bits + M, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    for buf in (w, s, b, x, out):
        buf.free()
    assert rel_err(got, exp) <= 2e-2


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_direct_qmm_split_k(oracle, options, bits, dt):
    """K cut into splits whose f32 partial tiles a second kernel adds in order: forced split counts that
    do and do not divide the iteration count (K = 1792 is 7 iterations of 256 and 14 of 128), ragged M and
    N, group sizes 32 and 128 (a split may start inside a group), and the automatic choice on a short, wide
    matrix. Against the mma-semantics oracle, 2e-2 as for the prefill configuration; a guard band after the
    output must stay untouched."""
    for (M, N, K, G) in ((20, 200, 1792, 128), (70, 72, 1792, 32)):
        c = make_case(5900 + bits + M, dt, bits, G, M, N, K)
        exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
        exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
        w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                      GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
        options("qmm.kernel", 2)
        for ks in (0, 1, 2, 3, 5, 7):
            print(f"[case] split-K qmm {dt.name} b{bits} M{M} N{N} K{K} g{G} ksplit={ks}", flush=True)
            options("qmm.ksplit", ks)
            out = GpuBuffer.from_bytes(np.full(M * N + 512, 0x7B7B, np.uint16).tobytes())
            ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
            raw = np.frombuffer(out.read_bytes(), np.uint16)
            out.free()
            assert np.all(raw[M * N:] == 0x7B7B)
            err = rel_err(unpack_f32(raw[:M * N].tobytes(), dt), exp)
            assert err <= 2e-2, f"ksplit={ks}: rel err {err:.3e}"
        for buf in (w, s, b, x):
            buf.free()


def test_split_k_is_deterministic_and_close_to_unsplit(options):
    """Two runs of a split launch give the same bits (the splits are added in a fixed order), and the
    split result differs from the unsplit one only by the order of the f32 sums."""
    dt, bits, G, M, N, K = DType.BF16, 4, 64, 32, 256, 8192
    c = make_case(5999, dt, bits, G, M, N, K)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    res = {}
    for ks in (1, 0, 0):
        options("qmm.ksplit", ks)
        out = GpuBuffer(M * N * 2)
        ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
        res.setdefault(ks, []).append(out.read_bytes())
        out.free()
    for buf in (w, s, b, x):
        buf.free()
    assert res[0][0] == res[0][1]
    assert rel_err(unpack_f32(res[0][0], dt), unpack_f32(res[1][0], dt)) <= 1e-2


@pytest.mark.parametrize("M,N", [(300, 256), (1100, 384)])
def test_tall_tiles_on_long_rows(oracle, M, N):
    """256 rows and more against rows of 8192 codes: the default choice is the 128-row tile on 4-wave
    workgroups with K split (300 x 256: 6 tiles, 8 splits), and above one tile per compute unit an
    inexact multiple also takes the 4-wave form. Against the mma-semantics oracle, 2e-2 as for the prefill
    configuration."""
    K, G, bits, dt = 8192, 64, 4, DType.BF16
    print(f"[case] qmm M={M} N={N} K={K}", flush=True)
    c = make_case(6100 + M, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    for buf in (w, s, b, x, out):
        buf.free()
    assert rel_err(got, exp) <= 2e-2


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,N,K,G", [(300, 256, 256, 32),      # two iterations; ragged last tiles at every height
                                     (257, 200, 768, 32),      # six iterations, N % 8 == 0 but N % 128 != 0
                                     (70, 131, 1024, 128),     # N % 8 != 0: element-wise stores
                                     (512, 384, 4096, 64),     # 64 groups per row: the 256-row tile's LDS is full to the byte
                                     (260, 128, 2816, 32)])    # 22 iterations (not a multiple of the unroll), 88 groups per row
@pytest.mark.parametrize("bits", [4, 8])
def test_load_to_lds_tiles(oracle, options, dt, M, N, K, G, bits):
    """The 4- and 8-bit instances whose activation tile arrives by load-to-LDS instructions, on 64-, 128- and
    256-row tiles, against the oracle's mma semantics (2e-2, as above) and against the register-staged instance of
    the same tiling (same arithmetic, same order of the partial sums: bit-equal)."""
    c = make_case(5400 + M + K + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    options("qmm.kgroups", 2)
    for rows in (64, 128, 256):
        if rows == 256 and K // G > 64:
            continue  # two 64 KB tiles leave room for 64 groups per row
        print(f"[case] load-to-LDS qmm {dt.name} b{bits} M={M} N={N} K={K} g{G} tile_rows={rows}", flush=True)
        options("qmm.tile_rows", rows)
        options("qmm.dma", 3)
        out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
        cold()
        ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
        got_bytes = out.read_bytes()
        got = unpack_f32(got_bytes, dt)
        out.free()
        assert rel_err(got, exp) <= 2e-2, f"rows={rows}"
        if rows != 256:
            options("qmm.dma", 1)
            out = GpuBuffer(M * N * dt.size_bytes)
            cold()
            ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
            assert out.read_bytes() == got_bytes, f"rows={rows}: differs from the register-staged instance"
            out.free()
    for buf in (w, s, b, x):
        buf.free()


def test_256_row_tiles_refuse_what_they_cannot_take(options):
    """Forced 256-row tiles on a shape outside their limits (4 groups per row) are refused, not rerouted."""
    dt, bits, G, M, N, K = DType.BF16, 8, 64, 256, 128, 256
    c = make_case(5500, dt, bits, G, M, N, K)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * dt.size_bytes)
    options("qmm.kernel", 2)
    options("qmm.tile_rows", 256)
    with pytest.raises(Exception, match="256"):
        ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    for buf in (w, s, b, x, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,N,K,G", [(300, 256, 8192, 64),     # 128 groups per row: 4 windows of 32
                                     (130, 200, 14336, 64),    # 224 groups: 7 windows, 112 iterations, ragged N
                                     (257, 131, 8192, 128),    # groups of 128: a window lasts 32 iterations; N % 8 != 0
                                     (512, 128, 4096, 64),     # 64 groups: whole rows fit, windows forced (2 windows)
                                     (64, 128, 2560, 64),      # 40 groups: the last window is partial (20 iterations)
                                     (96, 128, 11008, 64)])    # 172 groups: not whole 8-group vectors, 6 windows (the last of 12 groups)
@pytest.mark.parametrize("bits", [4, 8])
def test_load_to_lds_tiles_with_windowed_scales(oracle, options, dt, M, N, K, G, bits):
    """Rows too long for their scales and biases to sit in LDS whole: two windows of 32 groups refilled along K by
    load-to-LDS instructions. Forced (qmm.dma = 2) on every tile height (8-bit codes: 64 and 128 rows, the 256-row
    instance does not fit the register file), against the oracle's mma semantics (2e-2) and bit-equal to the
    register-staged instance of the same tiling."""
    c = make_case(5600 + M + K + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    options("qmm.kgroups", 2)
    for rows in (64, 128, 256) if bits == 4 else (64, 128):
        print(f"[case] windowed load-to-LDS qmm {dt.name} b{bits} M={M} N={N} K={K} g{G} tile_rows={rows}", flush=True)
        options("qmm.tile_rows", rows)
        options("qmm.dma", 2)
        out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
        cold()
        ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
        got_bytes = out.read_bytes()
        out.free()
        assert rel_err(unpack_f32(got_bytes, dt), exp) <= 2e-2, f"rows={rows}"
        if rows != 256:
            options("qmm.dma", 1)
            out = GpuBuffer(M * N * dt.size_bytes)
            cold()
            ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
            assert out.read_bytes() == got_bytes, f"rows={rows}: differs from the register-staged instance"
            out.free()
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,N,K,G", [(20, 200, 1024, 64), (64, 131, 2048, 32), (33, 128, 4096, 64), (50, 64, 768, 32)])
@pytest.mark.parametrize("bits", [4, 8])
def test_load_to_lds_tiles_on_4_kgroups(oracle, options, dt, M, N, K, G, bits):
    """The tilings of few rows (32 x 64 and 64 x 64 tiles on 4 K-groups, 256 k per iteration) with load-to-LDS
    activation tiles, unsplit and with K split over 1, 2 and 3 workgroups (f32 partial tiles added by the reduce
    kernel): the oracle's mma semantics (2e-2) and bit-equal to the register-staged instances."""
    c = make_case(5700 + M + K + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    options("qmm.kgroups", 4)
    for rows in (32, 64):
        for ksplit in (1, 2, 3):
            if ksplit > K // 256:
                continue
            print(f"[case] load-to-LDS qmm on 4 K-groups {dt.name} b{bits} M={M} N={N} K={K} g{G} tile_rows={rows} ksplit={ksplit}", flush=True)
            options("qmm.tile_rows", rows)
            options("qmm.ksplit", ksplit)
            res = {}
            for dma in (3, 1):
                options("qmm.dma", dma)
                out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
                cold()
                ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
                res[dma] = out.read_bytes()
                out.free()
            assert rel_err(unpack_f32(res[3], dt), exp) <= 2e-2, f"rows={rows} ksplit={ksplit}"
            assert res[3] == res[1], f"rows={rows} ksplit={ksplit}: differs from the register-staged instance"
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K,G", [(130, 200, 4096, 64),     # 32 iterations, ragged tiles both ways
                                     (257, 131, 2048, 32),     # N % 8 != 0
                                     (64, 128, 14336, 64),     # 112 iterations, 224 groups: whole rows would not fit beside 128-row tiles
                                     (300, 256, 3072, 128),    # 24 groups: splits share 8-group vectors of scales
                                     (96, 136, 11008, 64)])    # 172 groups: rows of scales are not whole vectors (staged by dwords)
def test_load_to_lds_tiles_with_k_split(oracle, options, dt, M, N, K, G, bits):
    """64 x 128 and 128 x 128 load-to-LDS tiles with K split over 2, 3 and 5 workgroups (f32 partial tiles added in
    split order by the reduce kernel; every split stages its own share of the scales): the oracle's mma semantics
    (2e-2), and the unsplit instance's result to within the rounding of the element type (the sums are the same
    terms added in another order)."""
    c = make_case(5800 + M + K + bits, dt, bits, G, M, N, K)
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    options("qmm.kernel", 2)
    options("qmm.kgroups", 2)
    for rows in (64, 128):
        options("qmm.tile_rows", rows)
        got = {}
        for ksplit in (1, 2, 3, 5):
            print(f"[case] K-split load-to-LDS qmm {dt.name} b{bits} M={M} N={N} K={K} g{G} tile_rows={rows} ksplit={ksplit}", flush=True)
            options("qmm.ksplit", ksplit)
            out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
            cold()
            ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
            got[ksplit] = unpack_f32(out.read_bytes(), dt)
            out.free()
            assert rel_err(got[ksplit], exp) <= 2e-2, f"rows={rows} ksplit={ksplit}"
            if ksplit > 1:
                scale = float(np.abs(got[1]).max())
                assert float(np.abs(got[ksplit] - got[1]).max()) <= (2.0 ** -7 if dt == DType.BF16 else 2.0 ** -10) * scale * 2
    for buf in (w, s, b, x):
        buf.free()
