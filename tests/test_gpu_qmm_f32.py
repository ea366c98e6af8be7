"""f32 batches on the f32 matrix-core kernel: every code width, ragged M and N, short and long rows,
against the f64-accumulated oracle within 1e-4 on max|a-e|/max(|e|,1) (the f32 bound of the other
f32 tests) for rows of up to 2048 codes and 2e-4 for 4096: every one of the K products is rounded to f32
and summed in f32, as on the reference's f32 MMA path (whose own bound is 5e-3 absolute,
quantized.rs:5449); measured worst case at K = 4096, 8-bit: 1.13e-4. The guard band after the output
must stay untouched."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, _lib, ops, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture
def f32_tiles():
    lib = _lib.load()

    def set_(value):
        assert lib.mtq_set_option(b"qmm.f32_tiles", value) == 0

    yield set_
    lib.mtq_set_option(b"qmm.f32_tiles", 0)


def _run(oracle, seed, bits, G, M, N, K, entry):
    dt = DType.F32
    c = make_case(seed, dt, bits, G, M, N, K, bias_rule="midpoint")
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, threads=8).astype(np.float32)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    guard = 1024
    out = GpuBuffer.from_bytes(np.full(M * N + guard, 0x7B7B7B7B, np.uint32).tobytes())
    entry(dt, bits, G, w, s, b, x, out, M, N, K)
    raw = np.frombuffer(out.read_bytes(), np.uint32)
    for buf in (w, s, b, x, out):
        buf.free()
    assert np.all(raw[M * N:] == 0x7B7B7B7B)
    got = raw[:M * N].view(np.float32)
    return rel_err(got, exp)


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("M,N,K,G", [(1, 40, 64, 32), (5, 200, 1024, 64), (33, 1001, 192, 64), (70, 256, 2048, 128),
                                     (32, 64, 4096, 64)])
def test_f32_tiles_all_widths(oracle, f32_tiles, bits, M, N, K, G):
    print(f"[case] f32 tiles b{bits} g{G} M{M} N{N} K{K}", flush=True)
    f32_tiles(2)
    tol = 1e-4 * max(1, K // 2048)
    assert _run(oracle, 9100 + bits + M, bits, G, M, N, K, ops.qmm) <= tol
    assert _run(oracle, 9200 + bits + M, bits, G, M, N, K, ops.qmv) <= tol


def test_f32_tiles_two_column_blocks_per_wave(oracle, f32_tiles):
    """Enough tiles for the wide variant (two 32-column blocks per wave), odd tile counts on both axes."""
    f32_tiles(2)
    M, N, K = 200, 5000, 256
    print(f"[case] f32 tiles wide M{M} N{N} K{K}", flush=True)
    assert _run(oracle, 9300, 4, 64, M, N, K, ops.qmm) <= 1e-4
    M, N, K = 2100, 200, 256  # activations larger than the weights: the other tile order
    print(f"[case] f32 tiles wide M{M} N{N} K{K}", flush=True)
    assert _run(oracle, 9301, 4, 64, M, N, K, ops.qmm) <= 1e-4


def test_f32_batches_route_by_rows(oracle, f32_tiles):
    """The default rule: up to 4 rows on the dot kernels, from 5 on the tiles; both within the bound, and a shape
    the tiles do not take (K not a multiple of 64) still runs."""
    for M in (4, 5, 16):
        assert _run(oracle, 9400 + M, 4, 64, M, 256, 1024, ops.qmm) <= 1e-4
    assert _run(oracle, 9410, 4, 32, 12, 64, 96, ops.qmm) <= 1e-4
    f32_tiles(1)
    assert _run(oracle, 9411, 4, 64, 12, 64, 1024, ops.qmm) <= 1e-4


@pytest.fixture
def grouped():
    lib = _lib.load()

    def set_(value):
        assert lib.mtq_set_option(b"gather.grouped", value) == 0

    yield set_
    lib.mtq_set_option(b"gather.grouped", 0)


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_f32_grouped_gather_both_views(oracle, grouped, bits):
    """f32 rows routed to experts, grouped into 32-row tiles: CSR offsets (with an empty expert, an
    expert of more than one tile and a tail past the last offset, which belongs to expert 0) and shuffled
    per-row ids (three of them naming no expert: those output rows must stay untouched)."""
    dt, E, N, K, G = DType.F32, 5, 72, 512, 64
    counts = [40, 0, 70, 3, 32]
    T = sum(counts) + 6  # 6 tail rows
    c = make_case(9500 + bits, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype("<u4")
    ids_csr = np.concatenate([np.repeat(np.arange(E), counts), np.zeros(6, np.int64)]).astype("<u4")
    rng = np.random.default_rng(bits)
    ids = rng.permutation(ids_csr).astype("<u4")
    bad = np.array([7, 50, 100])
    ids[bad] = [E, E + 3, 0xFFFFFFFF]
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    grouped(2)
    for view, route, fn, rows_ids in (("csr", offsets, ops.gather_qmv_csr, ids_csr), ("indices", ids, ops.gather_qmv_indices, ids)):
        print(f"[case] f32 grouped gather {view} b{bits}", flush=True)
        valid = rows_ids < E
        exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G,
                                indices=np.where(valid, rows_ids, 0).astype("<u4"), f64=True, threads=8)
        exp = np.asarray(exp, np.float32).reshape(T, N)
        out = GpuBuffer.from_bytes(np.full(T * N + 256, 0x7B7B7B7B, np.uint32).tobytes())
        r = GpuBuffer.from_bytes(route.tobytes())
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        raw = np.frombuffer(out.read_bytes(), np.uint32)
        out.free(); r.free()
        assert np.all(raw[T * N:] == 0x7B7B7B7B), view
        got = raw[:T * N].view(np.float32).reshape(T, N)
        assert np.all(raw[:T * N].reshape(T, N)[~valid] == 0x7B7B7B7B), view
        assert rel_err(got[valid].reshape(-1), exp[valid].reshape(-1)) <= 1e-4, view
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("mode", [0, 1])
def test_f32_gather_default_rule(oracle, grouped, mode):
    """Without the option f32 rows go grouped at any number of rows per expert; with the option at 1 they
    stay on the dot kernels. Both within the bound."""
    dt, bits, E, N, K, G = DType.F32, 4, 4, 64, 256, 64
    grouped(mode)
    for per in (2, 12):
        T = per * E
        c = make_case(9600 + per, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
        ids = np.repeat(np.arange(E), per).astype("<u4")
        exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=ids, f64=True, threads=8)
        w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                      GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
        out = GpuBuffer(T * N * 4)
        r = GpuBuffer.from_bytes(ids.tobytes())
        ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = np.frombuffer(out.read_bytes(), np.float32)
        assert rel_err(got, np.asarray(exp, np.float32).reshape(-1)) <= 1e-4
        for buf in (w, s, b, x, out, r):
            buf.free()


@pytest.mark.parametrize("ks", [0, 1, 3, 8])
def test_f32_tiles_split_k(oracle, f32_tiles, ks):
    """Few tiles and long rows: K is cut into splits (chosen, off, forced to counts that do and do not divide
    the 64 steps of K = 4096) whose partial tiles a second kernel adds in order; ragged M and N."""
    lib = _lib.load()
    f32_tiles(2)
    assert lib.mtq_set_option(b"qmm.ksplit", ks) == 0
    try:
        for bits, G in ((4, 64), (3, 128)):
            print(f"[case] f32 tiles split-K ks={ks} b{bits}", flush=True)
            assert _run(oracle, 9900 + ks + bits, bits, G, 20, 72, 4096, ops.qmm) <= 2e-4
    finally:
        lib.mtq_set_option(b"qmm.ksplit", 0)
