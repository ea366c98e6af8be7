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
