"""The 16-row matrix-core GEMV (qmv_wide_kernel: 4-bit codes, f16 / bf16, batches of up to 16 rows on the
16x16x32 MFMA), forced through the library's option on shapes that exercise every branch of its geometry, against
the f64-accumulated oracle of the exact-dequant form (out = sum_g s * sum q x + b * sum x, the arithmetic of the
reference's mt_qmm, crates/metaltile-std/src/mlx/quantized.rs:1330-1500). Tolerance on max|a-e|/max(|e|,1): 1e-2
for f16 / bf16, the benchmark configurations' bound."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, _lib, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F16: 1, DType.BF16: 2}


def pack_f32_rows(rows, dt):
    return pack_f32(np.ascontiguousarray(rows, dtype=np.float32).reshape(-1), dt)


@pytest.fixture
def wide():
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.wide", 2) == 0

    def geometry(kp, nb):
        assert lib.mtq_set_option(b"qmv.wide_kp", kp) == 0 and lib.mtq_set_option(b"qmv.wide_nb", nb) == 0

    yield geometry
    for name in (b"qmv.wide", b"qmv.wide_kp", b"qmv.wide_nb"):
        lib.mtq_set_option(name, 0)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,N,K,G", [(16, 512, 1024, 64),     # two turns per row block, every wave of two workgroups busy
                                     (5, 100, 512, 64),       # one turn (odd total), ragged last row block, rows 5..15 repeated
                                     (9, 4100, 1536, 32),     # three turns, groups of 32: a group per MFMA; 257 row blocks
                                     (13, 333, 2048, 128),    # groups of 128: 8-byte scale loads
                                     (16, 40, 5120, 64),      # ten turns: K split in two slices of five (f32 partial rows)
                                     (7, 8200, 14336, 64),    # 28 turns in four slices of seven; several row blocks per wave
                                     (12, 70000, 512, 128)])  # 4375 row blocks: waves walk up to two blocks of one turn each
@pytest.mark.parametrize("kp,nb", [(0, 0), (1, 2), (4, 1), (16, 2)], ids=lambda v: str(v))
def test_wide_gemv(oracle, wide, dt, M, N, K, G, kp, nb):
    """kp, nb: waves that share a row block (each with a run of the turns; their sums meet in LDS) and row blocks
    per wave, chosen by the library (0, 0) or forced."""
    bits = 4
    wide(kp, nb)
    c = make_case(6100 + M + N % 97, dt, bits, G, M, N, K, bias_rule="midpoint")
    print(f"[case] wide qmv {dt.name} g{G} M{M} N{N} K{K} kp={kp} nb={nb}", flush=True)
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, bits, G, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
    assert _lib.load().mtq_flush_cache() == 0   # cold operands: hand-counted waits must not rely on data arriving early
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), dt)
    assert rel_err(got, exp) <= 1e-2
    for buf in (w, s, b, x, out):
        buf.free()


def test_wide_gemv_is_the_kernel_that_ran(wide):
    """The forced route is the wide kernel (a K split adds its reduce kernel), and shapes outside its limits fall
    through to the other kernels instead of failing."""
    rc, launches, scratch, n = ops.plan("qmm", DType.BF16, 4, 64, 16, 8192, 4096)
    assert rc == 0 and n == 1 and "qmv_wide_kernel<2, 64, " in launches[0][0] and launches[0][2][0] == 1024
    rc, launches, scratch, n = ops.plan("qmm", DType.F16, 4, 32, 9, 8192, 8192)
    assert rc == 0 and n == 2 and "qmv_wide_kernel<1, 32, 1, 1, 0>" in launches[0][0] and "qmv_wide_reduce_kernel" in launches[1][0]
    assert launches[0][1][1] == 2 and scratch >= 2 * 9 * 8192 * 4   # groups of 32: a wave keeps at most 4 turns of scales in registers
    for args in ((DType.BF16, 8, 64, 16, 8192, 4096), (DType.BF16, 4, 64, 16, 8192, 4352), (DType.BF16, 4, 64, 17, 8192, 4096)):
        rc, launches, _, n = ops.plan("qmm", *args)
        assert rc == 0 and all("qmv_wide" not in l[0] for l in launches)


@pytest.fixture
def wide_gather():
    lib = _lib.load()
    assert lib.mtq_set_option(b"gather.wide", 2) == 0

    def geometry(kp, nb):
        assert lib.mtq_set_option(b"qmv.wide_kp", kp) == 0 and lib.mtq_set_option(b"qmv.wide_nb", nb) == 0

    yield geometry
    for name in (b"gather.wide", b"qmv.wide_kp", b"qmv.wide_nb"):
        lib.mtq_set_option(name, 0)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("kp,nb", [(0, 0), (1, 2), (4, 1), (16, 2)], ids=lambda v: str(v))
@pytest.mark.parametrize("N,K,counts", [(200, 1024, [3, 0, 11, 1, 8]),          # an empty expert, ragged row blocks
                                        (1040, 4096, [6, 2, 4, 4, 5, 2, 5, 4]),  # the benchmark's routing on shorter experts
                                        (64, 512, [40, 1, 0, 17]),              # more than 16 rows: three passes, two passes
                                        (4096, 1536, [16, 16])])                # whole passes, three turns
def test_wide_gather(oracle, wide_gather, dt, N, K, counts, kp, nb):
    """Expert-routed rows on the 16-row matrix-core GEMV (forced with gather.wide = 2), both routing views, rows of an
    expert worked 16 per pass; CSR offsets that leave a tail (rows past the last offset belong to expert 0 in the
    reference) and per-row ids in any order, some naming no expert (their output rows stay untouched)."""
    bits, G, E = 4, 64, len(counts)
    T = sum(counts)
    wide_gather(kp, nb)
    c = make_case(6300 + N + K % 91, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    indices = np.repeat(np.arange(E), counts).astype("<u4")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype("<u4")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=indices, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt]).reshape(T, N)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    lib = _lib.load()
    for view, route, fn in (("csr", offsets, ops.gather_qmv_csr), ("indices", indices, ops.gather_qmv_indices)):
        print(f"[case] wide gather {view} {dt.name} N{N} K{K} counts={counts} kp={kp} nb={nb}", flush=True)
        rc, launches, _, n = ops.plan("gather_" + view, dt, bits, G, 1, N, K, E, T)
        assert rc == 0 and n == 1 and "qmv_wide_kernel" in launches[0][0], launches
        out = GpuBuffer.from_bytes(b"\xff" * (T * N * dt.size_bytes))
        r = GpuBuffer.from_bytes(route.tobytes())
        assert lib.mtq_flush_cache() == 0
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), dt).reshape(T, N)
        assert rel_err(got.reshape(-1), exp.reshape(-1)) <= 1e-2, view
        out.free(); r.free()
    # CSR offsets that stop short: the rows past the last offset belong to expert 0 (crates/metaltile-std/src/ffai/moe.rs:376-385)
    if counts[-1] > 1:
        short = offsets.copy()
        short[-1] -= 1
        ids_tail = indices.copy()
        ids_tail[-1] = 0
        exp_t = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=ids_tail, f64=True, threads=8)
        exp_t = oracle.round_through(exp_t.astype(np.float32), ODT[dt])
        out, r = GpuBuffer(T * N * dt.size_bytes), GpuBuffer.from_bytes(short.tobytes())
        ops.gather_qmv_csr(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        assert rel_err(unpack_f32(out.read_bytes(), dt), exp_t) <= 1e-2, "csr tail"
        out.free(); r.free()
    # per-row ids in another order, the first row naming no expert: its output row keeps its bytes
    perm = np.random.default_rng(T).permutation(T)
    ids_p = indices[perm].astype("<u4")
    ids_p[0] = E + 3
    xb = GpuBuffer.from_bytes(pack_f32_rows(c.x_f.reshape(T, K)[perm], dt))
    out, r = GpuBuffer.from_bytes(b"\xab" * (T * N * dt.size_bytes)), GpuBuffer.from_bytes(ids_p.tobytes())
    ops.gather_qmv_indices(dt, bits, G, xb, w, s, b, r, out, T, N, K, E)
    raw = out.read_bytes()
    got = unpack_f32(raw, dt).reshape(T, N)
    assert raw[: N * dt.size_bytes] == b"\xab" * (N * dt.size_bytes)
    assert rel_err(got[1:].reshape(-1), exp[perm][1:].reshape(-1)) <= 1e-2, "permuted ids"
    for buf in (w, s, b, x, xb, r, out):
        buf.free()
