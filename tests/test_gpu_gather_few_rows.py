"""gather_qmv with fewer rows than experts (a decode step of a mixture-of-experts layer: one or two tokens, top-k):
the launch has one grid row per activation row and each grid row finds the expert it serves on the device, instead
of one grid row per expert most of which find no row. Both routing views against the gather oracle
(crates/metaltile-std/src/ffai/moe.rs:3577-3622), 1e-2 on max|a-e| / max(|e|, 1) for f16 / bf16; more than 64
experts (the scan walks them in chunks of 64), rows that name the same expert, CSR offsets that leave rows past the
last offset to expert 0 (moe.rs:376-385), offsets that step back, and ids that name no expert."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, _lib, ops, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F16: 1, DType.BF16: 2}


def _offsets(ids, E):
    return np.concatenate([[0], np.cumsum(np.bincount(ids, minlength=E))]).astype("<u4")


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("E,ids", [(8, [3]), (8, [1, 6]), (8, [0, 7]), (8, [4, 4]), (64, [0, 63]), (8, [2, 2, 5]), (8, [0, 1, 2, 3, 4, 5, 6]),
                                   (130, [0, 63, 64, 65, 128, 129]), (130, [129]), (70, [64, 64, 64, 69]),
                                   (40, list(range(4, 36))), (130, list(range(0, 130, 5)))],
                         ids=lambda v: str(v) if isinstance(v, int) else "-".join(map(str, v[:6])))
@pytest.mark.parametrize("K", [1024, 2048])
def test_fewer_rows_than_experts(oracle, dt, E, ids, K):
    bits, G, N = 4, 64, 264
    T = len(ids)
    idn = np.array(ids, dtype="<u4")
    c = make_case(8400 + E + T + K, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=idn, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt]).reshape(T, N)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    for view, route, fn in (("csr", _offsets(idn, E), ops.gather_qmv_csr), ("indices", idn, ops.gather_qmv_indices)):
        print(f"[case] few-row gather {view} {dt.name} E{E} ids={ids}", flush=True)
        rc, launches, _, n = ops.plan("gather_" + view, dt, bits, G, 1, N, K, E, T)
        # up to eight rows on rows of 2048 codes: the kernel whose waves walk the rows, a grid row per expert that has a row;
        # otherwise the matrix-core GEMV
        # (and up to 32 rows on at least twice as many small experts)
        kernel = "qmv_rows_walk_routed_kernel" if (T <= 8 or (T <= 32 and E >= 2 * T)) and K == 2048 else "qmv_mfma_kernel"
        assert rc == 0 and n == 1 and kernel in launches[0][0] and launches[0][1][1] == T, launches
        out, r = GpuBuffer.from_bytes(b"\xff" * (T * N * dt.size_bytes)), GpuBuffer.from_bytes(route.tobytes())
        fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), dt).reshape(T, N)
        assert rel_err(got.reshape(-1), exp.reshape(-1)) <= 1e-2, view
        out.free(); r.free()
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
def test_fewer_rows_than_experts_odd_routing(oracle, dt):
    """Offsets that end short (the last rows go to expert 0), offsets that step back (a later, smaller offset gives its
    expert no row), and per-row ids that name no expert (those output rows keep their bytes)."""
    bits, G, N, K, E, T = 4, 64, 132, 512, 9, 5
    c = make_case(8500, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))

    def run_csr(off, ids_equiv, label):
        exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=np.array(ids_equiv, dtype="<u4"),
                                f64=True, threads=8)
        exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
        via_offsets = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G,
                                        expert_offsets=np.array(off, dtype="<u4"), f64=True, threads=8)
        assert np.array_equal(oracle.round_through(via_offsets.astype(np.float32), ODT[dt]), exp), label   # the rule, as the oracle reads it
        print(f"[case] few-row gather csr {dt.name} {label} off={off}", flush=True)
        out, r = GpuBuffer(T * N * dt.size_bytes), GpuBuffer.from_bytes(np.array(off, dtype="<u4").tobytes())
        ops.gather_qmv_csr(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        assert rel_err(unpack_f32(out.read_bytes(), dt), exp) <= 1e-2, label
        out.free(); r.free()

    #        e: 0  1  2  3  4  5  6  7  8
    run_csr([0, 0, 0, 2, 2, 2, 2, 3, 3, 3], [2, 2, 6, 0, 0], "tail to expert 0")
    run_csr([0, 1, 1, 3, 2, 2, 4, 4, 4, 5], [0, 2, 2, 5, 8], "an offset that steps back")
    ids = np.array([7, E + 1, 7, 0xFFFFFFFF, 2], dtype="<u4")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=np.array([7, 0, 7, 0, 2], dtype="<u4"),
                            f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt]).reshape(T, N)
    print(f"[case] few-row gather indices {dt.name} nameless ids", flush=True)
    out, r = GpuBuffer.from_bytes(b"\xab" * (T * N * dt.size_bytes)), GpuBuffer.from_bytes(ids.tobytes())
    ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
    raw = out.read_bytes()
    got = unpack_f32(raw, dt).reshape(T, N)
    rb = N * dt.size_bytes
    for t in (1, 3):
        assert raw[t * rb:(t + 1) * rb] == b"\xab" * rb
    for t in (0, 2, 4):
        assert rel_err(got[t], exp[t]) <= 1e-2
    for buf in (w, s, b, x, out, r):
        buf.free()


@pytest.fixture
def prefer_streaming():
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 2) == 0
    yield
    lib.mtq_set_option(b"qmv.kernel", 0)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
def test_two_rows_on_the_one_row_kernel(oracle, dt, prefer_streaming):
    """The one-row streaming kernel serves routed rows one at a time, each grid row once per row of its expert. It is
    chosen for one row; asked for by option it takes two, which is what runs its second pass: offsets that end short,
    offsets that step back, an id that names no expert, the same expert for both rows, two experts."""
    bits, G, N, K, E, T = 4, 64, 132, 2048, 9, 2
    c = make_case(8600, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))

    def expect(ids_equiv):
        e = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=np.array(ids_equiv, dtype="<u4"),
                              f64=True, threads=8)
        return oracle.round_through(e.astype(np.float32), ODT[dt]).reshape(T, N)

    #                      e: 0  1  2  3  4  5  6  7  8
    for off, ids_equiv, label in (([0, 0, 0, 0, 1, 1, 1, 1, 1, 1], [3, 0], "tail to expert 0"),
                                  ([0, 0, 0, 0, 0, 0, 0, 0, 0, 0], [0, 0], "every row in the tail"),
                                  ([0, 0, 2, 1, 1, 1, 1, 1, 1, 1], [1, 1], "an offset that steps back"),
                                  ([0, 0, 1, 1, 1, 1, 1, 2, 2, 2], [1, 6], "two experts"),
                                  ([0, 0, 0, 0, 0, 0, 0, 0, 0, 2], [8, 8], "both rows on the last expert")):
        via_offsets = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G,
                                        expert_offsets=np.array(off, dtype="<u4"), f64=True, threads=8)
        exp = expect(ids_equiv)
        assert np.array_equal(oracle.round_through(via_offsets.astype(np.float32), ODT[dt]).reshape(T, N), exp), label
        print(f"[case] two-row gather csr {dt.name} {label} off={off}", flush=True)
        _, launches, _, _ = ops.plan("gather_csr", dt, bits, G, 1, N, K, E, T)
        assert "qmv_stream_kernel" in launches[0][0] and launches[0][1][1] == T, launches
        out, r = GpuBuffer(T * N * dt.size_bytes), GpuBuffer.from_bytes(np.array(off, dtype="<u4").tobytes())
        ops.gather_qmv_csr(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        assert rel_err(unpack_f32(out.read_bytes(), dt), exp.reshape(-1)) <= 1e-2, label
        out.free(); r.free()
    rb = N * dt.size_bytes
    for ids, kept in (([E + 1, 4], 0), ([6, 0xFFFFFFFF], 1), ([5, 5], None), ([7, 2], None)):
        print(f"[case] two-row gather indices {dt.name} ids={ids}", flush=True)
        exp = expect([i if i < E else 0 for i in ids])
        out, r = GpuBuffer.from_bytes(b"\xab" * (T * rb)), GpuBuffer.from_bytes(np.array(ids, dtype="<u4").tobytes())
        ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        raw = out.read_bytes()
        got = unpack_f32(raw, dt).reshape(T, N)
        for t in range(T):
            if t == kept:
                assert raw[t * rb:(t + 1) * rb] == b"\xab" * rb, ids
            else:
                assert rel_err(got[t], exp[t]) <= 1e-2, ids
        out.free(); r.free()
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("K", [1024, 1536, 2048])
def test_one_routed_row_on_rows_the_streaming_kernel_cannot_tile(oracle, dt, K):
    """One routed row: rows of 2048 codes take the routed kernel whose waves walk the rows; shorter or ragged rows
    (K = 1024, 1536) must land on a gather instance of the tiled kernels, not on the one-wave-per-output fallback, and
    give the same answer either way."""
    bits, G, N, E, T = 4, 64, 264, 8, 1
    c = make_case(8700 + K, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    for view in ("csr", "indices"):
        rc, launches, _, _ = ops.plan("gather_" + view, dt, bits, G, 1, N, K, E=E, T=T)
        assert rc == 0
        name = launches[0][0]
        assert "generic" not in name, name
        assert ("qmv_rows_walk_routed_kernel" in name) == (K == 2048), name
    ids = np.array([5], dtype="<u4")
    exp = oracle.round_through(oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=ids, f64=True, threads=8)
                               .astype(np.float32), ODT[dt])
    out, r = GpuBuffer(T * N * dt.size_bytes), GpuBuffer.from_bytes(ids.tobytes())
    ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
    assert rel_err(unpack_f32(out.read_bytes(), dt), exp) <= 1e-2
    off = GpuBuffer.from_bytes(np.array([0, 0, 0, 0, 0, 0, 1, 1, 1], dtype="<u4").tobytes())   # the row belongs to expert 5
    out.zero()
    ops.gather_qmv_csr(dt, bits, G, x, w, s, b, off, out, T, N, K, E)
    assert rel_err(unpack_f32(out.read_bytes(), dt), exp) <= 1e-2
    for buf in (w, s, b, x, out, r, off):
        buf.free()


@pytest.fixture
def forced_qmv_kernel(request):
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", request.param) == 0
    yield
    lib.mtq_set_option(b"qmv.kernel", 0)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("N,K,kernel,forced_qmv_kernel",
                         [(20, 4096, "qmv_rows_routed_kernel", 3), (1028, 4096, "qmv_rows_routed_kernel", 3), (19, 14336, "qmv_rows_long_routed_kernel", 3),
                          (1030, 8192, "qmv_rows_long_routed_kernel", 3),
                          # the kernel whose waves walk the rows (qmv.kernel = 4): one row per wave, and 5000 rows so that waves walk
                          (20, 4096, "qmv_rows_walk_routed_kernel", 4), (5000, 4096, "qmv_rows_walk_routed_kernel", 4), (1030, 8192, "qmv_rows_walk_routed_kernel", 4),
                          # the expert widths of other models: 2048 codes, and rows that end inside a group of 64 chunks
                          (1030, 2048, "qmv_rows_walk_routed_kernel", 4), (40, 7168, "qmv_rows_walk_routed_ragged_kernel", 4), (2050, 5120, "qmv_rows_walk_routed_ragged_kernel", 4),
                          (1027, 6144, "qmv_rows_walk_routed_kernel", 4)],
                         indirect=["forced_qmv_kernel"])
def test_routed_rows_on_the_wave_per_row_kernels(oracle, dt, N, K, kernel, forced_qmv_kernel):
    """The wave-per-row GEMV kernels with a grid row per expert that has a row (their automatic range is up to four rows
    on fewer rows than experts from 1024 weight rows; forced here below that too): one row, two experts, the same expert
    twice (a second pass over its matrix), seven rows, both routing views, CSR offsets that end short or step back, ids
    that name no expert (those output rows keep their bytes), ragged last workgroups, behind a cache flush."""
    import metaltile_amd as m
    bits, G, E = 4, 64, 8
    rb = N * dt.size_bytes
    for ids in ([3], [1, 6], [4, 4], [2, 2, 5], [0, 1, 2, 3, 4, 5, 7]):
        T = len(ids)
        idn = np.array(ids, dtype="<u4")
        c = make_case(8700 + N + K + T, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
        exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=idn, f64=True, threads=8)
        exp = oracle.round_through(exp.astype(np.float32), ODT[dt]).reshape(T, N)
        w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                      GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
        for view, route, fn in (("csr", _offsets(idn, E), ops.gather_qmv_csr), ("indices", idn, ops.gather_qmv_indices)):
            print(f"[case] routed rows {view} {dt.name} N{N} K{K} ids={ids}", flush=True)
            rc, launches, _, n = ops.plan("gather_" + view, dt, bits, G, 1, N, K, E, T)
            assert rc == 0 and n == 1 and kernel in launches[0][0] and launches[0][1][1] == T, launches
            out, r = GpuBuffer.from_bytes(b"\xab" * (T * rb + 64)), GpuBuffer.from_bytes(route.tobytes())
            m.GpuRunner(0).flush_slc()
            fn(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
            raw = out.read_bytes()
            assert raw[T * rb:] == b"\xab" * 64
            assert rel_err(unpack_f32(raw[:T * rb], dt), exp.reshape(-1)) <= 1e-2, view
            out.free(); r.free()
        if T == 3:
            # the same rows under offsets that end short (the last row goes to expert 0) and offsets that step back
            #                      e: 0  1  2  3  4  5  6  7
            for off, ids_equiv, label in (([0, 0, 0, 2, 2, 2, 2, 2, 2], [2, 2, 0], "tail to expert 0"),
                                          ([0, 1, 1, 3, 2, 2, 3, 3, 3], [0, 2, 2], "an offset that steps back")):
                e2 = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=np.array(ids_equiv, dtype="<u4"),
                                       f64=True, threads=8)
                e2 = oracle.round_through(e2.astype(np.float32), ODT[dt])
                via = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, expert_offsets=np.array(off, dtype="<u4"),
                                        f64=True, threads=8)
                assert np.array_equal(oracle.round_through(via.astype(np.float32), ODT[dt]), e2), label   # the rule, as the oracle reads it
                print(f"[case] routed rows csr {dt.name} N{N} K{K} {label}", flush=True)
                out, r = GpuBuffer(T * rb), GpuBuffer.from_bytes(np.array(off, dtype="<u4").tobytes())
                ops.gather_qmv_csr(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
                assert rel_err(unpack_f32(out.read_bytes(), dt), e2) <= 1e-2, label
                out.free(); r.free()
            nameless = np.array([7, E + 1, 2], dtype="<u4")
            e3 = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=np.array([7, 0, 2], dtype="<u4"), f64=True, threads=8)
            e3 = oracle.round_through(e3.astype(np.float32), ODT[dt]).reshape(T, N)
            print(f"[case] routed rows indices {dt.name} N{N} K{K} an id that names no expert", flush=True)
            out, r = GpuBuffer.from_bytes(b"\xab" * (T * rb)), GpuBuffer.from_bytes(nameless.tobytes())
            ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
            raw = out.read_bytes()
            assert raw[rb:2 * rb] == b"\xab" * rb
            got = unpack_f32(raw, dt).reshape(T, N)
            assert rel_err(got[0], e3[0]) <= 1e-2 and rel_err(got[2], e3[2]) <= 1e-2
            out.free(); r.free()
        for buf in (w, s, b, x):
            buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("N,K,kernel,forced_qmv_kernel",
                         [(1028, 4096, "qmv_rows_routed_kernel", 3), (40, 14336, "qmv_rows_long_routed_kernel", 3), (1030, 8192, "qmv_rows_long_routed_kernel", 3),
                          (9000, 4096, "qmv_rows_walk_routed_kernel", 4), (40, 8192, "qmv_rows_walk_routed_kernel", 4),
                          (1030, 7168, "qmv_rows_walk_routed_ragged_kernel", 4), (768, 2048, "qmv_rows_walk_routed_kernel", 4)], indirect=["forced_qmv_kernel"])
def test_single_index_expert_on_the_wave_per_row_kernels(oracle, dt, N, K, kernel, forced_qmv_kernel):
    """One row against the expert whose index is read on the device (the reference's expert-indexed GEMV,
    crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs): the first, a middle and the last expert, and an index
    past the last expert, which names the last one as in the other kernels of this ABI."""
    import metaltile_amd as m
    bits, G, E = 4, 64, 6
    c = make_case(8800 + N + K, dt, bits, G, 1, N, K, E=E, bias_rule="midpoint")
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    rb = N * dt.size_bytes
    for idx in (0, 3, E - 1, E + 7):
        e = min(idx, E - 1)
        exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, 1, K, N, E, bits, G, indices=np.array([e], dtype="<u4"), f64=True, threads=8)
        exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
        print(f"[case] single-index expert {dt.name} N{N} K{K} index {idx}", flush=True)
        rc, launches, _, n = ops.plan("gather_single", dt, bits, G, 1, N, K, E, 1)
        assert rc == 0 and n == 1 and kernel in launches[0][0] and launches[0][1][1] == 1, launches
        out, ei = GpuBuffer.from_bytes(b"\xab" * (rb + 64)), GpuBuffer.from_bytes(np.array([idx], dtype="<u4").tobytes())
        m.GpuRunner(0).flush_slc()
        ops.gather_qmv_single(dt, bits, G, w, s, b, x, ei, out, N, K, E)
        raw = out.read_bytes()
        assert raw[rb:] == b"\xab" * 64
        assert rel_err(unpack_f32(raw[:rb], dt), exp) <= 1e-2, idx
        out.free(); ei.free()
    for buf in (w, s, b, x):
        buf.free()


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16], ids=lambda d: d.name)
@pytest.mark.parametrize("N,K,kernel", [(1030, 2048, "qmv_rows_walk_routed_kernel"), (520, 7168, "qmv_rows_walk_routed_ragged_kernel")])
def test_routed_walk_with_more_than_64_experts(oracle, dt, N, K, kernel):
    """Any number of experts under both routing views (up to 64 the offsets are read by one wave-wide load, beyond that
    scanned 64 at a time): 130 experts, rows on experts beyond the 64th, one expert named twice, an id that names no
    expert (its output row keeps its bytes). Forced with qmv.kernel = 4, behind a cache flush, against the f64 oracle."""
    import metaltile_amd as m
    bits, G, E = 4, 64, 130
    ids = [129, 3, 64, 129, 131]
    T = len(ids)
    idn = np.array(ids, dtype="<u4")
    valid = np.array([129, 3, 64, 129, 0], dtype="<u4")
    rb = N * dt.size_bytes
    print(f"[case] routed walk, 130 experts, ids {dt.name} N{N} K{K}", flush=True)
    c = make_case(8800 + N + K, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    exp = oracle.gather_qmm(c.x_f, c.w, c.scales_f, c.biases_f, T, K, N, E, bits, G, indices=valid, f64=True, threads=8)
    exp = oracle.round_through(exp.astype(np.float32), ODT[dt]).reshape(T, N)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    lib = _lib.load()
    assert lib.mtq_set_option(b"qmv.kernel", 4) == 0
    try:
        rc, launches, _, n = ops.plan("gather_indices", dt, bits, G, 1, N, K, E, T)
        assert rc == 0 and n == 1 and kernel in launches[0][0] and launches[0][1][1] == T, launches
        out, r = GpuBuffer.from_bytes(b"\xab" * (T * rb + 64)), GpuBuffer.from_bytes(idn.tobytes())
        m.GpuRunner(0).flush_slc()
        ops.gather_qmv_indices(dt, bits, G, x, w, s, b, r, out, T, N, K, E)
        # the offsets view of four sorted rows on the same experts (its offsets are scanned 64 at a time beyond 64 experts)
        srt = np.array([3, 64, 129, 129], dtype="<u4")
        rc, launches, _, n = ops.plan("gather_csr", dt, bits, G, 1, N, K, E, 4)
        assert rc == 0 and n == 1 and kernel in launches[0][0] and launches[0][1][1] == 4, launches
        e4 = oracle.gather_qmm(c.x_f[:4 * K], c.w, c.scales_f, c.biases_f, 4, K, N, E, bits, G, indices=srt, f64=True, threads=8)
        e4 = oracle.round_through(e4.astype(np.float32), ODT[dt])
        out4, r4 = GpuBuffer.from_bytes(b"\xab" * (4 * rb + 64)), GpuBuffer.from_bytes(_offsets(srt, E).tobytes())
        ops.gather_qmv_csr(dt, bits, G, x, w, s, b, r4, out4, 4, N, K, E)
        raw4 = out4.read_bytes()
        assert raw4[4 * rb:] == b"\xab" * 64
        assert rel_err(unpack_f32(raw4[:4 * rb], dt), e4.reshape(-1)) <= 1e-2
        out4.free(); r4.free()
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_bytes()
    assert raw[T * rb:] == b"\xab" * 64
    assert raw[4 * rb:5 * rb] == b"\xab" * rb          # the row whose id names no expert
    got = unpack_f32(raw[:4 * rb], dt).reshape(4, N)
    for t in range(4):
        assert rel_err(got[t], exp[t]) <= 1e-2, t
    for buf in (w, s, b, x, out, r):
        buf.free()
