"""Size-independent properties of the HIP path at full benchmark sizes, plus
edge cases (empty and ragged shapes, odd bit widths, fallback geometry)."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case, pack_codes
from tests.parity import rel_err

pytestmark = pytest.mark.gpu


def _run(dt, bits, G, w, s_f, b_f, x_f, M, N, K, entry=ops.qmv):
    bw, bs, bb = GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s_f, dt)), GpuBuffer.from_bytes(pack_f32(b_f, dt))
    bx = GpuBuffer.from_bytes(pack_f32(x_f, dt))
    out = GpuBuffer(max(M * N, 1) * dt.size_bytes)
    entry(dt, bits, G, bw, bs, bb, bx, out, M, N, K)
    got = unpack_f32(out.read_bytes(M * N * dt.size_bytes), dt)
    for buf in (bw, bs, bb, bx, out):
        buf.free()
    return got


def test_zero_codes_closed_form_full_size():
    """All codes 0 -> y[n] = sum_g b[n,g] * sum_{k in g} x[k], at 14336x4096 bf16."""
    N, K, G = 14336, 4096, 64
    print("[case] zero codes closed form", flush=True)
    c = make_case(11, DType.BF16, 4, G, 1, N, K)
    w0 = np.zeros_like(c.w)
    got = _run(DType.BF16, 4, G, w0, c.scales_f, c.biases_f, c.x_f, 1, N, K)
    xg = c.x_f.reshape(K // G, G).astype(np.float64).sum(axis=1)
    want = c.biases_f.reshape(N, K // G).astype(np.float64) @ xg
    assert rel_err(got, want) <= 1e-2


def test_unit_scale_constant_code_full_size():
    """scale 1, bias 0, every code c -> y = c * sum(x), f32 at 4096x4096 for each width."""
    N, K, G = 4096, 4096, 64
    rng = np.random.default_rng(12)
    x = rng.standard_normal(K).astype(np.float32)
    for bits, cval in ((2, 3), (4, 11), (8, 201)):
        print(f"[case] constant code b{bits}", flush=True)
        w = pack_codes(np.full((N, K), cval, np.uint8), bits)
        ones, zeros = np.ones(N * K // G, np.float32), np.zeros(N * K // G, np.float32)
        got = _run(DType.F32, bits, G, w, ones, zeros, x, 1, N, K)
        want = cval * float(x.astype(np.float64).sum())
        assert np.max(np.abs(got - want)) <= 1e-4 * max(abs(want), 1.0) + 2e-3


def test_linearity_full_size():
    N, K, G = 4096, 14336, 64
    print("[case] linearity", flush=True)
    c = make_case(13, DType.F32, 4, G, 2, N, K)
    x1, x2 = c.x_f[:K], c.x_f[K:]
    y1 = _run(DType.F32, 4, G, c.w, c.scales_f, c.biases_f, x1, 1, N, K).astype(np.float64)
    y2 = _run(DType.F32, 4, G, c.w, c.scales_f, c.biases_f, x2, 1, N, K).astype(np.float64)
    y = _run(DType.F32, 4, G, c.w, c.scales_f, c.biases_f, (2.0 * x1 - 0.5 * x2).astype(np.float32), 1, N, K)
    assert rel_err(y, 2.0 * y1 - 0.5 * y2) <= 1e-4


@pytest.mark.parametrize("M", [2, 3, 4, 7])
def test_batched_rows_equal_single_rows(M):
    """Row m of an M-row launch == the M=1 launch on x[m] (tests/qmm_gpu_correctness.rs:341),
    up to one bf16 ulp: the two instantiations may contract their FMAs differently."""
    N, K, G = 4096, 4096, 64
    print(f"[case] batched rows M={M}", flush=True)
    c = make_case(14 + M, DType.BF16, 4, G, M, N, K)
    got = _run(DType.BF16, 4, G, c.w, c.scales_f, c.biases_f, c.x_f, M, N, K).reshape(M, N)
    for mrow in range(M):
        one = _run(DType.BF16, 4, G, c.w, c.scales_f, c.biases_f, c.x_f[mrow * K:(mrow + 1) * K], 1, N, K)
        assert rel_err(got[mrow], one) <= 2.0 ** -7


def test_qmm_rows_match_qmv_within_tolerance():
    """M=2048 prefill (too large for the CPU oracle in this suite): every 64th row
    against the M=1 GEMV path, which is itself checked against the oracle. The
    MFMA path rounds dequantised weights to bf16 as the reference's mma kernels do,
    so the bound is the reference's bf16 one (tests/qmm_gpu_correctness.rs:2085-2106)."""
    M, N, K, G = 2048, 4096, 4096, 64
    print("[case] qmm M=2048 vs qmv rows", flush=True)
    c = make_case(15, DType.BF16, 4, G, M, N, K)
    got = _run(DType.BF16, 4, G, c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, entry=ops.qmm).reshape(M, N)
    for mrow in range(0, M, 64):
        one = _run(DType.BF16, 4, G, c.w, c.scales_f, c.biases_f, c.x_f[mrow * K:(mrow + 1) * K], 1, N, K)
        assert rel_err(got[mrow], one) <= 5e-2


def test_gather_single_expert_equals_plain_qmm():
    """All rows routed to one expert == plain batched qmv on that slab
    (tests/moe_gather_qmm_gpu_correctness.rs:652)."""
    E, N, K, G, T = 4, 1024, 2048, 64, 6
    print("[case] gather single expert", flush=True)
    c = make_case(16, DType.F16, 4, G, T, N, K, E=E)
    e = 2
    wpe, spe = N * K // 8, N * K // G
    plain = _run(DType.F16, 4, G, c.w[e * wpe:(e + 1) * wpe], c.scales_f[e * spe:(e + 1) * spe],
                 c.biases_f[e * spe:(e + 1) * spe], c.x_f, T, N, K)
    bw, bs, bb = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    bx = GpuBuffer.from_bytes(c.x_bytes)
    off = np.zeros(E + 1, "<u4")
    off[e + 1:] = T
    idx = np.full(T, e, "<u4")
    for fn, route in ((ops.gather_qmv_csr, off), (ops.gather_qmv_indices, idx)):
        out = GpuBuffer(T * N * 2)
        fn(DType.F16, 4, G, bx, bw, bs, bb, GpuBuffer.from_bytes(route.tobytes()), out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), DType.F16)
        assert rel_err(got, plain) <= 1e-3
        out.free()


def test_gather_unsorted_indices_and_permutation():
    """Per-row indices need not be sorted; permuting rows permutes outputs; rows
    beyond every CSR offset fall to expert 0 (moe.rs:376-385)."""
    E, N, K, G, T = 5, 512, 1024, 32, 11
    print("[case] gather unsorted / permutation", flush=True)
    c = make_case(17, DType.F32, 4, G, T, N, K, E=E)
    rng = np.random.default_rng(18)
    idx = rng.integers(0, E, size=T).astype("<u4")
    bw, bs, bb = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)

    def gather(xrows, ids):
        out = GpuBuffer(T * N * 4)
        ops.gather_qmv_indices(DType.F32, 4, G, GpuBuffer.from_bytes(pack_f32(xrows, DType.F32)), bw, bs, bb,
                               GpuBuffer.from_bytes(ids.tobytes()), out, T, N, K, E)
        return unpack_f32(out.read_bytes(), DType.F32).reshape(T, N)

    base = gather(c.x_f, idx)
    perm = rng.permutation(T)
    assert np.array_equal(gather(c.x_f.reshape(T, K)[perm].ravel(), idx[perm]), base[perm])
    # CSR with offsets ending before T: the tail rows use expert 0
    off = np.array([0, 2, 4, 6, 8, 9], "<u4")
    out = GpuBuffer(T * N * 4)
    ops.gather_qmv_csr(DType.F32, 4, G, GpuBuffer.from_bytes(c.x_bytes), bw, bs, bb,
                       GpuBuffer.from_bytes(off.tobytes()), out, T, N, K, E)
    got = unpack_f32(out.read_bytes(), DType.F32).reshape(T, N)
    ids_csr = np.array([0, 0, 1, 1, 2, 2, 3, 3, 4, 0, 0], "<u4")
    assert rel_err(got, gather(c.x_f, ids_csr)) <= 1e-5


@pytest.mark.parametrize("bits,G,N,K", [(3, 32, 40, 96), (5, 32, 17, 160), (6, 64, 33, 192), (4, 16, 24, 64),
                                        (4, 64, 7, 5120), (8, 32, 13, 96), (2, 32, 9, 192), (4, 64, 1000, 1536)])
def test_ragged_shapes_and_odd_widths(oracle, bits, G, N, K):
    """Shapes outside the tiled kernel's geometry (odd widths, N not a multiple of
    the tile, chunk counts that are not wave multiples) take the generic path."""
    print(f"[case] ragged b{bits} g{G} N{N} K{K}", flush=True)
    rng = np.random.default_rng(bits * 1000 + N)
    codes = rng.integers(0, 1 << bits, size=(N, K), dtype=np.uint8)
    w = pack_codes(codes, bits)
    s = (0.02 * np.abs(rng.standard_normal(N * K // G)) + 1e-3).astype(np.float32)
    b = (-(1 << (bits - 1)) * s).astype(np.float32)
    for M in (1, 3):
        x = rng.standard_normal(M * K).astype(np.float32)
        got = _run(DType.F32, bits, G, w, s, b, x, M, N, K)
        exp = oracle.qmm_f64(w, s, b, x, M, N, K, bits, G)
        assert rel_err(got, exp) <= 1e-4


def test_empty_and_invalid_inputs():
    c = make_case(19, DType.F32, 4, 64, 1, 64, 512)
    bw, bs, bb, bx = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                      GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(64 * 4)
    ops.qmv(DType.F32, 4, 64, bw, bs, bb, bx, out, 0, 64, 512)                 # M = 0: no-op
    ops.gather_qmv_indices(DType.F32, 4, 64, bx, bw, bs, bb, bx, out, 0, 64, 512, 1)  # T = 0: no-op
    for bad in (dict(bits=1), dict(bits=9), dict(G=0), dict(G=48), dict(K=0), dict(N=0), dict(dt=7)):
        with pytest.raises(MtqError):
            ops.qmv(bad.get("dt", DType.F32), bad.get("bits", 4), bad.get("G", 64), bw, bs, bb, bx, out, 1,
                    bad.get("N", 64), bad.get("K", 512))
    with pytest.raises(MtqError) as ei:
        ops.qmv(DType.F32, 4, 64, 0, bs, bb, bx, out, 1, 64, 512)              # null pointer
    assert ei.value.code == -2


@pytest.mark.parametrize("M,entry", [(1, ops.qmv), (4, ops.qmv), (16, ops.qmv), (64, ops.qmm)], ids=["m1", "m4", "m16", "m64"])
@pytest.mark.parametrize("scale", [3e-5, 1e-6])
def test_f16_activations_below_the_smallest_normal(oracle, M, entry, scale):
    """f16 activations in the subnormal range (|x| < 6.1e-5) count in full, as they do in the reference's f32
    arithmetic: the split dot adds MAGIC x scale x sum(x) on one side and takes it off on the other, so a kernel that
    dropped such an operand on one side only would be wrong by two orders of magnitude. Outputs are of the order of
    the activations, so the bound is relative to the largest expected output: 5e-3 (the f16 rounding of the output
    itself is 1.4e-3 there)."""
    dt, N, K, G = DType.F16, 512, 4096, 64
    print(f"[case] f16 activations x {scale:g}, M={M}", flush=True)
    c = make_case(9, dt, 4, G, M, N, K, bias_rule="midpoint")
    x = oracle.round_through((c.x_f * np.float32(scale)).astype(np.float32), 1)
    assert np.count_nonzero(np.abs(x) < 6.1e-5) > x.size // 2 and np.count_nonzero(x) > x.size // 2
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, x, M, N, K, 4, G).reshape(-1)
    got = _run(dt, 4, G, c.w, c.scales_f, c.biases_f, x, M, N, K, entry=entry)
    assert np.max(np.abs(got - exp)) <= 5e-3 * np.max(np.abs(exp))
