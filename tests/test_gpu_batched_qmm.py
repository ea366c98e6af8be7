"""Batched Q/K/V and 4-way quantized matmul over several activation rows (the prefill siblings of the batched GEMV),
through the C-ABI.

Reference kernels: ffai_batched_qkv_qmm_fast (crates/metaltile-std/src/ffai/batched_qkv_qmm.rs:49-68) and
ffai_batched_4_qmm_fast (crates/metaltile-std/src/ffai/batched_4_qmm.rs:61-85): every output row m of every matrix is
the GEMV of activation row m, which is what the reference's test holds them to (crates/metaltile-std/tests/
batched_qkv_qmm_gpu_correctness.rs:207-258: the one-row fused kernel run once per row). The first block runs that
test's setups (in_dim 512, group 64, out_q 16, out_k = out_v 8; M 2 and 8 in f32, 4 in f16 and bf16; xsorshift inputs
with another value in every row, min/max int4 rows) under the kernels' names with its metric and bounds,
max |a-e| / max(|e|, 1e-3) <= 5e-3 (f32), 2e-2 (f16), 5e-2 (bf16). The second block: prefill shapes against the
f64-accumulated oracle, max |a-e| / max(|e|, 1) <= 1e-4 (f32), 1e-2 (f16, bf16) where mtq_qmm keeps the exact weights,
2e-2 against the oracle's mt_qmm_mma arithmetic and 1e-1 against exact dequantisation where it takes the MFMA tiles
(weights rounded to the element type), and bit-equality with one mtq_qmm call per matrix.
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err
from tests.test_gpu_batched import REF_TOL, _quantize_int4, _ref_err, _source

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}


def _ref_mats(oracle, dt, M, K, G, Ns, seeds):
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    x = rt(_source(M * K, 0x11, 2.0, 0.05))
    mats = []
    for N, seed in zip(Ns, seeds):
        w, s, b = _quantize_int4(_source(N * K, seed, 3.0, 0.0), N, K, G)
        s, b = rt(s), rt(b)
        mats.append((w, s, b, np.asarray(oracle.qmm(w, s, b, x, M, N, K, 4, G), dtype=np.float32).reshape(M, N)))
    return x, mats


@pytest.mark.parametrize("dt,M", [(DType.F32, 2), (DType.F32, 8), (DType.F16, 4), (DType.BF16, 4)], ids=lambda v: getattr(v, "name", str(v)))
def test_reference_qkv_qmm_setups(ctx, oracle, dt, M):
    K, G, Ns = 512, 64, (16, 8, 8)
    print(f"[case] ffai_batched_qkv_qmm_fast {dt.name} M={M}", flush=True)
    x, mats = _ref_mats(oracle, dt, M, K, G, Ns, (0x22, 0x33, 0x44))
    bufs = {"x": pack_f32(x, dt)}
    consts = {"in_dim": K, "group_size": G}
    for tag, (w, s, b, _), N in zip("qkv", mats, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = w.tobytes(), pack_f32(s, dt), pack_f32(b, dt)
        bufs[f"{tag}_buf"] = bytes(M * N * dt.size_bytes)
        consts[f"out_{tag}"] = N
    res = ctx.dispatch_with_grid("ffai_batched_qkv_qmm_fast", dt, bufs, consts, (-(-max(Ns) // 8), M, 3), (64, 1, 1))
    for tag, (_, _, _, exp) in zip("qkv", mats):
        got = unpack_f32(res.outputs[f"{tag}_buf"], dt)
        assert got.size == exp.size and np.any(got != 0.0)
        assert _ref_err(got, exp.reshape(-1)) <= REF_TOL[dt], tag


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
def test_reference_like_4way_qmm(ctx, oracle, dt):
    K, G, Ns, M = 512, 64, (16, 8, 24, 8), 4
    print(f"[case] ffai_batched_4_qmm_fast {dt.name} M={M}", flush=True)
    x, mats = _ref_mats(oracle, dt, M, K, G, Ns, (0x22, 0x33, 0x44, 0x55))
    bufs = {"x": pack_f32(x, dt)}
    consts = {"in_dim": K, "group_size": G}
    for tag, (w, s, b, _), N in zip("abcd", mats, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = w.tobytes(), pack_f32(s, dt), pack_f32(b, dt)
        bufs[f"{tag}_buf"] = bytes(M * N * dt.size_bytes)
        consts[f"out_{tag}"] = N
    res = ctx.dispatch_with_grid("ffai_batched_4_qmm_fast", dt, bufs, consts, (-(-max(Ns) // 8), M, 4), (64, 1, 1))
    for tag, (_, _, _, exp) in zip("abcd", mats):
        got = unpack_f32(res.outputs[f"{tag}_buf"], dt)
        assert got.size == exp.size and np.any(got != 0.0)
        assert _ref_err(got, exp.reshape(-1)) <= REF_TOL[dt], tag

@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
def test_row_count_comes_from_the_grid(ctx, oracle, dt):
    """The reference takes M from the grid's second dimension (crates/metaltile-std/src/ffai/batched_qkv_qmm.rs:46-70): a
    caller that binds buffers allocated for a longer sequence gets exactly grid[1] rows; the rows past them keep their
    bytes. With the all-ones placeholder grid the row count is what x holds."""
    K, G, Ns, M, cap = 512, 64, (16, 8, 8), 3, 7
    x, mats = _ref_mats(oracle, dt, cap, K, G, Ns, (0x22, 0x33, 0x44))
    bufs = {"x": pack_f32(x, dt)}
    consts = {"in_dim": K, "group_size": G}
    for tag, (w, s, b, _), N in zip("qkv", mats, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = w.tobytes(), pack_f32(s, dt), pack_f32(b, dt)
        bufs[f"{tag}_buf"] = b"\xab" * (cap * N * dt.size_bytes)
        consts[f"out_{tag}"] = N
    res = ctx.dispatch_with_grid("ffai_batched_qkv_qmm_fast", dt, bufs, consts, (-(-max(Ns) // 8), M, 3), (64, 1, 1))
    for tag, (_, _, _, exp), N in zip("qkv", mats, Ns):
        raw = res.outputs[f"{tag}_buf"]
        assert raw[M * N * dt.size_bytes:] == b"\xab" * ((cap - M) * N * dt.size_bytes), "rows past grid[1] must stay untouched"
        got = unpack_f32(raw[:M * N * dt.size_bytes], dt)
        assert _ref_err(got, exp[:M].reshape(-1)) <= REF_TOL[dt], tag
    res = ctx.dispatch_with_grid("ffai_batched_qkv_qmm_fast", dt, bufs, consts, (1, 1, 1), (64, 1, 1))   # no grid: all 7 rows
    for tag, (_, _, _, exp) in zip("qkv", mats):
        assert _ref_err(unpack_f32(res.outputs[f"{tag}_buf"], dt), exp.reshape(-1)) <= REF_TOL[dt], tag
    with pytest.raises(MtqError) as e:   # more rows asked for than x holds
        ctx.dispatch_with_grid("ffai_batched_qkv_qmm_fast", dt, bufs, consts, (2, cap + 1, 3), (64, 1, 1))
    assert e.value.code == -4


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("M,K,Ns", [(2, 2048, (2048, 512, 512)), (8, 4096, (4096, 1024, 1024)), (37, 1024, (520, 8, 136)),
                                    (128, 2048, (1024, 256, 256, 2048)), (5, 576, (40,))])
def test_prefill_shapes(oracle, dt, M, K, Ns):
    print(f"[case] qmm_batched {dt.name} M{M} K{K} N={Ns}", flush=True)
    G = 64
    cases = [make_case(3100 + j + M, dt, 4, G, M, N, K, bias_rule="midpoint") for j, N in enumerate(Ns)]
    x_f = cases[0].x_f
    xb = GpuBuffer.from_bytes(cases[0].x_bytes)
    ws = [GpuBuffer.from_bytes(c.w.tobytes()) for c in cases]
    ss = [GpuBuffer.from_bytes(c.scales_bytes) for c in cases]
    bs = [GpuBuffer.from_bytes(c.biases_bytes) for c in cases]
    outs = [GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes)) for N in Ns]
    ops.qmm_batched(dt, 4, G, ws, ss, bs, xb, outs, list(Ns), M, K)
    for j, (c, N) in enumerate(zip(cases, Ns)):
        raw = outs[j].read_bytes(M * N * dt.size_bytes)
        _, launches, _, _ = ops.plan("qmm", dt, 4, G, M, N, K)
        if dt != DType.F32 and any("qmm_" in l[0] for l in launches):
            # mtq_qmm took this matrix to the MFMA tiles, which multiply weights rounded to the element type (the
            # reference's mt_qmm_mma arithmetic): 2e-2 against that, 1e-1 against exact dequantisation
            mma = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, x_f, M, N, K, 4, G, ODT[dt], threads=8).reshape(-1)
            assert rel_err(unpack_f32(raw, dt), oracle.round_through(mma.astype(np.float32), ODT[dt])) <= 2e-2, j
            bound = 1e-1
        else:
            bound = TOL[dt]
        exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, x_f, M, N, K, 4, G).reshape(-1)
        exp = oracle.round_through(exp.astype(np.float32), ODT[dt])
        assert rel_err(unpack_f32(raw, dt), exp) <= bound, j
        single = GpuBuffer(M * N * dt.size_bytes)
        ops.qmm(dt, 4, G, ws[j], ss[j], bs[j], xb, single, M, N, K)
        assert single.read_bytes(M * N * dt.size_bytes) == raw, j    # the same kernels, one matrix after the other
        single.free()
    for buf in [xb] + ws + ss + bs + outs:
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
def test_names_keep_exact_weights_at_prefill_sizes(ctx, oracle, dt):
    """Under the reference kernel's name a prefill-sized call still multiplies by the exact s * q + b, as that kernel
    does (the typed call would take these matrices to the MFMA tiles and their rounded weights): 1e-2 against the
    f64-accumulated oracle."""
    M, K, G, Ns = 64, 2048, 64, (1024, 256, 256)
    print(f"[case] ffai_batched_qkv_qmm_fast {dt.name} M={M} K={K} N={Ns}", flush=True)
    cases = [make_case(3200 + j, dt, 4, G, M, N, K, bias_rule="midpoint") for j, N in enumerate(Ns)]
    bufs = {"x": cases[0].x_bytes}
    consts = {"in_dim": K, "group_size": G}
    for tag, c, N in zip("qkv", cases, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = c.w.tobytes(), c.scales_bytes, c.biases_bytes
        bufs[f"{tag}_buf"] = bytes(M * N * dt.size_bytes)
        consts[f"out_{tag}"] = N
    res = ctx.dispatch_with_grid("ffai_batched_qkv_qmm_fast", dt, bufs, consts, (max(Ns) // 8, M, 3), (64, 1, 1))
    for tag, c, N in zip("qkv", cases, Ns):
        exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, cases[0].x_f, M, N, K, 4, G).reshape(-1)
        got = unpack_f32(res.outputs[f"{tag}_buf"], dt)
        assert rel_err(got, oracle.round_through(exp.astype(np.float32), ODT[dt])) <= 1e-2, tag


def test_argument_errors():
    dt, one = DType.BF16, GpuBuffer(4096)
    four = [one] * 4
    for n, Ns, M, K, G in ((0, [], 4, 512, 64), (5, [8] * 5, 4, 512, 64), (2, [8, 0], 4, 512, 64), (2, [8, 8], 4, 500, 64), (2, [8, 8], 4, 512, 0)):
        with pytest.raises(MtqError):
            ops.qmm_batched(dt, 4, G, [one] * n, [one] * n, [one] * n, one, [one] * n, Ns, M, K)
    ops.qmm_batched(dt, 4, 64, four[:2], four[:2], four[:2], one, four[:2], [8, 8], 0, 512)   # no rows: nothing to do
    one.free()
