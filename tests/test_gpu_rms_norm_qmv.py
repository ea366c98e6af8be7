"""Fused RMSNorm + quantized GEMV against the oracle, through the C-ABI.

Reference kernels: ffai_rms_norm_qgemv / _fast / _int8_fast
(crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:53-125,128-456,459-). The first block runs
the reference's own setups (crates/metaltile-std/tests/rms_norm_qgemv_gpu_correctness.rs:
126-295: xorshift inputs, min/max int4 rows, eps 1e-5) with its metric and bounds,
max |a-e| / max(|e|, 1e-3) <= 5e-3 (f32), 2e-2 (f16), 5e-2 (bf16). The second block covers
the shapes the fused streaming kernel takes (rows of whole 512-code segments, decode sizes)
against the f64-accumulated oracle: max |a-e| / max(|e|, 1) <= 1e-4 (f32), 1e-2 (f16, bf16);
for f16 / bf16 the library rounds the normalised activation to the element type before the
dot, which is inside these bounds.
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err
from tests.test_gpu_batched import REF_TOL, _quantize_int4, _ref_err, _source

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}

REF_CASES = [("ffai_rms_norm_qgemv", DType.F32, 256, 64, 8, 128), ("ffai_rms_norm_qgemv", DType.F32, 512, 128, 6, 128),
             ("ffai_rms_norm_qgemv", DType.F16, 256, 64, 8, 128), ("ffai_rms_norm_qgemv", DType.BF16, 256, 64, 8, 128),
             ("ffai_rms_norm_qgemv_fast", DType.F32, 512, 64, 16, 64), ("ffai_rms_norm_qgemv_fast", DType.F16, 512, 64, 16, 64),
             ("ffai_rms_norm_qgemv_fast", DType.BF16, 512, 64, 16, 64), ("ffai_rms_norm_qgemv_fast", DType.F32, 1024, 64, 32, 64)]


@pytest.mark.parametrize("name,dt,K,G,N,tpg", REF_CASES, ids=lambda v: getattr(v, "name", str(v)))
def test_reference_setups(ctx, oracle, name, dt, K, G, N, tpg):
    print(f"[case] {name} {dt.name} in_dim={K} g{G} out_dim={N}", flush=True)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    eps = np.float32(1e-5)
    x = rt(_source(K, 0xA1, 2.0, 0.1))
    nw = rt(_source(K, 0xB2, 0.4, 1.0))
    w, s, b = _quantize_int4(_source(N * K, 0xC3, 3.0, 0.0), N, K, G)
    s, b = rt(s), rt(b)
    exp, _, _ = oracle.rms_norm_qgemv(w, s, b, x, nw, K, G, N, 4, eps)
    bufs = {"x": pack_f32(x, dt), "norm_weight": pack_f32(nw, dt), "weight": w.tobytes(), "scales": pack_f32(s, dt),
            "biases": pack_f32(b, dt), "output": bytes(N * dt.size_bytes), "eps_buf": eps.tobytes()}
    grid = (N if tpg == 128 else N // 8, 1, 1)
    res = ctx.dispatch_with_grid(name, dt, bufs, {"in_dim": K, "group_size": G}, grid, (tpg, 1, 1))
    got = unpack_f32(res.outputs["output"], dt)
    assert got.size == N and np.any(got != 0.0)
    assert _ref_err(got, exp) <= REF_TOL[dt]


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits,N,K,G", [(4, 4096, 4096, 64), (4, 1000, 2048, 64), (8, 512, 2048, 64), (4, 333, 8192, 128),
                                        (4, 64, 576, 64), (3, 64, 1024, 64), (3, 4096, 4096, 64), (3, 64, 2048, 64),
                                        (5, 1024, 8192, 64)])
def test_decode_shapes(oracle, dt, bits, N, K, G):
    """The shapes from (4, 64, 576) on do not fit the fused kernel and take the two-step path; in the last
    three the f32 qmv of that path splits K over workgroups, whose partial tiles share the library-owned
    buffer with the normalised row and must not overwrite it."""
    print(f"[case] rms_norm_qmv {dt.name} b{bits} g{G} N{N} K{K}", flush=True)
    c = make_case(1300 + bits + N, dt, bits, G, 1, N, K, bias_rule="midpoint")
    rng = np.random.default_rng(N + K)
    nw = oracle.round_through((1.0 + 0.2 * rng.standard_normal(K)).astype(np.float32), ODT[dt])
    eps = np.float32(1e-5)
    _, exp64, _ = oracle.rms_norm_qgemv(c.w, c.scales_f, c.biases_f, c.x_f, nw, K, G, N, bits, eps)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    nwb, epsb = GpuBuffer.from_bytes(pack_f32(nw, dt)), GpuBuffer.from_bytes(eps.tobytes())
    out = GpuBuffer.from_bytes(b"\xff" * (N * dt.size_bytes))
    ops.rms_norm_qmv(dt, bits, G, x, nwb, w, s, b, out, epsb, N, K)
    got = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= TOL[dt]
    # unit norm weights and a row of rms 1 reduce to the plain qmv of the same row
    for buf in (w, s, b, x, nwb, epsb, out):
        buf.free()


def test_fused_equals_norm_then_qmv_f32(oracle):
    """f32 keeps the normalised row unrounded, so the fused launch and the two-step path
    (forced by a row length of 576) agree with the oracle to the same bound; and the fused
    kernel with unit weights on a row scaled to rms 1 (eps 0) reproduces plain qmv."""
    dt, bits, G, N, K = DType.F32, 4, 64, 256, 2048
    c = make_case(77, dt, bits, G, 1, N, K, bias_rule="midpoint")
    x = c.x_f / np.float32(np.sqrt(np.mean(c.x_f.astype(np.float64) ** 2)))
    ones, eps = np.ones(K, dtype=np.float32), np.float32(0.0)
    w, s, b = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes))
    xb, nwb, epsb = GpuBuffer.from_bytes(x.tobytes()), GpuBuffer.from_bytes(ones.tobytes()), GpuBuffer.from_bytes(eps.tobytes())
    o1, o2 = GpuBuffer(N * 4), GpuBuffer(N * 4)
    ops.rms_norm_qmv(dt, bits, G, xb, nwb, w, s, b, o1, epsb, N, K)
    ops.qmv(dt, bits, G, w, s, b, xb, o2, 1, N, K)
    a, p = unpack_f32(o1.read_bytes(N * 4), dt), unpack_f32(o2.read_bytes(N * 4), dt)
    assert rel_err(a, p) <= 1e-5
    for buf in (w, s, b, xb, nwb, epsb, o1, o2):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("N,K,G", [(4096, 4096, 64), (1000, 2048, 64), (333, 8192, 128), (14336, 4096, 64), (100, 14336, 64), (64, 1024, 32)])
def test_norm_fused_into_the_matrix_core_gemv(oracle, dt, N, K, G):
    """The same operation with the norm applied as the matrix-core GEMV stages its row (4-bit codes; forced with
    qmv.norm_mfma = 2), against the oracle at the bound of the other fused kernel."""
    from metaltile_amd import _lib
    lib = _lib.load()
    bits = 4
    print(f"[case] rms_norm_qmv on the matrix-core GEMV {dt.name} g{G} N{N} K{K}", flush=True)
    c = make_case(1400 + N, dt, bits, G, 1, N, K, bias_rule="midpoint")
    rng = np.random.default_rng(N + K)
    nw = oracle.round_through((1.0 + 0.2 * rng.standard_normal(K)).astype(np.float32), ODT[dt])
    eps = np.float32(1e-5)
    _, exp64, _ = oracle.rms_norm_qgemv(c.w, c.scales_f, c.biases_f, c.x_f, nw, K, G, N, bits, eps)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    nwb, epsb = GpuBuffer.from_bytes(pack_f32(nw, dt)), GpuBuffer.from_bytes(eps.tobytes())
    out = GpuBuffer.from_bytes(b"\xff" * (N * dt.size_bytes))
    assert lib.mtq_set_option(b"qmv.norm_mfma", 2) == 0
    try:
        rc, launches, _, n = ops.plan("rms_norm_qmv", dt, bits, G, 1, N, K)
        assert rc == 0 and n == 1 and "qmv_mfma_kernel" in launches[0][0], launches
        ops.rms_norm_qmv(dt, bits, G, x, nwb, w, s, b, out, epsb, N, K)
    finally:
        lib.mtq_set_option(b"qmv.norm_mfma", 0)
    got = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= TOL[dt]
    for buf in (w, s, b, x, nwb, epsb, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("N,K,G", [(14336, 4096, 64), (16390, 4096, 64), (1030, 4096, 32), (19, 4096, 128), (1, 4096, 64), (4096, 8192, 64), (33, 8192, 32), (1028, 8192, 128),
                                   (1030, 2048, 64), (4100, 3072, 32), (18944, 3584, 64), (50, 5120, 128), (4096, 6144, 64), (1028, 7168, 64), (20, 3584, 128)])
def test_norm_fused_into_the_one_row_per_wave_kernel(oracle, dt, N, K, G):
    """The same operation with the norm applied as the one-row-per-wave GEMV puts the activation row into LDS (4-bit
    codes, rows of 2048 ... 8192 codes in steps of 1024 or 3584, the last group of 64 chunks full or not; forced with
    qmv.kernel = 3 where it is not the automatic route): every group size, ragged last workgroups, behind a cache flush, guard elements after the output, against the oracle at the
    bound of the other fused kernels."""
    import metaltile_amd as m
    from metaltile_amd import _lib
    lib = _lib.load()
    bits = 4
    print(f"[case] rms_norm_qmv on the one-row-per-wave GEMV {dt.name} g{G} N{N} K{K}", flush=True)
    c = make_case(1500 + N + G, dt, bits, G, 1, N, K, bias_rule="midpoint")
    rng = np.random.default_rng(N + K + G)
    nw = oracle.round_through((1.0 + 0.2 * rng.standard_normal(K)).astype(np.float32), ODT[dt])
    eps = np.float32(1e-5)
    _, exp64, _ = oracle.rms_norm_qgemv(c.w, c.scales_f, c.biases_f, c.x_f, nw, K, G, N, bits, eps)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    nwb, epsb = GpuBuffer.from_bytes(pack_f32(nw, dt)), GpuBuffer.from_bytes(eps.tobytes())
    rb = N * dt.size_bytes
    out = GpuBuffer.from_bytes(b"\xab" * (rb + 64))
    assert lib.mtq_set_option(b"qmv.kernel", 3) == 0
    try:
        rc, launches, _, n = ops.plan("rms_norm_qmv", dt, bits, G, 1, N, K)
        assert rc == 0 and n == 1 and ("qmv_rows_norm_kernel" in launches[0][0] or "qmv_rows_norm_ragged_kernel" in launches[0][0]), launches
        m.GpuRunner(0).flush_slc()
        ops.rms_norm_qmv(dt, bits, G, x, nwb, w, s, b, out, epsb, N, K)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    raw = out.read_bytes()
    assert raw[rb:] == b"\xab" * 64
    got = unpack_f32(raw[:rb], dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= TOL[dt]
    for buf in (w, s, b, x, nwb, epsb, out):
        buf.free()
