"""GPU parity of the affine quantise / dequantise kernels (the packed format's
writer and reader) against the C oracle. Codes, and the element bits of scales,
biases and dequantised values, must be identical: the kernels round every
operation separately exactly as the oracle does."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, ops, pack_f32, unpack_f32
from metaltile_amd.synth import pack_codes
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
DTYPES = [DType.F32, DType.F16, DType.BF16]


def _quantize_gpu(v_bytes, dt, bits, G, n):
    w = GpuBuffer.from_bytes(v_bytes)
    out, s, b = GpuBuffer(n * bits // 8), GpuBuffer(n // G * dt.size_bytes), GpuBuffer(n // G * dt.size_bytes)
    ops.affine_quantize(dt, bits, G, w, out, s, b, n)
    res = (np.frombuffer(out.read_bytes(), dtype="<u4").copy(), s.read_bytes(), b.read_bytes())
    for buf in (w, out, s, b):
        buf.free()
    return res


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("bits,G", [(2, 64), (3, 32), (4, 64), (5, 32), (6, 32), (8, 64)])
def test_reference_quantize_setup_by_name(ctx, oracle, bits, G, dt):
    """The reference's own setup (ramp input, 8 groups), dispatched by kernel name:
    scales and biases against its closed form within its tolerance
    (crates/metaltile-std/src/mlx/quantized.rs:5280-5339), codes bit-exact against the oracle."""
    n_groups = 8
    n = n_groups * G
    w = ((np.arange(n) % 37).astype(np.float32) - np.float32(18.0)) * np.float32(0.05)
    wb = pack_f32(w, dt)
    wd = unpack_f32(wb, dt)
    print(f"[case] mt_affine_quantize_int{bits} {dt.name}", flush=True)
    res = ctx.dispatch_with_grid(f"mt_affine_quantize_int{bits}", dt,
                                 {"w": wb, "out": bytes(n * bits // 8), "scales": bytes(n_groups * dt.size_bytes),
                                  "biases": bytes(n_groups * dt.size_bytes)}, {"group_size": G}, (n_groups, 1, 1), (32, 1, 1))
    g = wd.reshape(n_groups, G)
    raw = (g.max(axis=1) - g.min(axis=1)) / np.float32((1 << bits) - 1)
    exp_s = np.where(raw < 1e-7, np.float32(1.0), raw).astype(np.float32)
    tol = {DType.F32: 1e-4, DType.F16: 1e-3, DType.BF16: 1e-2}[dt]
    assert np.max(np.abs(unpack_f32(res.outputs["scales"], dt) - exp_s)) <= tol
    assert np.max(np.abs(unpack_f32(res.outputs["biases"], dt) - g.min(axis=1))) <= tol
    codes, s, b = oracle.affine_quantize(wd, G, bits, ODT[dt])
    assert res.outputs["scales"] == pack_f32(s, dt) and res.outputs["biases"] == pack_f32(b, dt)
    assert np.array_equal(np.frombuffer(res.outputs["out"], dtype="<u4"), pack_codes(codes.reshape(1, n), bits))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("bits,G", [(2, 32), (2, 128), (3, 64), (4, 32), (4, 64), (4, 128), (5, 128), (6, 64), (7, 32), (8, 32), (8, 128)])
def test_quantize_codes_bit_exact(oracle, bits, G, dt):
    rng = np.random.default_rng(bits * 1000 + G)
    n = G * 4099   # ragged against the 256-thread workgroups
    v = (rng.standard_normal(n) * rng.uniform(0.01, 3.0)).astype(np.float32)
    v[:G] = 0.25                       # a constant group: scale falls back to 1
    v[G:2 * G] = np.linspace(-1, 1, G)  # values landing on code boundaries
    vb = pack_f32(v, dt)
    vd = unpack_f32(vb, dt)
    print(f"[case] affine_quantize b{bits} g{G} {dt.name} n={n}", flush=True)
    words, s, b = _quantize_gpu(vb, dt, bits, G, n)
    codes, es, eb = oracle.affine_quantize(vd, G, bits, ODT[dt])
    assert s == pack_f32(es, dt), "scales differ"
    assert b == pack_f32(eb, dt), "biases differ"
    exp_words = pack_codes(codes.reshape(1, n), bits)
    bad = np.flatnonzero(words != exp_words)
    assert bad.size == 0, f"{bad.size} packed words differ, first at {bad[:4]}"
    assert unpack_f32(s, dt)[0] == 1.0


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("bits,G", [(2, 64), (3, 32), (4, 64), (5, 32), (6, 64), (8, 64)])
def test_dequantize_bit_exact_and_by_name(ctx, oracle, bits, G, dt):
    rng = np.random.default_rng(77 + bits)
    n = G * 1031
    codes = rng.integers(0, 1 << bits, size=(1, n), dtype=np.uint8)
    w = pack_codes(codes, bits)
    s = unpack_f32(pack_f32((0.02 * np.abs(rng.standard_normal(n // G)) + 1e-3).astype(np.float32), dt), dt)
    b = unpack_f32(pack_f32((-(1 << (bits - 1)) * s).astype(np.float32), dt), dt)
    exp = pack_f32(oracle.affine_dequantize(w, s, b, n, G, bits), dt)
    print(f"[case] affine_dequantize b{bits} g{G} {dt.name}", flush=True)
    bw, bs, bb, bo = (GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s, dt)),
                      GpuBuffer.from_bytes(pack_f32(b, dt)), GpuBuffer(n * dt.size_bytes))
    ops.affine_dequantize(dt, bits, G, bw, bs, bb, bo, n)
    assert bo.read_bytes() == exp
    for buf in (bw, bs, bb, bo):
        buf.free()
    res = ctx.dispatch_with_grid(f"mt_affine_dequantize_int{bits}", dt,
                                 {"w": w.tobytes(), "scales": pack_f32(s, dt), "biases": pack_f32(b, dt),
                                  "out": bytes(n * dt.size_bytes)}, {"group_size": G}, (n * bits // 32, 1, 1), (1, 1, 1))
    assert res.outputs["out"] == exp


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quantize_dequantize_round_trip(bits, dt):
    """|dequantise(quantise(v)) - v| <= scale/2 plus the dtype's rounding of scale, bias and result."""
    G, n = 64, 64 * 2048
    rng = np.random.default_rng(5 + bits)
    v = rng.standard_normal(n).astype(np.float32)
    vb = pack_f32(v, dt)
    vd = unpack_f32(vb, dt)
    bw = GpuBuffer.from_bytes(vb)
    bo, bs, bb, br = GpuBuffer(n * bits // 8), GpuBuffer(n // G * dt.size_bytes), GpuBuffer(n // G * dt.size_bytes), GpuBuffer(n * dt.size_bytes)
    ops.affine_quantize(dt, bits, G, bw, bo, bs, bb, n)
    ops.affine_dequantize(dt, bits, G, bo, bs, bb, br, n)
    back = unpack_f32(br.read_bytes(), dt)
    scale = np.repeat(unpack_f32(bs.read_bytes(), dt), G)
    eps = {DType.F32: 1e-6, DType.F16: 2 ** -10, DType.BF16: 2 ** -7}[dt]
    bound = 0.5 * scale + eps * ((1 << bits) * scale + 2 * np.abs(vd) + 1e-3)
    assert np.all(np.abs(back - vd) <= bound)
    for buf in (bw, bo, bs, bb, br):
        buf.free()


def test_quantize_then_qmv_closes_the_loop(oracle):
    """A real f32 matrix quantised on the GPU feeds qmv on the GPU; the oracle does the same on the CPU."""
    dt, bits, G, N, K = DType.BF16, 4, 64, 512, 4096
    rng = np.random.default_rng(99)
    wf = (rng.standard_normal(N * K) * 0.05).astype(np.float32)
    x = unpack_f32(pack_f32(rng.standard_normal(K).astype(np.float32), dt), dt)
    wb = pack_f32(wf, dt)
    bw = GpuBuffer.from_bytes(wb)
    bq, bs, bb = GpuBuffer(N * K // 2), GpuBuffer(N * K // G * 2), GpuBuffer(N * K // G * 2)
    bx, bo = GpuBuffer.from_bytes(pack_f32(x, dt)), GpuBuffer(N * 2)
    ops.affine_quantize(dt, bits, G, bw, bq, bs, bb, N * K)
    ops.qmv(dt, bits, G, bq, bs, bb, bx, bo, 1, N, K)
    got = unpack_f32(bo.read_bytes(), dt)
    codes, es, eb = oracle.affine_quantize(unpack_f32(wb, dt), G, bits, 2)
    exp = oracle.qmm_f64(pack_codes(codes.reshape(N, K), bits), es, eb, x, 1, N, K, bits, G)
    assert rel_err(got, oracle.round_through(exp.astype(np.float32), 2)) <= 1e-2
    for buf in (bw, bq, bs, bb, bx, bo):
        buf.free()


def test_affine_rejects_bad_shapes():
    from metaltile_amd import MtqError
    a = GpuBuffer(4096)
    with pytest.raises(MtqError):
        ops.affine_quantize(DType.F32, 4, 64, a, a, a, a, 100)      # not a whole number of groups
    with pytest.raises(MtqError):
        ops.affine_quantize(DType.F32, 9, 64, a, a, a, a, 128)      # bits out of range
    with pytest.raises(MtqError):
        ops.affine_dequantize(DType.F32, 4, 12, a, a, a, a, 120)    # group not a multiple of the lane's run
    ops.affine_quantize(DType.F32, 4, 64, a, a, a, a, 0)            # nothing to do
    a.free()
