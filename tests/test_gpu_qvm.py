"""qvm (x @ W against the transposed packed weight [K, N]) against the oracle, through the C-ABI.

Reference kernels: mt_qvm_b{3,4,5,6,8} and mt_qvm_int4_fast
(crates/metaltile-std/src/mlx/quantized.rs:4397-4530, 4582-4700). The first test is the
reference's own setup (test_qvm_int4_fast, :5637-5665: n32 k512 g64, synth_packed_w(k, n, 4),
ramp scales / biases / x) with its absolute bounds 5e-3 / 5e-2 / 2e-1 (f32 / f16 / bf16). The
others compare with the f64-accumulated oracle: max |a-e| / max(|e|, 1) <= 1e-4 (f32), 1e-2
(f16, bf16).
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from tests.parity import abs_err, rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}


@pytest.mark.parametrize("dt,tol", [(DType.F32, 5e-3), (DType.F16, 5e-2), (DType.BF16, 2e-1)], ids=lambda v: getattr(v, "name", str(v)))
def test_reference_setup_qvm_int4_fast(ctx, oracle, dt, tol):
    n, k, g = 32, 512, 64
    gpc = k // g
    w = oracle.synth_packed_w(k, n, 4)
    i = np.arange(gpc * n)
    scales = (np.float32(0.004) + (i % 7).astype(np.float32) * np.float32(0.0008)).astype(np.float32)
    biases = (((i % 5).astype(np.float32) - np.float32(2.0)) * np.float32(0.0009)).astype(np.float32)
    x = (((np.arange(k) % 11).astype(np.float32) - np.float32(5.0)) * np.float32(0.01)).astype(np.float32)
    rt = lambda v: oracle.round_through(v, ODT[dt])
    exp, _ = oracle.qvm(w, rt(scales), rt(biases), rt(x), 1, n, k, 4, g)
    res = ctx.dispatch_with_grid("mt_qvm_int4_fast", dt,
                                 {"w": w.tobytes(), "scales": pack_f32(scales, dt), "biases": pack_f32(biases, dt),
                                  "x": pack_f32(x, dt), "out": bytes(n * dt.size_bytes)},
                                 {"k": k, "n": n, "gs_per_col": gpc}, (n // 8, 1, 1), (64, 1, 1))
    got = unpack_f32(res.outputs["out"], dt)
    assert np.any(got != 0.0)
    assert abs_err(got, oracle.round_through(exp, ODT[dt])) <= tol


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 7, 8])
# N = 64, 4096, 96 and 32 take the kernel whose threads own 32 columns; N = 8 and 40 (8-bit: 8 too) are not
# multiples of 32 and take the one whose threads own one word or one column (their N * bits is a multiple of 32
# for the even code widths only).
@pytest.mark.parametrize("M,N,K,G", [(1, 64, 256, 64), (1, 4096, 4096, 64), (3, 96, 1024, 32), (1, 32, 192, 64),
                                     (2, 40, 256, 64), (1, 8, 128, 32), (1, 1056, 2048, 64)])
def test_qvm_widths(oracle, dt, bits, M, N, K, G):
    if N * K > 1 << 22 and (bits not in (3, 4, 8) or dt == DType.F16):
        pytest.skip("the 4096 x 4096 case runs for 3-, 4- and 8-bit codes in f32 and bf16")
    if N * bits % 32:
        pytest.skip("N * bits must be a multiple of 32")
    print(f"[case] qvm {dt.name} b{bits} g{G} M{M} N{N} K{K}", flush=True)
    rng = np.random.default_rng(bits * 100 + N + K)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    codes = rng.integers(0, 1 << bits, size=(K, N), dtype=np.uint8)
    w = oracle.pack_codes(codes, bits)
    s = rt(0.02 * np.abs(rng.standard_normal((K // G) * N)) + 1e-3)
    b = rt(-(1 << (bits - 1)) * s + rng.standard_normal(s.size) * 1e-3)
    x = rt(rng.standard_normal(M * K))
    _, exp64 = oracle.qvm(w, s, b, x, M, N, K, bits, G)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    wb, sb, bb, xb = (GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s, dt)),
                      GpuBuffer.from_bytes(pack_f32(b, dt)), GpuBuffer.from_bytes(pack_f32(x, dt)))
    out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
    ops.qvm(dt, bits, G, wb, sb, bb, xb, out, M, N, K)
    got = unpack_f32(out.read_bytes(M * N * dt.size_bytes), dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= TOL[dt]
    for buf in (wb, sb, bb, xb, out):
        buf.free()


def test_qvm_by_family_name_and_bad_shapes(ctx, oracle):
    dt, bits, M, N, K, G = DType.F32, 5, 2, 64, 128, 64
    rng = np.random.default_rng(2)
    codes = rng.integers(0, 1 << bits, size=(K, N), dtype=np.uint8)
    w = oracle.pack_codes(codes, bits)
    s = (0.02 * np.abs(rng.standard_normal((K // G) * N)) + 1e-3).astype(np.float32)
    b = (rng.standard_normal(s.size) * 0.01).astype(np.float32)
    x = rng.standard_normal(M * K).astype(np.float32)
    res = ctx.dispatch_with_grid("mt_qvm_b5", dt, {"w": w.tobytes(), "scales": s.tobytes(), "biases": b.tobytes(),
                                                   "x": x.tobytes(), "out": bytes(M * N * 4)},
                                 {"k": K, "n": N, "group_size": G}, (N, M, 1), (32, 1, 1))
    _, exp64 = oracle.qvm(w, s, b, x, M, N, K, bits, G)
    assert rel_err(np.frombuffer(res.outputs["out"], dtype="<f4"), exp64) <= 1e-4
    buf = GpuBuffer(4096)
    for bits_, N_, K_, G_ in ((4, 0, 64, 64), (4, 64, 100, 64), (3, 40, 64, 64), (9, 64, 64, 64)):
        with pytest.raises(MtqError):
            ops.qvm(dt, bits_, G_, buf, buf, buf, buf, buf, 1, N_, K_)
    buf.free()
