"""Fused gated RMSNorm + 4-bit GEMV against the oracle, through the C-ABI.

Reference kernel: ffai_gated_rms_norm_qgemv_int4_fast (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:88-291):
y f32 [hv, dv], z / norm_weight of the element type, inner = y * inv_rms[row] * norm_weight[d] * silu(z) kept in f32,
then the 4-bit GEMV over the hv * dv values. The first block runs the reference's own setup (:372-437: hv 4, dv 128,
out_dim 512, group 64, eps 1e-5, xorshift inputs, min/max int4 rows) under the kernel's name, with the reference's
bounds 5e-3 (f32), 3e-2 (f16), 6e-2 (bf16) on max |a-e| / max(|e|, 1e-3). The second block covers other shapes, its
bench shape first (:449-476: hv 16, dv 128, out_dim 2048), including ones outside the reference kernel's invariants
(odd hv, dv not a multiple of 32, hv * dv not a multiple of 512, group 32 / 128), against the f64-accumulated oracle
(rows of whole multiples of 2048 values with dv = 32 .. 2048 in powers of two run as one launch of the streaming kernel,
a row's sum of squares over 1 .. 64 neighbouring lanes; the others stage the activation in a library-owned buffer):
max |a-e| / max(|e|, 1) <= 1e-4 (f32), 1e-2 (f16, bf16).
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err
from tests.test_gpu_batched import _quantize_int4, _ref_err, _source

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}
REF_TOL = {DType.F32: 5e-3, DType.F16: 3e-2, DType.BF16: 6e-2}
NAME = "ffai_gated_rms_norm_qgemv_int4_fast"


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("hv,dv,N", [(4, 128, 512)])
def test_reference_setup(ctx, oracle, dt, hv, dv, N):
    print(f"[case] {NAME} {dt.name} hv={hv} dv={dv} out_dim={N}", flush=True)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    G, K, eps = 64, hv * dv, np.float32(1e-5)
    y = _source(K, 0xA1, 2.0, 0.1)            # stays f32
    z = rt(_source(K, 0xD4, 1.5, 0.0))
    nw = rt(_source(dv, 0xB2, 0.4, 1.0))
    w, s, b = _quantize_int4(_source(N * K, 0xC3, 3.0, 0.0), N, K, G)
    s, b = rt(s), rt(b)
    exp, _, _ = oracle.gated_rms_norm_qgemv(w, s, b, y, z, nw, hv, dv, G, N, eps)
    bufs = {"y": y.tobytes(), "z": pack_f32(z, dt), "norm_weight": pack_f32(nw, dt), "eps_buf": eps.tobytes(),
            "q_weight": w.tobytes(), "q_scales": pack_f32(s, dt), "q_biases": pack_f32(b, dt), "out": bytes(N * dt.size_bytes)}
    res = ctx.dispatch_with_grid(NAME, dt, bufs, {"hv": hv, "dv": dv, "out_dim": N, "group_size": G}, (N // 8, 1, 1), (64, 1, 1))
    got = unpack_f32(res.outputs["out"], dt)
    assert got.size == N and np.any(got != 0.0)
    assert _ref_err(got, exp) <= REF_TOL[dt]


def _case(oracle, dt, hv, dv, N, G, seed):
    K = hv * dv
    c = make_case(seed, dt, 4, G, 1, N, K, bias_rule="midpoint")
    rng = np.random.default_rng(seed)
    y = (rng.standard_normal((hv, dv)) * rng.uniform(0.2, 5.0, size=(hv, 1))).astype(np.float32)
    z = oracle.round_through((1.5 * rng.standard_normal(K)).astype(np.float32), ODT[dt])
    nw = oracle.round_through((1.0 + 0.2 * rng.standard_normal(dv)).astype(np.float32), ODT[dt])
    return c, y, z, nw


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("hv,dv,N,G", [(16, 128, 2048, 64), (32, 128, 4096, 64), (4, 128, 512, 64), (1, 512, 64, 64), (3, 96, 40, 32),
                                       (5, 128, 1000, 128), (64, 128, 333, 64), (2, 36, 8, 8), (16, 256, 4096, 64), (1, 2048, 100, 64),
                                       (64, 32, 64, 32), (8, 512, 256, 128), (3, 2048, 17, 64), (32, 1024, 24, 64),
                                       (8, 2048, 48, 64), (80, 128, 40, 64), (112, 128, 24, 64)])   # K = 16384 (512 threads), 10240, 14336
def test_shapes(oracle, dt, hv, dv, N, G):
    print(f"[case] gated_rms_norm_qmv {dt.name} hv{hv} dv{dv} g{G} N{N}", flush=True)
    K, eps = hv * dv, np.float32(1e-5)
    c, y, z, nw = _case(oracle, dt, hv, dv, N, G, 2100 + hv + dv + N)
    _, exp64, _ = oracle.gated_rms_norm_qgemv(c.w, c.scales_f, c.biases_f, y, z, nw, hv, dv, G, N, eps)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    w, s, b = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    yb, zb, nwb, epsb = (GpuBuffer.from_bytes(y.tobytes()), GpuBuffer.from_bytes(pack_f32(z, dt)), GpuBuffer.from_bytes(pack_f32(nw, dt)),
                         GpuBuffer.from_bytes(eps.tobytes()))
    out = GpuBuffer.from_bytes(b"\xff" * (N * dt.size_bytes))
    ops.gated_rms_norm_qmv(dt, G, yb, zb, nwb, epsb, w, s, b, out, hv, dv, N)
    got = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= TOL[dt]
    # a second call with other inputs writes the same library-owned buffer again
    y2 = (0.5 * y[::-1]).copy()
    yb.upload(y2.tobytes())
    _, exp64, _ = oracle.gated_rms_norm_qgemv(c.w, c.scales_f, c.biases_f, y2, z, nw, hv, dv, G, N, eps)
    ops.gated_rms_norm_qmv(dt, G, yb, zb, nwb, epsb, w, s, b, out, hv, dv, N)
    got = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
    assert rel_err(got, oracle.round_through(exp64.astype(np.float32), ODT[dt])) <= TOL[dt]
    for buf in (w, s, b, yb, zb, nwb, epsb, out):
        buf.free()


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("hv,dv,N", [(16, 128, 2048), (4, 1024, 200), (64, 64, 72)])
def test_one_launch_and_staged_agree(oracle, dt, hv, dv, N):
    """The same call as one launch of the streaming kernel (what f16 / bf16 take by themselves) and through the staged
    activation (what f32 takes): each against the oracle, and against each other within twice the bound."""
    from metaltile_amd import _lib
    lib = _lib.load()
    G, eps = 64, np.float32(1e-5)
    c, y, z, nw = _case(oracle, dt, hv, dv, N, G, 2300 + hv + N)
    _, exp64, _ = oracle.gated_rms_norm_qgemv(c.w, c.scales_f, c.biases_f, y, z, nw, hv, dv, G, N, eps)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    w, s, b = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    yb, zb, nwb, epsb = (GpuBuffer.from_bytes(y.tobytes()), GpuBuffer.from_bytes(pack_f32(z, dt)), GpuBuffer.from_bytes(pack_f32(nw, dt)),
                         GpuBuffer.from_bytes(eps.tobytes()))
    got = {}
    try:
        for mode in (2, 1):
            print(f"[case] gated_rms_norm_qmv {dt.name} hv{hv} dv{dv} N{N} qmv.gated_fused={mode}", flush=True)
            assert lib.mtq_set_option(b"qmv.gated_fused", mode) == 0
            out = GpuBuffer.from_bytes(b"\xff" * (N * dt.size_bytes))
            ops.gated_rms_norm_qmv(dt, G, yb, zb, nwb, epsb, w, s, b, out, hv, dv, N)
            got[mode] = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
            out.free()
            assert rel_err(got[mode], exp) <= TOL[dt]
    finally:
        lib.mtq_set_option(b"qmv.gated_fused", 0)
    assert rel_err(got[2], got[1]) <= 2 * TOL[dt]
    for buf in (w, s, b, yb, zb, nwb, epsb):
        buf.free()


def test_closed_gates_and_open_gates(oracle):
    """z = 0 closes every gate: the output is exactly zero whatever y holds. A gate of silu(z0) everywhere on one row with
    unit norm weights is silu(z0) times the library's own RMSNorm + qmv of that row."""
    dt, hv, dv, N, G = DType.F32, 8, 128, 256, 64
    K, eps = hv * dv, np.float32(1e-5)
    c, y, z, nw = _case(oracle, dt, hv, dv, N, G, 2200)
    w, s, b = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    yb, zb, nwb, epsb = (GpuBuffer.from_bytes(y.tobytes()), GpuBuffer.from_bytes(bytes(K * 4)), GpuBuffer.from_bytes(nw.tobytes()),
                         GpuBuffer.from_bytes(eps.tobytes()))
    out = GpuBuffer.from_bytes(b"\xff" * (N * 4))
    print("[case] gated_rms_norm_qmv closed gates", flush=True)
    ops.gated_rms_norm_qmv(dt, G, yb, zb, nwb, epsb, w, s, b, out, hv, dv, N)
    assert not unpack_f32(out.read_bytes(N * 4), dt).any()
    print("[case] gated_rms_norm_qmv one row, constant gate", flush=True)
    z0 = np.float32(0.8)
    zb.upload(np.full(K, z0, np.float32).tobytes())
    ones = GpuBuffer.from_bytes(np.ones(K, np.float32).tobytes())
    o2 = GpuBuffer(N * 4)
    ops.gated_rms_norm_qmv(dt, G, yb, zb, ones, epsb, w, s, b, out, 1, K, N)
    ops.rms_norm_qmv(dt, 4, G, yb, ones, w, s, b, o2, epsb, N, K)
    a, p = unpack_f32(out.read_bytes(N * 4), dt), unpack_f32(o2.read_bytes(N * 4), dt)
    silu = float(z0) / (1.0 + np.exp(-float(z0)))
    assert rel_err(a, (p * silu).astype(np.float32)) <= 1e-5
    for buf in (w, s, b, yb, zb, nwb, epsb, out, ones, o2):
        buf.free()


def test_argument_errors(oracle):
    dt = DType.BF16
    one = GpuBuffer(4096)
    for hv, dv, N, G in ((0, 128, 8, 64), (4, 0, 8, 64), (4, 128, 0, 64), (4, 128, 8, 0), (3, 96, 8, 64), (1, 4, 8, 4)):
        with pytest.raises(MtqError):
            ops.gated_rms_norm_qmv(dt, G, one, one, one, one, one, one, one, one, hv, dv, N)
    with pytest.raises(MtqError):
        ops.gated_rms_norm_qmv(dt, 64, 0, one, one, one, one, one, one, one, 4, 128, 8)
    one.free()
