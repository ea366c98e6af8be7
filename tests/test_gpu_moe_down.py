"""Fused MoE decode step (SwiGLU + indexed 4-bit down projection + weighted slot sum) against
the oracle, through the C-ABI. Reference kernel: ffai_moe_down_swiglu_accum_int4_chain8
(crates/metaltile-std/src/ffai/moe_down_swiglu_accum.rs:146-282). The first test is the
reference's own setup (crates/metaltile-std/tests/moe_down_swiglu_accum_gpu_correctness.rs:
199-296: Qwen3.6-A3B shape, xorshift gate / up rows, experts 3 17 41 58 72 89 104 121, unnormalised
slot weights) with its metric and bounds: max |a-e| / max(|e|, 1e-3) <= 1e-3 (f32), 5e-2
(f16, bf16). The others use the f64-accumulated oracle, max |a-e| / max(|e|, 1) <= 1e-4 (f32),
1e-2 (f16, bf16).
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from tests.parity import rel_err
from tests.test_gpu_batched import _quantize_int4, _ref_err, _source

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}


@pytest.mark.parametrize("dt,tol", [(DType.F32, 1e-3), (DType.BF16, 5e-2), (DType.F16, 5e-2)], ids=lambda v: getattr(v, "name", str(v)))
def test_reference_setup_qwen36(ctx, oracle, dt, tol):
    K, N, G, E = 768, 2048, 64, 128
    print(f"[case] ffai_moe_down_swiglu_accum_int4_chain8 {dt.name} in_dim={K} out_dim={N} E={E}", flush=True)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    gates = np.stack([rt(_source(K, 0x1001 + k * 0x91, 3.0, 0.0)) for k in range(8)])
    ups = np.stack([rt(_source(K, 0x2002 + k * 0x91, 2.0, 0.05)) for k in range(8)])
    experts = np.array([3, 17, 41, 58, 72, 89, 104, 121], dtype="<u4")
    sw = rt(np.array([0.31, 0.19, 0.12, 0.08, 0.06, 0.05, 0.04, 0.03], dtype=np.float32))
    # Weights: the reference draws all 128 x 2048 x 768 values from one sequential xorshift
    # stream (201 M draws); here only the eight routed experts' slabs are filled, from a numpy
    # generator over the same range (-0.25, 0.25), and the other slabs stay zero.
    w = np.zeros(E * N * K // 8, dtype="<u4")
    s = np.zeros(E * N * (K // G), dtype=np.float32)
    b = np.zeros_like(s)
    rng = np.random.default_rng(0x3003)
    for e in experts:
        slab = ((rng.random(N * K, dtype=np.float32) - np.float32(0.5)) * np.float32(0.5)).astype(np.float32)
        we, se, be = _quantize_int4(slab, N, K, G)
        w[e * N * K // 8:(e + 1) * N * K // 8] = we
        s[e * N * (K // G):(e + 1) * N * (K // G)] = rt(se)
        b[e * N * (K // G):(e + 1) * N * (K // G)] = rt(be)
    exp, _ = oracle.moe_down_swiglu_accum(gates, ups, experts, sw, w, s, b, K, N, G)
    bufs = {"expert_indices": experts.tobytes(), "slot_weights": pack_f32(sw, dt), "weights_stacked": w.tobytes(),
            "scales_stacked": pack_f32(s, dt), "biases_stacked": pack_f32(b, dt), "output": bytes(N * dt.size_bytes)}
    for k in range(8):
        bufs[f"gate_{k}"], bufs[f"up_{k}"] = pack_f32(gates[k], dt), pack_f32(ups[k], dt)
    res = ctx.dispatch_with_grid("ffai_moe_down_swiglu_accum_int4_chain8", dt, bufs,
                                 {"in_dim": K, "out_dim": N, "group_size": G}, (N, 1, 1), (128, 1, 1))
    got = unpack_f32(res.outputs["output"], dt)
    assert got.size == N and np.any(got != 0.0)
    assert _ref_err(got, exp) <= tol


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("slots,K,N,G,E", [(8, 768, 2048, 64, 16), (8, 1024, 300, 128, 9), (3, 256, 64, 32, 4), (1, 4096, 130, 64, 2)])
def test_shapes(oracle, dt, slots, K, N, G, E):
    print(f"[case] moe_down_swiglu {dt.name} slots={slots} K={K} N={N} g{G} E={E}", flush=True)
    rng = np.random.default_rng(K + N + slots)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    gates, ups = rt(rng.standard_normal((slots, K)) * 1.5).reshape(slots, K), rt(rng.standard_normal((slots, K))).reshape(slots, K)
    experts = rng.integers(0, E, slots).astype("<u4")
    sw = rt(rng.random(slots))
    w, s, b = _quantize_int4(((rng.random(E * N * K, dtype=np.float32) - 0.5) * 0.5).astype(np.float32), E * N, K, G)
    s, b = rt(s), rt(b)
    _, exp64 = oracle.moe_down_swiglu_accum(gates, ups, experts, sw, w, s, b, K, N, G)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    gb = [GpuBuffer.from_bytes(pack_f32(gates[k], dt)) for k in range(slots)]
    ub = [GpuBuffer.from_bytes(pack_f32(ups[k], dt)) for k in range(slots)]
    eb, swb = GpuBuffer.from_bytes(experts.tobytes()), GpuBuffer.from_bytes(pack_f32(sw, dt))
    wb, sb, bb = GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s, dt)), GpuBuffer.from_bytes(pack_f32(b, dt))
    out = GpuBuffer.from_bytes(b"\xff" * (N * dt.size_bytes))
    ops.moe_down_swiglu_accum(dt, G, gb, ub, eb, swb, wb, sb, bb, out, K, N, E)
    got = unpack_f32(out.read_bytes(N * dt.size_bytes), dt)
    assert np.isfinite(got).all()
    assert rel_err(got, exp) <= (1e-4 if dt == DType.F32 else 1e-2)
    for buf in gb + ub + [eb, swb, wb, sb, bb, out]:
        buf.free()


def test_rejects_unsupported_shapes():
    b = GpuBuffer(1 << 16)
    for K, G, slots in ((100, 64, 8), (8192, 64, 8), (768, 48, 8), (768, 64, 9), (768, 64, 0)):
        with pytest.raises(MtqError):
            ops.moe_down_swiglu_accum(DType.F32, G, [b] * slots, [b] * slots, b, b, b, b, b, b, K, 4, 1)
    b.free()
