"""Prefill with an arbitrary token count (the reference's dynamic-M path,
crates/metaltile-std/src/mlx/quantized_mma_dynamic_m.rs:1-110): one call at T rows must give
the first T rows of the reference's padded dispatch (zero rows appended to a multiple of 32,
`mt_qmm_mma` over the padded shape, trailing rows dropped), and both must match the oracle's
mma variant (weights rounded to the element type) within max |a-e| / max(|e|, 1) <= 1e-4 (f32),
1e-2 (f16, bf16)."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, dynamic_m, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("T,N,K", [(1, 256, 512), (37, 256, 1024), (33, 128, 512), (100, 384, 512), (257, 128, 1024)])
def test_ragged_token_counts(ctx, oracle, dt, T, N, K):
    bits, G = 4, 64
    print(f"[case] dynamic-M {dt.name} T={T} N={N} K={K}", flush=True)
    c = make_case(3100 + T, dt, bits, G, T, N, K, bias_rule="midpoint")
    exp = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, T, N, K, bits, G, ODT[dt], threads=8)
    exp = oracle.round_through(np.asarray(exp, dtype=np.float32), ODT[dt])
    esz = dt.size_bytes
    w, s, b = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    x, out = GpuBuffer.from_bytes(c.x_bytes), GpuBuffer.from_bytes(b"\xff" * (T * N * esz))
    dynamic_m.qmm_dynamic_m(dt, bits, G, w, s, b, x, out, T, N, K)
    got = unpack_f32(out.read_bytes(T * N * esz), dt)
    assert np.isfinite(got).all() and rel_err(got, exp) <= TOL[dt]
    # the reference's way: pad, dispatch mt_qmm_mma by name over the padded shape, slice
    mp = dynamic_m.pad_t_to_bm(T)
    res = ctx.dispatch_with_grid(dynamic_m.kernel_name_for(dt), dt,
                                 {"w": c.w.tobytes(), "scales": c.scales_bytes, "biases": c.biases_bytes,
                                  "x": dynamic_m.pad_x_rows_bytes(c.x_bytes, T, K, esz), "out": bytes(mp * N * esz)},
                                 {"k": K, "n": N, "gs_per_row": K // G}, tuple(dynamic_m.dispatch_grid(T, N)), (dynamic_m.TPG, 1, 1))
    padded = unpack_f32(res.outputs["out"], dt)
    assert rel_err(padded[:T * N], exp) <= TOL[dt]
    assert not padded[T * N:].any()      # zero activation rows give exactly zero
    for buf in (w, s, b, x, out):
        buf.free()
