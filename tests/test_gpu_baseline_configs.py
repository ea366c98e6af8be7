"""GPU parity at the benchmark configurations' real shapes, through the typed
C-ABI entry points, against the f64-accumulated oracle on the same seeded,
dtype-rounded inputs. Tolerance = the configuration's stated relative bound on
max|a-e| / max(|e|, 1)."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, ops, unpack_f32
from metaltile_amd.synth import make_case, top2_routing
from tests.parity import rel_err, cosine

pytestmark = pytest.mark.gpu


def _upload(case):
    return (GpuBuffer.from_bytes(case.w.tobytes()), GpuBuffer.from_bytes(case.scales_bytes),
            GpuBuffer.from_bytes(case.biases_bytes), GpuBuffer.from_bytes(case.x_bytes))


def _qmv_gpu(case, entry=ops.qmv):
    w, s, b, x = _upload(case)
    out = GpuBuffer(case.M * case.N * case.dtype.size_bytes)
    entry(case.dtype, case.bits, case.group_size, w, s, b, x, out, case.M, case.N, case.K)
    got = unpack_f32(out.read_bytes(), case.dtype)
    for buf in (w, s, b, x, out):
        buf.free()
    return got


def _check(case, oracle, tol, entry=ops.qmv, mma=False):
    print(f"[case] {entry.__name__} {case.dtype.name} b{case.bits} g{case.group_size} M{case.M} N{case.N} K{case.K}", flush=True)
    got = _qmv_gpu(case, entry)
    odt = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}[case.dtype]
    if mma:
        exp = oracle.qmm_mma(case.w, case.scales_f, case.biases_f, case.x_f, case.M, case.N, case.K,
                             case.bits, case.group_size, odt, threads=8)
    else:
        exp = oracle.qmm_f64(case.w, case.scales_f, case.biases_f, case.x_f, case.M, case.N, case.K,
                             case.bits, case.group_size, threads=8)
    exp_t = oracle.round_through(exp.astype(np.float32), odt)   # expected after the store cast
    err = rel_err(got, exp_t)
    assert err <= tol, f"rel err {err:.3e} > {tol}"
    assert cosine(got, exp) >= 0.999
    return got, exp


def test_config0_qmv_f32_4096(oracle):
    """qmv f32, N=K=4096, 4-bit g64: rel 1e-4."""
    case = make_case(1000, DType.F32, 4, 64, 1, 4096, 4096)
    got, exp = _check(case, oracle, 1e-4)
    # context for the 1e-4 budget: the reference-faithful f32-sequential oracle's own distance
    seq = oracle.qmm(case.w, case.scales_f, case.biases_f, case.x_f, 1, 4096, 4096, 4, 64, threads=8)
    print(f"gpu rel={rel_err(got, exp):.2e}  f32-sequential-oracle rel={rel_err(seq, exp):.2e}")


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_config1_qmv_bf16_llama(oracle, N, K):
    """qmv bf16, Llama-3-8B MLP shapes, 4-bit g64: rel 1e-2."""
    _check(make_case(1001 + N, DType.BF16, 4, 64, 1, N, K), oracle, 1e-2)


@pytest.mark.parametrize("M", [1, 4])
@pytest.mark.parametrize("G", [32, 64, 128])
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_config2_sweep_f16(oracle, bits, G, M):
    """bits x group-size sweep, f16, N=K=8192, M in {1,4}: rel 1e-2."""
    case = make_case(2000 + bits * 100 + G + M, DType.F16, bits, G, M, 8192, 8192, bias_rule="midpoint")
    _check(case, oracle, 1e-2)


@pytest.mark.parametrize("M", [32, 128, 512])
def test_config3_qmm_bf16(oracle, M):
    """qmm bf16 prefill, N=K=4096, 4-bit g64: rel 2e-2 against the reference's
    semantics for this configuration -- weight tiles dequantised to bf16 before
    the multiply (crates/metaltile-std/src/mlx/quantized.rs:2267-2274), which
    the oracle's qmm_mma restates. (That rounding alone moves results by up to
    3.4e-2 on this metric relative to exact dequantisation and the GPU's own
    sums add to that -- 5.1e-2 measured at M = 512 -- so against the exact
    oracle the GPU is held to 1e-1 only: a guard against gross error, the
    binding bound is the 2e-2 above.)
    M=2048 has a test of its own below (32 sampled rows: the oracle works row by row)."""
    case = make_case(3000 + M, DType.BF16, 4, 64, M, 4096, 4096)
    got, _ = _check(case, oracle, 2e-2, entry=ops.qmm, mma=True)
    exact = oracle.qmm_f64(case.w, case.scales_f, case.biases_f, case.x_f, M, 4096, 4096, 4, 64, threads=8)
    dev = rel_err(got, exact)
    print(f"deviation from exact dequantisation: {dev:.3e}")
    assert dev <= 1e-1


def test_config3_qmm_bf16_m2048_sampled_rows(oracle):
    """The M = 2048 point of the same configuration. An output row depends on its own activation row only, so 32
    rows drawn from the 2048 (first and last among them) are checked against the oracle run on those rows alone,
    at the cost of M = 32: 2e-2 against the mma semantics, 1e-1 against exact dequantisation; every other row must
    at least be finite and non-trivial."""
    M, N, K = 2048, 4096, 4096
    case = make_case(3000 + M, DType.BF16, 4, 64, M, N, K)
    w, s, b, x = (GpuBuffer.from_bytes(case.w.tobytes()), GpuBuffer.from_bytes(case.scales_bytes),
                  GpuBuffer.from_bytes(case.biases_bytes), GpuBuffer.from_bytes(case.x_bytes))
    out = GpuBuffer.from_bytes(b"\xff" * (M * N * 2))
    ops.qmm(DType.BF16, 4, 64, w, s, b, x, out, M, N, K)
    got = unpack_f32(out.read_bytes(), DType.BF16).reshape(M, N)
    for buf in (w, s, b, x, out):
        buf.free()
    assert np.isfinite(got).all() and np.all(np.abs(got).max(axis=1) > 0)
    rng = np.random.default_rng(3)
    rows = np.unique(np.concatenate([[0, M - 1, 127, 128, 1023, 1024], rng.choice(M, size=26, replace=False)]))
    xs = np.ascontiguousarray(case.x_f.reshape(M, K)[rows]).reshape(-1)
    mma = oracle.qmm_mma(case.w, case.scales_f, case.biases_f, xs, rows.size, N, K, 4, 64, 2, threads=8)
    exact = oracle.qmm_f64(case.w, case.scales_f, case.biases_f, xs, rows.size, N, K, 4, 64, threads=8)
    e_mma = rel_err(got[rows], oracle.round_through(mma.astype(np.float32), 2))
    e_exact = rel_err(got[rows], exact)
    print(f"M=2048, {rows.size} sampled rows: vs mma semantics {e_mma:.3e}, vs exact dequantisation {e_exact:.3e}")
    assert e_mma <= 2e-2 and e_exact <= 1e-1


def test_config4_gather_bf16(oracle):
    """gather_qmv bf16: 8 experts x W[14336,4096], 16 tokens x top-2 = 32 rows: rel 1e-2,
    through both routing views."""
    E, N, K, G = 8, 14336, 4096, 64
    case = make_case(4000, DType.BF16, 4, G, 16, N, K, E=E)
    tok, exp_id, offsets = top2_routing(4001, 16, E)
    T = tok.size
    x_rows = case.x_f.reshape(16, K)[tok].reshape(-1)            # (token, expert) pairs, sorted by expert
    from metaltile_amd import pack_f32
    w, s, b = (GpuBuffer.from_bytes(case.w.tobytes()), GpuBuffer.from_bytes(case.scales_bytes),
               GpuBuffer.from_bytes(case.biases_bytes))
    x = GpuBuffer.from_bytes(pack_f32(x_rows, DType.BF16))
    off = GpuBuffer.from_bytes(offsets.astype("<u4").tobytes())
    idx = GpuBuffer.from_bytes(exp_id.astype("<u4").tobytes())
    expected = oracle.gather_qmm(x_rows, case.w, case.scales_f, case.biases_f, T, K, N, E, 4, G,
                                 expert_offsets=offsets, f64=True, threads=8)
    exp_t = oracle.round_through(expected.astype(np.float32), 2)
    for name, fn, route in (("csr", ops.gather_qmv_csr, off), ("indices", ops.gather_qmv_indices, idx)):
        print(f"[case] gather {name} T={T} experts hit={np.unique(exp_id).size}", flush=True)
        out = GpuBuffer(T * N * 2)
        fn(DType.BF16, 4, G, x, w, s, b, route, out, T, N, K, E)
        got = unpack_f32(out.read_bytes(), DType.BF16)
        err = rel_err(got, exp_t)
        assert err <= 1e-2, f"{name}: rel err {err:.3e}"
        out.free()
    # single view: row 5 against its expert == the gather's row 5
    ei = GpuBuffer.from_bytes(np.array([exp_id[5]], "<u4").tobytes())
    x5 = GpuBuffer.from_bytes(pack_f32(x_rows.reshape(T, K)[5], DType.BF16))
    out1 = GpuBuffer(N * 2)
    ops.gather_qmv_single(DType.BF16, 4, G, w, s, b, x5, ei, out1, N, K, E)
    got1 = unpack_f32(out1.read_bytes(), DType.BF16)
    assert rel_err(got1, exp_t.reshape(T, N)[5]) <= 1e-2
    for buf in (w, s, b, x, off, idx, ei, x5, out1):
        buf.free()


def test_bench_launches_by_reference_name_at_full_size(ctx, oracle):
    """What bench.py times, checked: the headline qmv (both orientations), qmm at M = 512 and the 32-row gather at their
    full sizes through the name-keyed dispatch (mt_qmv, mt_qmm_mma, mt_moe_gather_qmm_int4: the names of
    crates/metaltile-std/src/mlx/quantized.rs:8, :2106 and crates/metaltile-std/src/ffai/moe.rs:358) against the oracle,
    with the bounds of the configurations above."""
    from metaltile_amd import pack_f32
    dt = DType.BF16
    for N, K in ((14336, 4096), (4096, 14336)):
        c = make_case(1100 + N % 97, dt, 4, 64, 1, N, K)
        r = ctx.dispatch_with_grid("mt_qmv", dt, {"w": c.w.tobytes(), "scales": c.scales_bytes, "biases": c.biases_bytes, "x": c.x_bytes,
                                                  "out": bytes(N * 2)}, {"k": K, "gs_per_row": K // 64}, (N // 8, 1, 1), (64, 1, 1))
        exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, c.x_f, 1, N, K, 4, 64, threads=8)
        e = rel_err(unpack_f32(r.outputs["out"], dt), exp)
        print(f"mt_qmv {N}x{K}: {e:.3e}")
        assert e <= 1e-2
    M, N, K = 512, 4096, 4096
    c = make_case(3000 + M, dt, 4, 64, M, N, K)
    r = ctx.dispatch_with_grid("mt_qmm_mma", dt, {"w": c.w.tobytes(), "scales": c.scales_bytes, "biases": c.biases_bytes, "x": c.x_bytes,
                                                  "out": bytes(M * N * 2)}, {"k": K, "n": N, "gs_per_row": K // 64}, (N // 32, M // 32, 1), (128, 1, 1))
    mma = oracle.qmm_mma(c.w, c.scales_f, c.biases_f, c.x_f, M, N, K, 4, 64, 2, threads=8)
    e = rel_err(unpack_f32(r.outputs["out"], dt), oracle.round_through(mma.astype(np.float32), 2))
    print(f"mt_qmm_mma M=512: {e:.3e}")
    assert e <= 2e-2
    E, N, K, G = 8, 14336, 4096, 64
    c = make_case(4000, dt, 4, G, 16, N, K, E=E)
    tok, exp_id, offsets = top2_routing(4001, 16, E)
    T = tok.size
    x_rows = c.x_f.reshape(16, K)[tok].reshape(-1)
    r = ctx.dispatch_with_grid("mt_moe_gather_qmm_int4", dt,
                               {"x": pack_f32(x_rows, dt), "weight_packed": c.w.tobytes(), "scales": c.scales_bytes, "biases": c.biases_bytes,
                                "expert_offsets": offsets.astype("<u4").tobytes(), "out": bytes(T * N * 2)},
                               {"k_in": K, "m_out": N, "n_experts": E, "group_size": G}, (N, T, 1), (32, 1, 1))
    exp = oracle.gather_qmm(x_rows, c.w, c.scales_f, c.biases_f, T, K, N, E, 4, G, expert_offsets=offsets, f64=True, threads=8)
    e = rel_err(unpack_f32(r.outputs["out"], dt), oracle.round_through(exp.astype(np.float32), 2))
    print(f"mt_moe_gather_qmm_int4 32 rows: {e:.3e}")
    assert e <= 1e-2
