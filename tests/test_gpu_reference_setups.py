"""GPU parity on the reference's own test setups (closed-form inputs, CPU
oracle, absolute tolerance per dtype), dispatched by the reference kernel's
name through the C-ABI exactly as its harness does
(crates/metaltile-std/src/run_kernel.rs:97-155)."""
import numpy as np
import pytest

from metaltile_amd import DType, MtqError, unpack_f32
from tests import ref_setups as R
from tests.parity import abs_err, cosine

pytestmark = pytest.mark.gpu


def _run(ctx, su):
    print(f"[case] {su['kernel']} {su['dtype'].name} consts={su['consts']}", flush=True)
    res = ctx.dispatch_with_grid(su["kernel"], su["dtype"], su["buffers"], su["consts"], su["grid"], su["tpg"])
    got = unpack_f32(res.outputs[su["out"]], su["dtype"])
    assert got.size == su["expected"].size
    assert np.any(got != 0.0), "output is all zero"
    err = abs_err(got, su["expected"])
    assert err <= su["tol"], f"{su['kernel']} {su['dtype'].name}: max abs err {err:.3e} > {su['tol']}"
    return got


@pytest.mark.parametrize("dt", R.DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("name", sorted(R.QX_TESTS))
def test_quantized_rs_setups(ctx, name, dt):
    _run(ctx, R.qx_test(name, dt))


@pytest.mark.parametrize("dt", R.DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("name", sorted(R.GEMV_TESTS))
def test_dequant_gemv_setups(ctx, name, dt):
    _run(ctx, R.gemv_test(name, dt))


@pytest.mark.parametrize("dt", R.DTYPES, ids=lambda d: d.name)
def test_dequant_gemv_int4_expert_indexed(ctx, dt):
    _run(ctx, R.expert_indexed_test(dt))


@pytest.mark.parametrize("dt", R.DTYPES, ids=lambda d: d.name)
@pytest.mark.parametrize("kernel,grid_x", [("mt_moe_gather_qmm_int4", 8), ("mt_moe_gather_qmm_int4_m8", 1),
                                           ("mt_moe_gather_qmm_int4_m16", 1), ("mt_moe_gather_qmm_int4_m32", 1)])
def test_moe_gather_csr_setups(ctx, kernel, grid_x, dt):
    _run(ctx, R.moe_int4_test(kernel, grid_x, dt))


@pytest.mark.parametrize("dt", R.DTYPES, ids=lambda d: d.name)
def test_moe_gather_indices_equals_csr(ctx, dt):
    """The per-row-index ABI on the same inputs: indices expanded from the CSR
    offsets must give the same rows (cosine >= 0.999 is the reference's bar,
    tests/moe_gather_qmm_gpu_correctness.rs:740; here the abs tolerance holds too)."""
    su = R.moe_int4_test("mt_moe_gather_qmm_int4", 8, dt)
    d = R.moe_int4_inputs(dt)
    idx = np.array([0, 0, 1, 1, 1, 2], dtype="<u4")
    bufs = {"x": su["buffers"]["x"], "w": su["buffers"]["weight_packed"], "scales": su["buffers"]["scales"],
            "biases": su["buffers"]["biases"], "indices": idx.tobytes(), "out": su["buffers"]["out"]}
    consts = {"m_total": d["t_rows"], "n_out": d["m_out"], "k_in": d["k_in"], "group_size": d["group_size"]}
    print("[case] mt_moe_gather_qmm_mma_int4", dt.name, flush=True)
    res = ctx.dispatch_with_grid("mt_moe_gather_qmm_mma_int4", dt, bufs, consts, (1, 1, 1), (128, 1, 1))
    got = unpack_f32(res.outputs["out"], dt)
    assert abs_err(got, su["expected"]) <= su["tol"]
    assert cosine(got, su["expected"]) >= 0.999


def test_legacy_mt_qmv_f32(ctx):
    _run(ctx, R.legacy_qmv_f32())


def test_short_buffer_is_rejected(ctx):
    # reference: single_dispatch.rs:154-158 (BufferSize error)
    su = R.qx_test("test_qmv", DType.F32)
    bad = dict(su["buffers"])
    bad["scales"] = bad["scales"][:-4]
    with pytest.raises(MtqError) as ei:
        ctx.dispatch_with_grid(su["kernel"], su["dtype"], bad, su["consts"], su["grid"], su["tpg"])
    assert ei.value.code == -4 and "scales" in str(ei.value)


def test_unknown_kernel_and_bad_shape(ctx):
    su = R.qx_test("test_qmv", DType.F32)
    with pytest.raises(MtqError) as ei:
        ctx.dispatch_with_grid("mt_not_a_kernel", su["dtype"], su["buffers"], su["consts"])
    assert ei.value.code == -5
    consts = dict(su["consts"])
    consts["gs_per_row"] = 7          # does not divide k
    with pytest.raises(MtqError) as ei:
        ctx.dispatch_with_grid(su["kernel"], su["dtype"], su["buffers"], consts)
    assert ei.value.code == -3
    missing = {k: v for k, v in su["buffers"].items() if k != "x"}
    with pytest.raises(MtqError) as ei:
        ctx.dispatch_with_grid(su["kernel"], su["dtype"], missing, su["consts"])
    assert ei.value.code == -2
