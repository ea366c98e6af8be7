"""The reference's own `#[test_kernel]` setups and legacy-test inputs for the
affine-quantized matmul path, restated as data + oracle calls.

Each function returns a dict: kernel name, buffers (name -> bytes, in the
kernel's binding names), constexprs, grid / tpg as the reference passes them,
the expected output (f32 values from the oracle on dtype-rounded inputs), the
output parameter name and the reference's absolute tolerance for the dtype.
"""
from __future__ import annotations

import numpy as np

from metaltile_amd import DType, pack_f32
from oracle import oracle as o

ODT = {DType.F32: o.F32, DType.F16: o.F16, DType.BF16: o.BF16}
DTYPES = (DType.F32, DType.F16, DType.BF16)
TOL = {DType.F32: 5e-3, DType.F16: 5e-2, DType.BF16: 2e-1}  # quantized.rs:5449


def _u32b(a) -> bytes:
    return np.ascontiguousarray(a, dtype="<u4").tobytes()


def _ramps(count_sb: int, count_x: int):
    """scales 0.004+(i%7)*0.0008, biases ((i%5)-2)*0.0009, x ((i%11)-5)*0.01
    (crates/metaltile-std/src/mlx/quantized.rs:5425-5427), formed in f32."""
    i = np.arange(count_sb)
    s = (np.float32(0.004) + (i % 7).astype(np.float32) * np.float32(0.0008)).astype(np.float32)
    b = (((i % 5).astype(np.float32) - np.float32(2.0)) * np.float32(0.0009)).astype(np.float32)
    j = np.arange(count_x)
    x = (((j % 11).astype(np.float32) - np.float32(5.0)) * np.float32(0.01)).astype(np.float32)
    return s, b, x


def qx_setup(kernel, m, n, k, bits, group_size, has_n, grid, tpg, dt: DType):
    """crates/metaltile-std/src/mlx/quantized.rs:5411-5446."""
    gspr = k // group_size
    w = o.synth_packed_w(n, k, bits)
    s_f, b_f, x_f = _ramps(n * gspr, m * k)
    s, b, x = (o.round_through(v, ODT[dt]) for v in (s_f, b_f, x_f))
    expected = o.qmm(w, s, b, x, m, n, k, bits, group_size)
    consts = {"k": k, "gs_per_row": gspr}
    if has_n:
        consts["n"] = n
    return dict(kernel=kernel, dtype=dt, consts=consts, grid=grid, tpg=tpg, out="out",
                buffers={"w": _u32b(w), "scales": pack_f32(s_f, dt), "biases": pack_f32(b_f, dt),
                         "x": pack_f32(x_f, dt), "out": bytes(m * n * dt.size_bytes)},
                expected=expected, tol=TOL[dt], shape=(m, n, k, bits, group_size))


# name -> (kernel, m, n, k, bits, G, has_n, grid, tpg)   quantized.rs:5449-5605
QX_TESTS = {
    "test_qmv": ("mt_qmv", 1, 32, 512, 4, 64, False, (4, 1, 1), (64, 1, 1)),
    "test_qmv_int8_fast": ("mt_qmv_int8_fast", 1, 32, 512, 8, 64, False, (4, 1, 1), (64, 1, 1)),
    "test_qmm": ("mt_qmm", 8, 16, 512, 4, 64, True, (2, 8, 1), (64, 1, 1)),
    "test_qmm_bm2": ("mt_qmm_bm2", 8, 16, 512, 4, 64, True, (2, 4, 1), (64, 1, 1)),
    "test_qmm_bm4": ("mt_qmm_bm4", 8, 16, 512, 4, 64, True, (2, 2, 1), (64, 1, 1)),
    "test_qmm_int8_fast": ("mt_qmm_int8_fast", 8, 16, 512, 8, 64, True, (2, 8, 1), (64, 1, 1)),
    "test_qmm_bm2_int8_fast": ("mt_qmm_bm2_int8_fast", 8, 16, 512, 8, 64, True, (2, 4, 1), (64, 1, 1)),
    "test_qmm_bm4_int8_fast": ("mt_qmm_bm4_int8_fast", 8, 16, 512, 8, 64, True, (2, 2, 1), (64, 1, 1)),
    "test_qmm_mma": ("mt_qmm_mma", 32, 64, 512, 4, 64, True, (2, 1, 1), (128, 1, 1)),
    "test_qmm_mma_m16": ("mt_qmm_mma_m16", 16, 64, 512, 4, 64, True, (2, 1, 1), (64, 1, 1)),
    "test_qmm_mma_int8": ("mt_qmm_mma_int8", 32, 64, 512, 8, 64, True, (2, 1, 1), (128, 1, 1)),
    "test_qmm_mma_m16_int8": ("mt_qmm_mma_m16_int8", 16, 64, 512, 8, 64, True, (2, 1, 1), (64, 1, 1)),
    "test_qmm_mma_int2": ("mt_qmm_mma_int2", 32, 64, 512, 2, 64, True, (2, 1, 1), (128, 1, 1)),
}


def qx_test(name: str, dt: DType):
    return qx_setup(*QX_TESTS[name], dt)


def gemv_setup(kernel, bits, out_dim, in_dim, group_size, grid_rows, tpg, dt: DType):
    """crates/metaltile-std/src/ffai/dequant_gemv.rs:460-495."""
    ng = in_dim // group_size
    w = o.synth_bitstream_w(out_dim, in_dim, bits)
    s_f, b_f, x_f = _ramps(out_dim * ng, in_dim)
    s, b, x = (o.round_through(v, ODT[dt]) for v in (s_f, b_f, x_f))
    expected = o.qmm(w, s, b, x, 1, out_dim, in_dim, bits, group_size)
    return dict(kernel=kernel, dtype=dt, consts={"in_dim": in_dim, "group_size": group_size},
                grid=(grid_rows, 1, 1), tpg=(tpg, 1, 1), out="output",
                buffers={"weight": _u32b(w), "scales": pack_f32(s_f, dt), "biases": pack_f32(b_f, dt),
                         "input": pack_f32(x_f, dt), "output": bytes(out_dim * dt.size_bytes)},
                expected=expected, tol=TOL[dt], shape=(1, out_dim, in_dim, bits, group_size))


# dequant_gemv.rs:497-542
GEMV_TESTS = {
    "test_dequant_gemv_int2": ("dequant_gemv_int2", 2, 4, 256, 64, 4, 64),
    "test_dequant_gemv_int4": ("dequant_gemv_int4", 4, 4, 256, 64, 4, 64),
    "test_dequant_gemv_int8": ("dequant_gemv_int8", 8, 4, 256, 64, 4, 64),
    "test_dequant_gemv_int3": ("dequant_gemv_int3", 3, 4, 64, 32, 4, 64),
    "test_dequant_gemv_int5": ("dequant_gemv_int5", 5, 4, 64, 32, 4, 64),
    "test_dequant_gemv_int6": ("dequant_gemv_int6", 6, 4, 64, 32, 4, 64),
    "test_dequant_gemv_int4_fast": ("dequant_gemv_int4_fast", 4, 8, 512, 64, 1, 64),
}


def gemv_test(name: str, dt: DType):
    return gemv_setup(*GEMV_TESTS[name], dt)


def expert_indexed_test(dt: DType):
    """crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:186-214."""
    n_experts, out_dim, in_dim, group_size, expert = 4, 4, 256, 64, 2
    ng = in_dim // group_size
    w = o.synth_stacked_w(n_experts, out_dim, in_dim)
    s_f, b_f, x_f = _ramps(n_experts * out_dim * ng, in_dim)
    s, b, x = (o.round_through(v, ODT[dt]) for v in (s_f, b_f, x_f))
    expected = o.expert_indexed(w, s, b, x, expert, out_dim, in_dim, group_size)
    return dict(kernel="dequant_gemv_int4_expert_indexed", dtype=dt,
                consts={"in_dim": in_dim, "out_dim": out_dim, "group_size": group_size},
                grid=(out_dim, 1, 1), tpg=(64, 1, 1), out="output",
                buffers={"weights_stacked": _u32b(w), "scales_stacked": pack_f32(s_f, dt),
                         "biases_stacked": pack_f32(b_f, dt), "input": pack_f32(x_f, dt),
                         "expert_index": _u32b([expert]), "output": bytes(out_dim * dt.size_bytes)},
                expected=expected, tol=TOL[dt], shape=(1, out_dim, in_dim, 4, group_size))


def moe_int4_inputs(dt: DType):
    """crates/metaltile-std/src/ffai/moe.rs:3628-3651: 3 experts, k 64, m 8, g 32, 6 rows."""
    n_experts, k_in, m_out, group_size, t_rows = 3, 64, 8, 32, 6
    offsets = np.array([0, 2, 5, 6], dtype=np.uint32)
    i = np.arange(n_experts * m_out * k_in, dtype=np.uint32)
    codes = ((i * np.uint32(7) + np.uint32(3)) & np.uint32(0xF)).astype(np.uint8)
    w = o.pack_codes(codes.reshape(n_experts * m_out, k_in), 4)
    ng = k_in // group_size
    j = np.arange(n_experts * m_out * ng).astype(np.float32)
    s_f = (np.float32(0.01) + np.float32(0.001) * j).astype(np.float32)
    b_f = (np.float32(-0.05) + np.float32(0.002) * j).astype(np.float32)
    t = np.arange(t_rows * k_in).astype(np.float32)
    x_f = (np.float32(0.1) * np.sin((t * np.float32(0.17)).astype(np.float32)).astype(np.float32)).astype(np.float32)
    return dict(n_experts=n_experts, k_in=k_in, m_out=m_out, group_size=group_size, t_rows=t_rows,
                offsets=offsets, w=w, s_f=s_f, b_f=b_f, x_f=x_f)


def moe_int4_test(kernel: str, grid_x: int, dt: DType):
    """crates/metaltile-std/src/ffai/moe.rs:3624-3695 (CSR ABI)."""
    d = moe_int4_inputs(dt)
    s, b, x = (o.round_through(v, ODT[dt]) for v in (d["s_f"], d["b_f"], d["x_f"]))
    expected = o.gather_qmm(x, d["w"], s, b, d["t_rows"], d["k_in"], d["m_out"], d["n_experts"], 4,
                            d["group_size"], expert_offsets=d["offsets"])
    return dict(kernel=kernel, dtype=dt,
                consts={"k_in": d["k_in"], "m_out": d["m_out"], "n_experts": d["n_experts"],
                        "group_size": d["group_size"]},
                grid=(grid_x, d["t_rows"], 1), tpg=(32, 1, 1), out="out",
                buffers={"x": pack_f32(d["x_f"], dt), "weight_packed": _u32b(d["w"]),
                         "scales": pack_f32(d["s_f"], dt), "biases": pack_f32(d["b_f"], dt),
                         "expert_offsets": _u32b(d["offsets"]),
                         "out": bytes(d["t_rows"] * d["m_out"] * dt.size_bytes)},
                expected=expected, tol=TOL[dt])


def legacy_qmv_f32():
    """crates/metaltile-std/tests/mt_qmv_gpu_correctness.rs:90-140: 32 rows, k 4096,
    rows ((i*7+j)%23-11)*0.02 quantised per group of 64 with round-half-away
    (`.round()`), x ((j*13)%11-5)*0.05; abs tol 5e-3."""
    m, k, g = 32, 4096, 64
    i = np.arange(m)[:, None]
    j = np.arange(k)[None, :]
    rows = ((((i * 7 + j) % 23).astype(np.float32) - np.float32(11.0)) * np.float32(0.02)).astype(np.float32)
    grp = rows.reshape(m, k // g, g)
    mn = grp.min(axis=2, keepdims=True)
    mx = grp.max(axis=2, keepdims=True)
    scale = np.where(np.abs(mx - mn) < 1e-10, np.float32(1.0), ((mx - mn) / np.float32(15.0))).astype(np.float32)
    t = ((grp - mn) / scale).astype(np.float32)
    q = np.clip(np.floor(np.abs(t) + np.float32(0.5)) * np.sign(t), 0, 15).astype(np.uint8)  # f32::round
    w = o.pack_codes(q.reshape(m, k), 4)
    s = scale.reshape(-1).astype(np.float32)
    b = mn.reshape(-1).astype(np.float32)
    jj = np.arange(k)
    x = ((((jj * 13) % 11).astype(np.float32) - np.float32(5.0)) * np.float32(0.05)).astype(np.float32)
    expected = o.qmm(w, s, b, x, 1, m, k, 4, g)
    return dict(kernel="mt_qmv", dtype=DType.F32, consts={"k": k, "gs_per_row": k // g},
                grid=(m // 8, 1, 1), tpg=(64, 1, 1), out="out",
                buffers={"w": _u32b(w), "scales": s.tobytes(), "biases": b.tobytes(), "x": x.tobytes(),
                         "out": bytes(m * 4)},
                expected=expected, tol=5e-3, shape=(1, m, k, 4, g))


def legacy_qmm_inputs(m, n, k, dt: DType):
    """crates/metaltile-std/tests/qmm_gpu_correctness.rs:121-133: nibble (i+bit)&15,
    scales 0.1+0.001i, biases 0.0001i, x 1+0.001i."""
    g = 64
    gspr = k // g
    i = np.arange(n * k // 8, dtype=np.uint32)
    w = np.zeros_like(i)
    for bit in range(8):
        w |= ((i + np.uint32(bit)) & np.uint32(0xF)) << np.uint32(bit * 4)
    s_f = (np.float32(0.1) + np.arange(n * gspr).astype(np.float32) * np.float32(0.001)).astype(np.float32)
    b_f = (np.arange(n * gspr).astype(np.float32) * np.float32(0.0001)).astype(np.float32)
    x_f = (np.float32(1.0) + np.arange(m * k).astype(np.float32) * np.float32(0.001)).astype(np.float32)
    return w, s_f, b_f, x_f, g
