"""MoE routing kernels (router top-k, expert sort, permute, unpermute) against the oracle,
through the C-ABI; setups and bounds follow crates/metaltile-std/tests/moe_gpu_correctness.rs.

Integer outputs (chosen experts, both permutations, CSR bounds, permuted rows) must be equal
bit for bit. Softmax weights: |a-e| < 1e-5 in f32, relative < 5e-3 in f16 and < 2e-2 in bf16
(the reference's bounds, :125-131, :281-284, :517-520). Unpermute in f32 is bit-equal to the
oracle (same operation order, no contraction); f16 / bf16 within one rounding of the output.
The last test chains router -> sort -> permute -> gather_qmv (CSR) -> unpermute on the device
and compares with the same chain of oracle functions.
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}


def _u32(buf, n):
    return np.frombuffer(buf.read_bytes(n * 4), dtype="<u4")


def _ref_logits(n):
    i = np.arange(n, dtype=np.float32)
    return np.fmod(i * np.float32(0.13), np.float32(7.0)) - np.float32(3.5) + i * np.float32(0.001)


def _run_topk(dt, logits, rows, E, k, mode=1):
    lg = GpuBuffer.from_bytes(pack_f32(logits, dt))
    idx, w = GpuBuffer(rows * k * 4), GpuBuffer(rows * k * dt.size_bytes)
    ops.moe_router_topk(dt, lg, idx, w, rows, E, k, mode)
    out = _u32(idx, rows * k).copy(), unpack_f32(w.read_bytes(rows * k * dt.size_bytes), dt)
    for b in (lg, idx, w):
        b.free()
    return out


@pytest.mark.parametrize("rows,E,k,mode", [(8, 64, 4, 1), (16, 128, 8, 1), (16, 128, 8, 0), (5, 60, 6, 1), (3, 1024, 32, 1),
                                            (7, 512, 10, 0), (2, 3, 3, 1), (1000, 128, 8, 1)])
def test_router_topk_f32(oracle, rows, E, k, mode):
    print(f"[case] router_topk f32 rows={rows} E={E} k={k} mode={mode}", flush=True)
    logits = _ref_logits(rows * E) if rows * E < 5000 else np.random.default_rng(E).standard_normal(rows * E).astype(np.float32)
    ridx, rw = oracle.moe_router_topk(logits, rows, E, k, mode)
    idx, w = _run_topk(DType.F32, logits, rows, E, k, mode)
    assert np.array_equal(idx, ridx)
    assert np.max(np.abs(w - rw)) < 1e-5
    sums = w.reshape(rows, k).sum(axis=1)
    assert np.allclose(sums, 1.0, atol=1e-5) if mode == 1 else np.all(sums < 1.0)


@pytest.mark.parametrize("dt,tol", [(DType.F16, 5e-3), (DType.BF16, 2e-2)], ids=lambda v: getattr(v, "name", str(v)))
def test_router_topk_half_types(oracle, dt, tol):
    rows, E, k = 16, 128, 8
    logits = oracle.round_through(np.random.default_rng(5).standard_normal(rows * E).astype(np.float32) * 2.0, ODT[dt])
    ridx, rw = oracle.moe_router_topk(logits, rows, E, k, 1)
    idx, w = _run_topk(dt, logits, rows, E, k)
    assert np.array_equal(idx, ridx)
    assert np.max(np.abs(w - rw) / np.maximum(np.abs(rw), 1e-3)) < tol


def test_router_topk_edge_cases(oracle):
    # tie -> smaller index first; k = 1 -> weight 1; NaN never chosen, +Inf first, no duplicates
    z = np.zeros(8, dtype=np.float32)
    z[2] = z[5] = 3.0
    idx, _ = _run_topk(DType.F32, z, 1, 8, 2)
    assert idx.tolist() == [2, 5]
    idx, w = _run_topk(DType.F32, np.arange(32, dtype=np.float32), 1, 32, 1)
    assert idx.tolist() == [31] and w.tolist() == [1.0]
    E, k = 16, 4
    lg = np.tile(np.arange(E, dtype=np.float32) * np.float32(0.1), 4)
    lg[5] = np.nan
    lg[E + 7] = np.inf
    lg[2 * E + 3] = -np.inf
    lg[3 * E + 2] = np.nan
    lg[3 * E + 11] = np.inf
    idx, _ = _run_topk(DType.F32, lg, 4, E, k)
    ridx, _ = oracle.moe_router_topk(lg, 4, E, k, 1)
    assert np.array_equal(idx, ridx)
    idx = idx.reshape(4, k)
    assert all(len(set(r.tolist())) == k for r in idx)
    assert idx[1, 0] == 7 and idx[3, 0] == 11 and 3 not in idx[2] and 5 not in idx[0] and 2 not in idx[3]


def test_router_rejects_bad_shapes():
    b = GpuBuffer(4096)
    for E, k in ((0, 1), (2000, 4), (64, 0), (64, 33), (4, 5)):
        with pytest.raises(MtqError):
            ops.moe_router_topk(DType.F32, b, b, b, 1, E, k, 1)
    b.free()


@pytest.mark.parametrize("T,k,E", [(1, 8, 128), (16, 2, 8), (37, 6, 60), (512, 8, 128), (4096, 8, 128), (3, 1, 1), (100, 4, 1024),
                                   (10000, 8, 128), (700, 3, 2048), (1000, 8, 4096), (129, 8, 1), (20000, 2, 7)])
def test_sort_by_expert(oracle, T, k, E):
    print(f"[case] moe_sort T={T} k={k} E={E}", flush=True)
    rng = np.random.default_rng(T + k + E)
    idx = np.stack([rng.permutation(E)[:k] if E >= k else rng.integers(0, E, k) for _ in range(T)]).astype("<u4").reshape(-1)
    rsti, rinv, roffs = oracle.moe_sort_by_expert(idx, T, k, E)
    di = GpuBuffer.from_bytes(idx.tobytes())
    sti, inv, offs = GpuBuffer(T * k * 4), GpuBuffer(T * k * 4), GpuBuffer.from_bytes(b"\xff" * ((E + 1) * 4))
    ops.moe_sort_by_expert(di, T, k, E, sti, inv, offs)
    assert np.array_equal(_u32(sti, T * k), rsti)
    assert np.array_equal(_u32(inv, T * k), rinv)
    assert np.array_equal(_u32(offs, E + 1), roffs)
    for b in (di, sti, inv, offs):
        b.free()


def test_sort_network_equals_counting_sort(oracle):
    """Both device sorts give the oracle's permutation (the counting sort serves up to 2048 experts,
    the network up to 32768 entries)."""
    from metaltile_amd.runtime import _ensure_init
    lib = _ensure_init()
    T, k, E = 2000, 8, 128
    idx = np.random.default_rng(4).integers(0, E, T * k).astype("<u4")
    rsti, rinv, roffs = oracle.moe_sort_by_expert(idx, T, k, E)
    di = GpuBuffer.from_bytes(idx.tobytes())
    for mode in (1, 0):
        assert lib.mtq_set_option(b"moe.sort", mode) == 0
        sti, inv, offs = GpuBuffer(T * k * 4), GpuBuffer(T * k * 4), GpuBuffer((E + 1) * 4)
        ops.moe_sort_by_expert(di, T, k, E, sti, inv, offs)
        assert np.array_equal(_u32(sti, T * k), rsti) and np.array_equal(_u32(inv, T * k), rinv)
        assert np.array_equal(_u32(offs, E + 1), roffs)
        for b in (sti, inv, offs):
            b.free()
    di.free()


def test_sort_limits():
    b = GpuBuffer(1 << 20)
    with pytest.raises(MtqError):
        ops.moe_sort_by_expert(b, 4097, 8, 4096, b, b, b)   # 32776 entries and more experts than the counting sort takes
    ops.moe_sort_by_expert(b, 0, 8, 4, b, b, b)             # no entries: offsets all zero
    assert _u32(b, 5).tolist() == [0, 0, 0, 0, 0]
    b.free()


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("T,k,H", [(8, 2, 64), (64, 8, 2048), (5, 3, 100), (7, 2, 33)])
def test_permute_unpermute(oracle, dt, T, k, H):
    print(f"[case] permute/unpermute {dt.name} T={T} k={k} H={H}", flush=True)
    rng = np.random.default_rng(T * 31 + H)
    E = 16
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype("<u4").reshape(-1)
    sti, inv, _ = oracle.moe_sort_by_expert(idx, T, k, E)
    tokens = oracle.round_through(rng.standard_normal(T * H).astype(np.float32), ODT[dt])
    w = oracle.round_through(rng.random(T * k).astype(np.float32), ODT[dt])
    esz = dt.size_bytes
    tb, sb, pb = GpuBuffer.from_bytes(pack_f32(tokens, dt)), GpuBuffer.from_bytes(sti.tobytes()), GpuBuffer(T * k * H * esz)
    ops.moe_permute(dt, tb, sb, pb, T, T * k, H)
    raw = pb.read_bytes(T * k * H * esz)
    exp_perm = oracle.moe_permute(np.frombuffer(pack_f32(tokens, dt), dtype=np.uint8).reshape(T, H * esz), sti, H * esz)
    assert raw == exp_perm.tobytes()
    # unpermute of other data at the permuted positions
    eo = oracle.round_through(rng.standard_normal(T * k * H).astype(np.float32), ODT[dt])
    eb, ib, wb, ob = (GpuBuffer.from_bytes(pack_f32(eo, dt)), GpuBuffer.from_bytes(inv.tobytes()),
                      GpuBuffer.from_bytes(pack_f32(w, dt)), GpuBuffer(T * H * esz))
    ops.moe_unpermute(dt, eb, ib, wb, ob, T, T * k, H, k)
    got = unpack_f32(ob.read_bytes(T * H * esz), dt)
    exp = oracle.round_through(oracle.moe_unpermute(eo, inv, w, T, H, k), ODT[dt])
    assert np.array_equal(got, exp)
    for b in (tb, sb, pb, eb, ib, wb, ob):
        b.free()


def test_permute_out_of_range_source_gives_zero_row():
    dt, H = DType.F32, 8
    tokens = np.arange(2 * H, dtype=np.float32)
    tb, sb, pb = GpuBuffer.from_bytes(tokens.tobytes()), GpuBuffer.from_bytes(np.array([1, 7, 0], dtype="<u4").tobytes()), GpuBuffer(3 * H * 4)
    ops.moe_permute(dt, tb, sb, pb, 2, 3, H)
    got = np.frombuffer(pb.read_bytes(3 * H * 4), dtype=np.float32).reshape(3, H)
    assert np.array_equal(got[0], tokens[H:]) and not got[1].any() and np.array_equal(got[2], tokens[:H])
    for b in (tb, sb, pb):
        b.free()


@pytest.mark.parametrize("name", ["mt_moe_router_topk", "mt_moe_permute", "mt_moe_unpermute"])
def test_dispatch_by_reference_name(ctx, oracle, name):
    dt, T, k, E, H = DType.F32, 8, 4, 64, 96
    rng = np.random.default_rng(1)
    if name == "mt_moe_router_topk":
        logits = _ref_logits(T * E)
        res = ctx.dispatch_with_grid(name, dt, {"router_logits": logits.tobytes(), "indices_out": bytes(T * k * 4),
                                                "weights_out": bytes(T * k * 4)},
                                     {"n_experts": E, "k": k, "norm_topk_prob": 1}, (T, 1, 1), (32, 1, 1))
        ridx, rw = oracle.moe_router_topk(logits, T, E, k, 1)
        assert np.array_equal(np.frombuffer(res.outputs["indices_out"], dtype="<u4"), ridx)
        assert np.max(np.abs(np.frombuffer(res.outputs["weights_out"], dtype="<f4") - rw)) < 1e-5
        return
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype("<u4").reshape(-1)
    sti, inv, _ = oracle.moe_sort_by_expert(idx, T, k, E)
    if name == "mt_moe_permute":
        tokens = rng.standard_normal(T * H).astype(np.float32)
        res = ctx.dispatch_with_grid(name, dt, {"tokens": tokens.tobytes(), "sort_token_idx": sti.tobytes(),
                                                "permuted": bytes(T * k * H * 4)}, {"hidden": H}, (T * k, 1, 1), (128, 1, 1))
        assert res.outputs["permuted"] == oracle.moe_permute(tokens, sti, H).tobytes()
    else:
        eo, w = rng.standard_normal(T * k * H).astype(np.float32), rng.random(T * k).astype(np.float32)
        res = ctx.dispatch_with_grid(name, dt, {"expert_outputs": eo.tobytes(), "inv_perm": inv.tobytes(),
                                                "top_k_weights": w.tobytes(), "out": bytes(T * H * 4)},
                                     {"hidden": H, "k": k}, (T, 1, 1), (128, 1, 1))
        assert res.outputs["out"] == oracle.moe_unpermute(eo, inv, w, T, H, k).tobytes()


@pytest.mark.parametrize("dt", [DType.F32, DType.BF16], ids=lambda d: d.name)
def test_moe_layer_on_device(oracle, dt):
    """router -> sort -> permute -> gather_qmv (CSR) -> unpermute, all on the device."""
    T, E, k, K, N, G, bits = 24, 16, 4, 512, 192, 64, 4
    odt, esz = ODT[dt], dt.size_bytes
    c = make_case(2024, dt, bits, G, T, N, K, E=E, bias_rule="midpoint")
    logits = oracle.round_through(np.random.default_rng(8).standard_normal(T * E).astype(np.float32), odt)
    # oracle chain
    ridx, rw = oracle.moe_router_topk(logits, T, E, k, 1)
    rw = oracle.round_through(rw, odt)
    sti, inv, offs = oracle.moe_sort_by_expert(ridx, T, k, E)
    perm = oracle.moe_permute(c.x_f, sti, K)
    ge = oracle.gather_qmm(perm, c.w, c.scales_f, c.biases_f, T * k, K, N, E, bits, G, expert_offsets=offs, f64=True, threads=8)
    ge = oracle.round_through(ge.astype(np.float32), odt)
    exp = oracle.round_through(oracle.moe_unpermute(ge, inv, rw, T, N, k), odt)
    # device chain
    lg, x = GpuBuffer.from_bytes(pack_f32(logits, dt)), GpuBuffer.from_bytes(c.x_bytes)
    w, s, b = GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes)
    d_idx, d_w = GpuBuffer(T * k * 4), GpuBuffer(T * k * esz)
    d_sti, d_inv, d_offs = GpuBuffer(T * k * 4), GpuBuffer(T * k * 4), GpuBuffer((E + 1) * 4)
    d_perm, d_ge, d_out = GpuBuffer(T * k * K * esz), GpuBuffer(T * k * N * esz), GpuBuffer(T * N * esz)
    ops.moe_router_topk(dt, lg, d_idx, d_w, T, E, k, 1)
    ops.moe_sort_by_expert(d_idx, T, k, E, d_sti, d_inv, d_offs)
    ops.moe_permute(dt, x, d_sti, d_perm, T, T * k, K)
    ops.gather_qmv_csr(dt, bits, G, d_perm, w, s, b, d_offs, d_ge, T * k, N, K, E)
    ops.moe_unpermute(dt, d_ge, d_inv, d_w, d_out, T, T * k, N, k)
    assert np.array_equal(_u32(d_idx, T * k), ridx)
    assert np.array_equal(_u32(d_offs, E + 1), offs)
    got = unpack_f32(d_out.read_bytes(T * N * esz), dt)
    assert rel_err(got, exp) <= (1e-4 if dt == DType.F32 else 2e-2)
    for buf in (lg, x, w, s, b, d_idx, d_w, d_sti, d_inv, d_offs, d_perm, d_ge, d_out):
        buf.free()
