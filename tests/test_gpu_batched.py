"""Batched qmv (several weight matrices against one activation row, one launch).

Covers the reference's fused-projection kernels: ffai_batched_qkv_qgemv(_fast)
(crates/metaltile-std/src/ffai/batched_qkv_qgemv.rs:42-59,157-174: Q, K and V written
into one concatenated vector) and ffai_batched_4_qgemv_fast
(crates/metaltile-std/src/ffai/batched_4_qgemv.rs:60-84: four outputs). Each output is
checked against the f64-accumulated oracle (max|a-e|/max(|e|,1) <= 1e-2 for f16/bf16,
1e-4 for f32, the bound of the single-matrix tests) and, for the widths the streaming
kernel serves, must be bit-equal to the single-matrix launch on the same operands.
"""
import numpy as np
import pytest

from metaltile_amd import _lib
from metaltile_amd import DType, GpuBuffer, ops, unpack_f32
from metaltile_amd.synth import make_case
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}

CASES = [
    # dtype, bits, G, K, row counts
    (DType.BF16, 4, 64, 4096, (4096, 1024, 1024)),   # llama-3 8B Q, K, V
    (DType.F16, 4, 64, 4096, (4096, 1024, 1024)),
    (DType.BF16, 4, 64, 4096, (14336, 14336)),        # gate + up
    (DType.BF16, 4, 64, 2048, (2048, 512, 512, 96)),  # four unequal outputs
    (DType.F16, 8, 64, 1024, (256, 256, 64)),
    (DType.BF16, 2, 64, 2048, (512, 384)),
    (DType.BF16, 4, 32, 1024, (130, 7, 64)),          # ragged row counts
    (DType.F32, 4, 64, 1024, (128, 64, 64)),
    (DType.BF16, 4, 64, 576, (64, 64, 64)),           # a row length the streaming kernel refuses: one launch per matrix
    (DType.BF16, 3, 64, 1024, (128, 64, 64)),         # odd width: one launch per matrix
    (DType.BF16, 4, 64, 1024, (96,)),                 # a single matrix is accepted too
]


def _operands(seed, dt, bits, G, K, Ns):
    cases = [make_case(seed + j, dt, bits, G, 1, N, K, bias_rule="midpoint") for j, N in enumerate(Ns)]
    x = GpuBuffer.from_bytes(cases[0].x_bytes)
    dev = [(GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes))
           for c in cases]
    return cases, x, dev


def _expected(oracle, c, x_f, dt):
    exp = oracle.qmm_f64(c.w, c.scales_f, c.biases_f, x_f, 1, c.N, c.K, c.bits, c.group_size, threads=8)
    return oracle.round_through(exp.astype(np.float32), ODT[dt])


def _walks(dt, bits, G, K, Ns):
    """What the kernel whose waves walk the rows takes of a batch: 2 to 4 matrices of 4-bit codes in rows of 2048 ... 8192
    codes in steps of 1024, or 3584, groups of 32 / 64 / 128, f16 / bf16."""
    return bits == 4 and (K == 3584 or (2048 <= K <= 8192 and K % 1024 == 0)) and G in (32, 64, 128) and dt != DType.F32 and 2 <= len(Ns) <= 4


CASES += [
    (DType.F16, 4, 32, 4096, (5, 1030, 77, 4100)),    # the walking kernel, ragged: four matrices, 5212 rows (two per wave and one)
    (DType.BF16, 4, 128, 8192, (1024, 40)),           # rows of 8192 codes, one row per wave
    (DType.BF16, 4, 64, 8192, (8192, 1024, 1027)),    # 10243 rows of 8192 codes: its automatic size
    (DType.F16, 4, 64, 4096, (16, 16)),               # two waves' worth
    (DType.BF16, 4, 64, 3072, (3072, 1024, 1030)),    # rows that end inside a group of 64 chunks: Q, K, V of a 3072-wide model
    (DType.F16, 4, 128, 3584, (3584, 512, 512)),
    (DType.BF16, 4, 32, 5120, (5120, 1024, 1024, 7)),
    (DType.BF16, 4, 64, 7168, (1536, 2050)),
    (DType.F16, 4, 64, 6144, (6144, 1024)),
]


@pytest.mark.parametrize("dt,bits,G,K,Ns", CASES, ids=lambda v: getattr(v, "name", str(v).replace(" ", "")))
def test_batched_matches_single_and_oracle(oracle, dt, bits, G, K, Ns):
    """As routed (qmv.kernel = 0), on the streaming kernel (2) and, where it applies, on the kernel whose waves walk the
    rows (4): against the oracle every time, and bit for bit against the single-matrix launch on the same kernel."""
    print(f"[case] qmv_batched {dt.name} b{bits} g{G} K{K} N{Ns}", flush=True)
    cases, x, dev = _operands(900, dt, bits, G, K, Ns)
    esz = dt.size_bytes
    lib = _lib.load()
    from metaltile_amd import GpuRunner
    for opt in (0, 2, 4):
        if opt == 4 and not _walks(dt, bits, G, K, Ns):
            continue
        outs = [GpuBuffer.from_bytes(b"\xff" * (N * esz + 16)) for N in Ns]  # NaN fill: every element must be written, none after the last
        assert lib.mtq_set_option(b"qmv.kernel", opt) == 0
        try:
            GpuRunner(0).flush_slc()
            ops.qmv_batched(dt, bits, G, [d[0] for d in dev], [d[1] for d in dev], [d[2] for d in dev], x, outs, list(Ns), K)
            for c, d, o, N in zip(cases, dev, outs, Ns):
                whole = o.read_bytes(N * esz + 16)
                raw = whole[:N * esz]
                assert whole[N * esz:] == b"\xff" * 16
                got = unpack_f32(raw, dt)
                assert np.isfinite(got).all()
                assert rel_err(got, _expected(oracle, c, cases[0].x_f, dt)) <= TOL[dt]
                if opt != 0 and bits in (2, 4, 8):
                    # (as routed, a single row of 4096 4-bit codes may take another kernel than the batch, whose f32 sums
                    # meet in another order; with the kernel named, batch and single launch are the same arithmetic)
                    single = GpuBuffer(N * esz)
                    ops.qmv(dt, bits, G, d[0], d[1], d[2], x, single, 1, N, K)
                    assert single.read_bytes(N * esz) == raw, "batched launch must reproduce the single launch bit for bit"
                    single.free()
        finally:
            lib.mtq_set_option(b"qmv.kernel", 0)
        for o in outs:
            o.free()
    for b in [x] + [t for d in dev for t in d]:
        b.free()


@pytest.mark.parametrize("name,n", [("ffai_batched_qkv_qgemv", 3), ("ffai_batched_qkv_qgemv_fast", 3),
                                    ("ffai_batched_4_qgemv_fast", 4)])
@pytest.mark.parametrize("dt", [DType.F16, DType.BF16], ids=lambda d: d.name)
def test_dispatch_by_reference_name(ctx, oracle, name, n, dt):
    bits, G, K = 4, 64, 2048
    Ns = (512, 128, 128, 256)[:n]
    print(f"[case] {name} {dt.name} N{Ns}", flush=True)
    cases = [make_case(950 + j, dt, bits, G, 1, N, K, bias_rule="midpoint") for j, N in enumerate(Ns)]
    bufs = {"x": cases[0].x_bytes}
    consts = {"in_dim": K, "group_size": G}
    tags = "qkv" if n == 3 else "abcd"
    for tag, c, N in zip(tags, cases, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = c.w.tobytes(), c.scales_bytes, c.biases_bytes
        consts[f"out_{tag}"] = N
        if n == 4:
            bufs[f"{tag}_out"] = b"\xff" * (N * dt.size_bytes)
    if n == 3:
        bufs["out"] = b"\xff" * (sum(Ns) * dt.size_bytes)
    res = ctx.dispatch_with_grid(name, dt, bufs, consts, (max(Ns), 1, 1), (32, 1, 1))
    if n == 3:
        parts = np.split(unpack_f32(res.outputs["out"], dt), np.cumsum(Ns)[:-1])
    else:
        parts = [unpack_f32(res.outputs[f"{tag}_out"], dt) for tag in tags]
    for c, got in zip(cases, parts):
        assert got.size == c.N and np.isfinite(got).all()
        assert rel_err(got, _expected(oracle, c, cases[0].x_f, dt)) <= TOL[dt]


def test_batched_rejects_bad_arguments():
    from metaltile_amd import MtqError
    buf = GpuBuffer(4096)
    with pytest.raises(MtqError):
        ops.qmv_batched(DType.BF16, 4, 64, [buf] * 5, [buf] * 5, [buf] * 5, buf, [buf] * 5, [8] * 5, 64)
    with pytest.raises(MtqError):
        ops.qmv_batched(DType.BF16, 4, 64, [buf, 0], [buf, buf], [buf, buf], buf, [buf, buf], [8, 8], 64)
    buf.free()


# ---- the reference's own setups for these kernels -------------------------------------------
# Inputs: the xorshift stream `source(n, seed, scale, off)` and the min/max int4 row quantiser of
# crates/metaltile-std/tests/batched_qkv_qgemv_gpu_correctness.rs:30-110 (the 4-way test,
# batched_4_qgemv_gpu_correctness.rs:40-95, uses the same two), restated in numpy. Expected values:
# the f32 dequant-dot of the same file (lines 73-97), here through the oracle's sequential f32 path.
# Metric and bounds are the reference's: max |a-e| / max(|e|, 1e-3) <= 5e-3 (f32), 2e-2 (f16),
# 5e-2 (bf16) (lines 159-181, 283-292; batched_4_...:302-312).
REF_TOL = {DType.F32: 5e-3, DType.F16: 2e-2, DType.BF16: 5e-2}


def _source(n, seed, scale, off):
    out = np.empty(n, dtype=np.float32)
    s, m = seed, (1 << 64) - 1
    for i in range(n):
        s ^= (s << 13) & m
        s ^= s >> 7
        s ^= (s << 17) & m
        out[i] = (np.float32(s % 20000) / np.float32(20000.0) - np.float32(0.5)) * np.float32(scale) + np.float32(off)
    return out


def _quantize_int4(rows, N, K, G):
    g = rows.reshape(N, K // G, G)
    mn, mx = g.min(axis=2), g.max(axis=2)
    rng = mx - mn
    scale = np.where(np.abs(rng) < 1e-10, np.float32(1.0), rng / np.float32(15.0)).astype(np.float32)
    t = (g - mn[..., None]) / scale[..., None]
    q = np.clip(np.where(t >= 0, np.floor(t + np.float32(0.5)), np.ceil(t - np.float32(0.5))), 0, 15).astype(np.uint32)  # f32::round
    q = q.reshape(N, K // 8, 8)
    packed = np.zeros((N, K // 8), dtype=np.uint32)
    for i in range(8):
        packed |= q[:, :, i] << np.uint32(4 * i)
    return packed.ravel().astype("<u4"), scale.ravel(), mn.ravel().astype(np.float32)


def _ref_case(oracle, dt, K, G, Ns, seeds):
    from metaltile_amd import pack_f32
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    x = rt(_source(K, 0x11, 2.0, 0.05))
    mats = []
    for N, seed in zip(Ns, seeds):
        w, s, b = _quantize_int4(_source(N * K, seed, 3.0, 0.0), N, K, G)
        s, b = rt(s), rt(b)
        exp = oracle.qmm(w, s, b, x, 1, N, K, 4, G)
        mats.append((w, s, b, np.asarray(exp, dtype=np.float32).ravel()))
    return x, mats, pack_f32


def _ref_err(got, exp):
    return float(np.max(np.abs(got - exp) / np.maximum(np.abs(exp), 1e-3)))


QKV_REF = [("ffai_batched_qkv_qgemv", 256, 64, 16, 4, 128), ("ffai_batched_qkv_qgemv", 512, 128, 12, 6, 128),
           ("ffai_batched_qkv_qgemv_fast", 512, 64, 16, 8, 64)]


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("name,K,G,nq,nk,tpg", QKV_REF)
def test_reference_qkv_setups(ctx, oracle, name, K, G, nq, nk, tpg, dt):
    if G == 128 and dt != DType.F32:
        pytest.skip("the reference runs the group-128 case in f32 only")
    Ns = (nq, nk, nk)
    print(f"[case] {name} {dt.name} in_dim={K} g{G} out={Ns}", flush=True)
    x, mats, pack = _ref_case(oracle, dt, K, G, Ns, (0x22, 0x33, 0x44))
    bufs = {"x": pack(x, dt), "out": bytes(sum(Ns) * dt.size_bytes)}
    consts = {"in_dim": K, "group_size": G}
    for tag, (w, s, b, _), N in zip("qkv", mats, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = w.tobytes(), pack(s, dt), pack(b, dt)
        consts[f"out_{tag}"] = N
    grid = (max(Ns) if tpg == 128 else -(-max(Ns) // 8), 1, 3)
    res = ctx.dispatch_with_grid(name, dt, bufs, consts, grid, (tpg, 1, 1))
    got = unpack_f32(res.outputs["out"], dt)
    exp = np.concatenate([m[3] for m in mats])
    assert got.size == sum(Ns) and np.any(got != 0.0)
    assert _ref_err(got, exp) <= REF_TOL[dt]


@pytest.mark.parametrize("dt,K,Ns", [(DType.F32, 2048, (768, 1024, 64, 64)), (DType.F16, 2048, (768, 1024, 64, 64)),
                                     (DType.BF16, 2048, (768, 1024, 64, 64)), (DType.F32, 512, (16, 8, 8, 8))],
                         ids=lambda v: getattr(v, "name", str(v).replace(" ", "")))
def test_reference_4way_setups(ctx, oracle, dt, K, Ns):
    print(f"[case] ffai_batched_4_qgemv_fast {dt.name} in_dim={K} out={Ns}", flush=True)
    x, mats, pack = _ref_case(oracle, dt, K, 64, Ns, (0x22, 0x33, 0x44, 0x55))
    bufs = {"x": pack(x, dt)}
    consts = {"in_dim": K, "group_size": 64}
    for tag, (w, s, b, _), N in zip("abcd", mats, Ns):
        bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = w.tobytes(), pack(s, dt), pack(b, dt)
        bufs[f"{tag}_out"] = bytes(N * dt.size_bytes)
        consts[f"out_{tag}"] = N
    res = ctx.dispatch_with_grid("ffai_batched_4_qgemv_fast", dt, bufs, consts, (-(-max(Ns) // 8), 1, 4), (64, 1, 1))
    for tag, (_, _, _, exp) in zip("abcd", mats):
        got = unpack_f32(res.outputs[f"{tag}_out"], dt)
        assert got.size == exp.size and np.any(got != 0.0)
        assert _ref_err(got, exp) <= REF_TOL[dt]
