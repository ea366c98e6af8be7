"""Dequantising gather (a quantized embedding table) against the oracle, through the C-ABI.

Reference kernels: dequant_gather_int{2,3,4,5,6,8} (crates/metaltile-std/src/ffai/dequant_gather.rs:45-100). The first
block runs the reference's own setups (:187-245: a table of 8 rows from its bit-stream generator, hidden 256 / group 64
for 2-, 4-, 8-bit and hidden 64 / group 32 for 3-, 5-, 6-bit, rows 3 0 7 1 4 4) under the kernels' names with its
absolute bounds 1e-4 (f32), 1e-2 (f16), 1e-1 (bf16); the arithmetic is one multiply-add per element rounded to the
element type, so the outputs are in fact held bit-equal to the oracle's rounded values. The second block: embedding-
sized tables, 7-bit codes, ids past the table (those output rows keep their bytes), no tokens.
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
REF_ABS = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-1}


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits,hidden,G", [(2, 256, 64), (4, 256, 64), (8, 256, 64), (3, 64, 32), (5, 64, 32), (6, 64, 32)])
def test_reference_setups(ctx, oracle, dt, bits, hidden, G):
    print(f"[case] dequant_gather_int{bits} {dt.name} hidden={hidden} g{G}", flush=True)
    vocab, ids = 8, np.array([3, 0, 7, 1, 4, 4], dtype="<u4")
    ng = hidden // G
    w = oracle.synth_bitstream_w(vocab, hidden, bits)
    s = oracle.round_through((0.02 + (np.arange(vocab * ng) % 7) * 0.01).astype(np.float32), ODT[dt])
    b = oracle.round_through((((np.arange(vocab * ng) % 5).astype(np.float32) - 2.0) * 0.05).astype(np.float32), ODT[dt])
    exp = oracle.dequant_gather(w, s, b, ids, vocab, hidden, G, bits).reshape(-1)
    bufs = {"weight": w.tobytes(), "scales": pack_f32(s, dt), "biases": pack_f32(b, dt), "indices": ids.tobytes(),
            "out": bytes(ids.size * hidden * dt.size_bytes)}
    n = ids.size * hidden
    res = ctx.dispatch_with_grid(f"dequant_gather_int{bits}", dt, bufs, {"hidden": hidden, "group_size": G}, (-(-n // 256), 1, 1), (256, 1, 1))
    got = unpack_f32(res.outputs["out"], dt)
    assert got.size == n and np.max(np.abs(got - exp)) <= REF_ABS[dt]
    assert res.outputs["out"] == pack_f32(exp, dt)


@pytest.mark.parametrize("dt", [DType.F32, DType.F16, DType.BF16], ids=lambda d: d.name)
@pytest.mark.parametrize("bits,vocab,hidden,G,T", [(4, 1000, 4096, 64, 300), (8, 257, 2048, 128, 33), (2, 64, 1024, 32, 1000), (3, 50, 1536, 32, 77),
                                                   (6, 31, 512, 64, 9), (7, 20, 256, 32, 40), (5, 9, 2048, 64, 2048), (4, 3, 8, 8, 5)])
def test_tables(oracle, dt, bits, vocab, hidden, G, T):
    print(f"[case] dequant_gather {dt.name} b{bits} vocab{vocab} hidden{hidden} g{G} T{T}", flush=True)
    rng = np.random.default_rng(bits * 1000 + vocab + T)
    ng = hidden // G
    w = rng.integers(0, 2 ** 32, size=vocab * hidden * bits // 32, dtype=np.uint32)
    s = oracle.round_through((0.02 * np.abs(rng.standard_normal(vocab * ng)) + 1e-3).astype(np.float32), ODT[dt])
    b = oracle.round_through((0.1 * rng.standard_normal(vocab * ng)).astype(np.float32), ODT[dt])
    ids = rng.integers(0, vocab, size=T, dtype=np.uint32)
    ids[:: max(T // 7, 1)] = vocab - 1                      # the table's last row, several times
    exp = oracle.dequant_gather(w, s, b, ids, vocab, hidden, G, bits).reshape(-1)
    wb, sb, bb, ib = (GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s, dt)), GpuBuffer.from_bytes(pack_f32(b, dt)),
                      GpuBuffer.from_bytes(ids.astype("<u4").tobytes()))
    out = GpuBuffer.from_bytes(b"\xab" * (T * hidden * dt.size_bytes))
    ops.dequant_gather(dt, bits, G, wb, sb, bb, ib, out, T, hidden, vocab)
    raw = out.read_bytes()
    assert raw == pack_f32(exp, dt)                         # one multiply-add per element: bit-equal
    # ids past the table: those rows keep their bytes, the others do not change
    bad = ids.copy()
    bad[0] = vocab
    bad[T // 2] = 0xFFFFFFFF
    ib.upload(bad.astype("<u4").tobytes())
    out.upload(np.frombuffer(b"\xab" * (T * hidden * dt.size_bytes), dtype=np.uint8))
    ops.dequant_gather(dt, bits, G, wb, sb, bb, ib, out, T, hidden, vocab)
    raw2 = out.read_bytes()
    rb = hidden * dt.size_bytes
    for t in range(T):
        if t in (0, T // 2):
            assert raw2[t * rb:(t + 1) * rb] == b"\xab" * rb, t
        else:
            assert raw2[t * rb:(t + 1) * rb] == raw[t * rb:(t + 1) * rb], t
    for buf in (wb, sb, bb, ib, out):
        buf.free()


def test_arguments():
    dt, one = DType.BF16, GpuBuffer(4096)
    ops.dequant_gather(dt, 4, 64, one, one, one, one, one, 0, 256, 8)      # no tokens: nothing to do
    for bits, G, H, vocab in ((1, 64, 256, 8), (9, 64, 256, 8), (4, 0, 256, 8), (4, 64, 0, 8), (4, 64, 256, 0), (4, 64, 96, 8), (3, 32, 48, 8),
                              (4, 4, 64, 8)):
        with pytest.raises(MtqError):
            ops.dequant_gather(dt, bits, G, one, one, one, one, one, 4, H, vocab)
    with pytest.raises(MtqError):
        ops.dequant_gather(dt, 4, 64, 0, one, one, one, one, 4, 256, 8)
    one.free()
