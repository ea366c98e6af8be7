"""mtq_qvm_noalloc (the entry point that allocates nothing) against mtq_qvm, through the C-ABI.

Both run the same two kernels; only the home of the f32 partial rows differs (an array inside the
library's code object instead of a library-owned allocation), so the outputs must be bit-identical.
Two calls in a row share the array, the second with a smaller input: stale partial rows of the first
call must not leak into the second. Both are also held to the oracle (1e-2 for bf16, 1e-4 for f32 on
max |a-e| / max(|e|, 1)), and a shape whose partial rows exceed the array must be refused.
"""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, MtqError, ops, pack_f32, unpack_f32
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
ODT = {DType.F32: 0, DType.F16: 1, DType.BF16: 2}
TOL = {DType.F32: 1e-4, DType.F16: 1e-2, DType.BF16: 1e-2}


def _case(oracle, dt, bits, M, N, K, G, seed):
    rng = np.random.default_rng(seed)
    rt = lambda v: oracle.round_through(np.asarray(v, dtype=np.float32), ODT[dt])
    codes = rng.integers(0, 1 << bits, size=(K, N), dtype=np.uint8)
    w = oracle.pack_codes(codes, bits)
    s = rt(0.02 * np.abs(rng.standard_normal((K // G) * N)) + 1e-3)
    b = rt(-(1 << (bits - 1)) * s + rng.standard_normal(s.size) * 1e-3)
    x = rt(rng.standard_normal(M * K))
    _, exp64 = oracle.qvm(w, s, b, x, M, N, K, bits, G)
    exp = oracle.round_through(exp64.astype(np.float32), ODT[dt])
    bufs = (GpuBuffer.from_bytes(w.tobytes()), GpuBuffer.from_bytes(pack_f32(s, dt)), GpuBuffer.from_bytes(pack_f32(b, dt)),
            GpuBuffer.from_bytes(pack_f32(x, dt)))
    return bufs, exp


def _run(fn, dt, bits, G, bufs, M, N, K):
    out = GpuBuffer.from_bytes(b"\xff" * (M * N * dt.size_bytes))
    fn(dt, bits, G, *bufs, out, M, N, K)
    raw = out.read_bytes(M * N * dt.size_bytes)
    out.free()
    return raw


@pytest.mark.parametrize("dt", [DType.BF16, DType.F32], ids=lambda d: d.name)
def test_qvm_noalloc_two_calls_in_a_row(oracle, dt):
    # first call: 4096 x 4096, one row (1 MiB of partial rows); second: a smaller, ragged shape, 3-bit, 2 rows
    for i, (bits, M, N, K, G) in enumerate([(4, 1, 4096, 4096, 64), (3, 2, 96, 1024, 32)]):
        print(f"[case] qvm_noalloc {dt.name} b{bits} g{G} M{M} N{N} K{K}", flush=True)
        bufs, exp = _case(oracle, dt, bits, M, N, K, G, 7100 + i)
        got_static = _run(ops.qvm_noalloc, dt, bits, G, bufs, M, N, K)
        got_plain = _run(ops.qvm, dt, bits, G, bufs, M, N, K)
        assert got_static == got_plain                      # bit-identical with the existing entry point
        vals = unpack_f32(got_static, dt)
        assert np.isfinite(vals).all()
        assert rel_err(vals, exp) <= TOL[dt]
        for b in bufs:
            b.free()


def test_qvm_noalloc_refuses_what_does_not_fit():
    buf = GpuBuffer(4096)
    # 128 rows x 1 slice x 16384 columns x 4 bytes = 8 MiB of partial rows: more than the 4 MiB array
    with pytest.raises(MtqError) as e:
        ops.qvm_noalloc(DType.BF16, 4, 64, buf, buf, buf, buf, buf, 128, 16384, 4096)
    assert e.value.code == -7 and "4194304" in str(e.value)
    with pytest.raises(MtqError):
        ops.qvm_noalloc(DType.BF16, 9, 64, buf, buf, buf, buf, buf, 1, 64, 64)
    buf.free()
