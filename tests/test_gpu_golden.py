"""The HIP path, through the typed C-ABI entry points, against the committed
golden vectors (tests/golden). Tolerance on max|a-e|/max(|e|,1): 1e-4 for f32,
1e-2 for f16/bf16 (the benchmark configurations' bounds), after rounding the
expected value to the element dtype as the store does."""
import numpy as np
import pytest

from metaltile_amd import DType, GpuBuffer, ops, pack_f32, unpack_f32
from tests.golden_vectors import load
from tests.parity import rel_err

pytestmark = pytest.mark.gpu
CASES = load()
DT = {"f32": DType.F32, "f16": DType.F16, "bf16": DType.BF16}
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def _bufs(c, dt):
    return (GpuBuffer.from_bytes(c["w"].tobytes()), GpuBuffer.from_bytes(pack_f32(c["scales"], dt)),
            GpuBuffer.from_bytes(pack_f32(c["biases"], dt)), GpuBuffer.from_bytes(pack_f32(c["x"], dt)))


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "qmm"], ids=lambda c: c["name"])
@pytest.mark.parametrize("entry", [ops.qmv, ops.qmm], ids=["qmv", "qmm"])
def test_qmm_matches_golden(c, entry):
    print(f"[case] {entry.__name__} {c['name']}", flush=True)
    dt = DT[c["dt"]]
    w, s, b, x = _bufs(c, dt)
    out = GpuBuffer(c["M"] * c["N"] * dt.size_bytes)
    entry(dt, c["bits"], c["G"], w, s, b, x, out, c["M"], c["N"], c["K"])
    got = unpack_f32(out.read_bytes(), dt)
    exp = unpack_f32(pack_f32(c["expected"].astype(np.float32), dt), dt)
    assert rel_err(got, exp) <= TOL[c["dt"]]


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "gather"], ids=lambda c: c["name"])
@pytest.mark.parametrize("view", ["indices", "offsets"])
def test_gather_matches_golden(c, view):
    print(f"[case] gather {view} {c['name']}", flush=True)
    dt = DT[c["dt"]]
    w, s, b, x = _bufs(c, dt)
    T = c["M"]
    out = GpuBuffer(T * c["N"] * dt.size_bytes)
    route = GpuBuffer.from_bytes(c[view].astype("<u4").tobytes())
    fn = ops.gather_qmv_indices if view == "indices" else ops.gather_qmv_csr
    fn(dt, c["bits"], c["G"], x, w, s, b, route, out, T, c["N"], c["K"], c["E"])
    got = unpack_f32(out.read_bytes(), dt)
    exp = unpack_f32(pack_f32(c["expected"].astype(np.float32), dt), dt)
    assert rel_err(got, exp) <= TOL[c["dt"]]
