"""The C oracle against the committed golden vectors (tests/golden): inputs and
f64 expected outputs produced by independent big-integer packing code."""
import numpy as np
import pytest

from tests.golden_vectors import load
from tests.parity import rel_err

CASES = load()


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "qmm"], ids=lambda c: c["name"])
def test_qmm_oracles_match_golden(oracle, c):
    args = (c["w"], c["scales"], c["biases"], c["x"], c["M"], c["N"], c["K"], c["bits"], c["G"])
    f64 = oracle.qmm_f64(*args)
    assert rel_err(f64, c["expected"]) <= 5e-6      # w_hat is formed in f32 as the reference does; sums are f64
    seq = oracle.qmm(*args)                         # reference-faithful f32 sequential sum
    assert rel_err(seq, c["expected"]) <= 1e-4
    if c["bits"] in (2, 4, 8):
        assert rel_err(oracle.qmm_split(*args), c["expected"]) <= 1e-4
    codes = oracle.unpack_codes(c["w"], c["N"], c["K"], c["bits"])
    assert np.array_equal(oracle.pack_codes(codes.reshape(c["N"], c["K"]), c["bits"]), c["w"])


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "gather"], ids=lambda c: c["name"])
def test_gather_oracle_matches_golden(oracle, c):
    T = c["M"]
    for view in ("indices", "offsets"):
        got = oracle.gather_qmm(c["x"], c["w"], c["scales"], c["biases"], T, c["K"], c["N"], c["E"], c["bits"],
                                c["G"], **{("indices" if view == "indices" else "expert_offsets"): c[view]},
                                f64=True)
        assert rel_err(got, c["expected"]) <= 5e-6, view


def test_handcheck_vector_is_what_arithmetic_says():
    c = [c for c in CASES if c["name"].endswith("handcheck")][0]
    assert list(c["w"][:2]) == [0x76543210, 0xFEDCBA98]
    assert c["expected"][0] == 0.5 * sum(list(range(16)) * 2) - 4.0 * 32 == -8.0
