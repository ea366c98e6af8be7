"""Pins the oracle's dtype packers.

Sources of truth: the reference's own unit-test values
(crates/metaltile-std/src/utils.rs:72-127), numpy's IEEE float16 as a second
implementation, exhaustive 16-bit round trips, and hand-computed
ties-to-even cases.
"""
import numpy as np
import pytest

F32, F16, BF16 = 0, 1, 2


def test_reference_unit_values_round_trip(oracle):
    # utils.rs:72-78, 81-87, 97-103
    for vals, dt in (([0.0, 1.5, -2.25, 1024.0], F32), ([0.0, 0.5, -0.5, 2.0], F16),
                     ([1.0, 2.0, -0.5, 0.0], BF16)):
        b = oracle.pack_f32(vals, dt)
        assert len(b) == len(vals) * (4 if dt == F32 else 2)
        assert oracle.unpack_f32(b, dt).tolist() == vals


def test_reference_lossy_f16(oracle):
    # utils.rs:106-110: 0.1 rounds, does not equal
    r = oracle.unpack_f32(oracle.pack_f32([0.1], F16), F16)[0]
    assert abs(r - 0.1) < 1e-3 and r != np.float32(0.1)


def test_reference_scalar_and_empty(oracle):
    # utils.rs:90-94, 113-118, 121-127
    assert oracle.pack_f32([3.5], F32) == np.float32(3.5).tobytes()
    assert len(oracle.pack_f32([1.0], F16)) == 2 and len(oracle.pack_f32([1.0], BF16)) == 2
    for dt in (F32, F16, BF16):
        assert oracle.pack_f32([], dt) == b"" and oracle.unpack_f32(b"", dt).size == 0
    assert oracle.unpack_f32(bytes([0, 0, 128, 63, 7]), F32).tolist() == [1.0]


def test_bf16_exhaustive_round_trip(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = (bits.astype(np.uint32) << 16).view(np.float32)
    finite = np.isfinite(f)
    back = np.frombuffer(oracle.pack_f32(f, BF16), dtype=np.uint16)
    assert np.array_equal(back[finite], bits[finite])
    assert np.array_equal(oracle.unpack_f32(bits.tobytes(), BF16).view(np.uint32), f.view(np.uint32))


def test_bf16_ties_to_even_closed_form(oracle):
    # 1 + 2^-8 is exactly half way between bf16 1.0 (even) and 1.0078125 (odd) -> 1.0
    # 1 + 3*2^-8 is half way between 1.0078125 (odd) and 1.015625 (even) -> 1.015625
    cases = {1.0 + 2.0 ** -8: 1.0, 1.0 + 3 * 2.0 ** -8: 1.015625, 1.0 + 2.0 ** -8 + 2.0 ** -20: 1.0078125,
             -(1.0 + 2.0 ** -8): -1.0, float(np.finfo(np.float32).max): np.inf, 3.3895313892515355e38: 3.3895313892515355e38}
    for v, want in cases.items():
        got = oracle.round_through([v], BF16)[0]
        assert got == np.float32(want), (v, got, want)


def test_f16_matches_numpy_ieee(oracle):
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(20000) * 1e-5).astype(np.float32),     # f16 subnormal range
        (rng.standard_normal(5000) * 3e4).astype(np.float32),       # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.9604645e-8, 2.9802322e-8,
                  2.98023224e-8 * 1.0001, 6.1035156e-5, 6.0975552e-5, np.inf, -np.inf], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.frombuffer(oracle.pack_f32(vals, F16), dtype=np.uint16)
    assert np.array_equal(got, want)


def test_f16_exhaustive_unpack_and_round_trip(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.unpack_f32(bits.tobytes(), F16)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.isnan(got[~ok]).all()
    back = np.frombuffer(oracle.pack_f32(got[ok], F16), dtype=np.uint16)
    assert np.array_equal(back, bits[ok])


def test_f16_ties_to_even_closed_form(oracle):
    # ulp(1.0) in f16 is 2^-10: 1 + 2^-11 ties to 1.0 (even); 1 + 3*2^-11 ties to 1 + 2^-9
    assert oracle.round_through([1.0 + 2.0 ** -11], F16)[0] == np.float32(1.0)
    assert oracle.round_through([1.0 + 3 * 2.0 ** -11], F16)[0] == np.float32(1.0 + 2.0 ** -9)
    # smallest subnormal 2^-24: 2^-25 ties to 0 (even), 1.5*2^-24 ties to 2^-23
    assert oracle.round_through([2.0 ** -25], F16)[0] == 0.0
    assert oracle.round_through([1.5 * 2.0 ** -24], F16)[0] == np.float32(2.0 ** -23)


def test_product_packers_agree_with_oracle(oracle):
    """The product's numpy packers and the oracle's C packers are two independent
    implementations of the same rule; they must agree bit for bit."""
    from metaltile_amd import DType, pack_f32, unpack_f32
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.standard_normal(50000), rng.standard_normal(20000) * 1e-5,
                           rng.standard_normal(20000) * 1e4]).astype(np.float32)
    for dt, odt in ((DType.F32, F32), (DType.F16, F16), (DType.BF16, BF16)):
        assert pack_f32(vals, dt) == oracle.pack_f32(vals, odt)
        b = oracle.pack_f32(vals, odt)
        assert np.array_equal(unpack_f32(b, dt).view(np.uint32), oracle.unpack_f32(b, odt).view(np.uint32))
