"""Pins the oracle's arithmetic: extraction, qmm/gemv, gather, quantise, stats.

Nothing here retypes the oracle's formula: checks are a library f64 matmul on
an independently unpacked matrix, closed forms, brute force on tiny inputs and
identities the reference's own tests rely on.
"""
import numpy as np
import pytest

F32, F16, BF16 = 0, 1, 2


def _rand_case(rng, n, k, bits, g, m):
    codes = rng.integers(0, 1 << bits, size=(n, k), dtype=np.uint8)
    s = (0.02 * np.abs(rng.standard_normal(n * (k // g))) + 1e-3).astype(np.float32)
    b = (-(1 << (bits - 1)) * s + rng.standard_normal(s.size).astype(np.float32) * 1e-3).astype(np.float32)
    x = rng.standard_normal(m * k).astype(np.float32)
    return codes, s, b, x


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_extraction_brute_force_and_round_trip(oracle, bits):
    rng = np.random.default_rng(bits)
    n, k = 5, 64
    codes = rng.integers(0, 1 << bits, size=(n, k), dtype=np.uint8)
    w = oracle.pack_codes(codes, bits)
    assert w.size == n * k * bits // 32
    # pure-Python reader of the format definition: bit string, LSB first
    for r in range(n):
        words = w[r * (k * bits // 32):(r + 1) * (k * bits // 32)]
        big = sum(int(v) << (32 * i) for i, v in enumerate(words))
        for j in range(k):
            assert (big >> (j * bits)) & ((1 << bits) - 1) == codes[r, j]
    assert np.array_equal(oracle.unpack_codes(w, n, k, bits), codes)
    assert np.array_equal(oracle.np_unpack_codes(w, n, k, bits), codes)


def test_synth_packed_w_closed_form(oracle):
    # quantized.rs:5355-5369: slot s of pack p holds (p*2654435761 + s) & mask
    for bits in (2, 4, 8):
        n, k = 3, 64
        w = oracle.synth_packed_w(n, k, bits)
        pf = 32 // bits
        codes = oracle.np_unpack_codes(w, n, k, bits).reshape(-1)
        for idx in (0, 1, pf - 1, pf, 5 * pf + 3, codes.size - 1):
            p, s = divmod(idx, pf)
            assert codes[idx] == ((p * 2654435761 + s) & 0xFFFFFFFF) & ((1 << bits) - 1)


def test_synth_bitstream_matches_packed_layout_for_pow2(oracle):
    # the bit-stream layout and the pack-aligned layout coincide for 2/4/8 bits
    for bits in (2, 4, 8):
        w = oracle.synth_bitstream_w(4, 64, bits)
        codes = oracle.np_unpack_codes(w, 4, 64, bits)
        for row, d in ((0, 0), (1, 7), (3, 63)):
            want = (((row * 64 + d) * 2654435761 + d) & 0xFFFFFFFF) & ((1 << bits) - 1)
            assert codes[row, d] == want


@pytest.mark.parametrize("bits,g", [(2, 32), (2, 64), (3, 32), (4, 32), (4, 64), (4, 128), (5, 32), (6, 32), (8, 64), (8, 128)])
def test_qmm_against_numpy_f64_matmul(oracle, bits, g):
    rng = np.random.default_rng(100 + bits * 7 + g)
    m, n, k = 3, 24, 256
    codes, s, b, x = _rand_case(rng, n, k, bits, g, m)
    w = oracle.pack_codes(codes, bits)
    ref = oracle.np_qmm_f64(w, s, b, x, m, n, k, bits, g).reshape(-1)
    got64 = oracle.qmm_f64(w, s, b, x, m, n, k, bits, g)
    got32 = oracle.qmm(w, s, b, x, m, n, k, bits, g)
    # the f64 oracle sums the same f32 weights as the library matmul: ~1e-13 apart
    assert np.max(np.abs(got64 - ref)) < 1e-9
    # sequential f32 accumulation over 256 terms of |.|~1: a few 1e-5
    assert np.max(np.abs(got32 - ref)) < 2e-4
    # a transposed operand, a dropped bias or a wrong group would be O(1) off
    assert np.max(np.abs(ref)) > 0.5


def test_qmm_closed_forms(oracle):
    n, k, g, m = 6, 128, 32, 2
    rng = np.random.default_rng(5)
    x = rng.standard_normal(m * k).astype(np.float32)
    s = (rng.random(n * k // g) + 0.5).astype(np.float32)
    b = rng.standard_normal(n * k // g).astype(np.float32)
    xg = x.reshape(m, k // g, g).astype(np.float64).sum(axis=2)            # [m, groups]
    # all codes zero -> y = sum_g b_g * sum_{k in g} x_k
    w0 = oracle.pack_codes(np.zeros((n, k), np.uint8), 4)
    want = xg @ b.reshape(n, k // g).astype(np.float64).T
    assert np.max(np.abs(oracle.qmm_f64(w0, s, b, x, m, n, k, 4, g).reshape(m, n) - want)) < 1e-9
    # scale 1, bias 0, constant code c -> y = c * sum(x)
    for bits, c in ((2, 3), (4, 9), (8, 200)):
        wc = oracle.pack_codes(np.full((n, k), c, np.uint8), bits)
        ones, zeros = np.ones(n * k // g, np.float32), np.zeros(n * k // g, np.float32)
        y = oracle.qmm_f64(wc, ones, zeros, x, m, n, k, bits, g).reshape(m, n)
        assert np.max(np.abs(y - c * x.reshape(m, k).astype(np.float64).sum(axis=1, keepdims=True))) < 1e-9


def test_qmm_linearity_and_m1_equals_qmv(oracle):
    rng = np.random.default_rng(9)
    n, k, g, bits = 16, 256, 64, 4
    codes, s, b, x = _rand_case(rng, n, k, bits, g, 2)
    w = oracle.pack_codes(codes, bits)
    x1, x2 = x[:k], x[k:]
    y1 = oracle.qmm_f64(w, s, b, x1, 1, n, k, bits, g)
    y2 = oracle.qmm_f64(w, s, b, x2, 1, n, k, bits, g)
    y12 = oracle.qmm_f64(w, s, b, (2.0 * x1 - 0.5 * x2).astype(np.float32), 1, n, k, bits, g)
    assert np.max(np.abs(y12 - (2.0 * y1 - 0.5 * y2))) < 1e-5
    # rows of an M=2 qmm are the two qmv results, bit for bit (tests/qmm_gpu_correctness.rs:341)
    both = oracle.qmm(w, s, b, x, 2, n, k, bits, g).reshape(2, n)
    assert np.array_equal(both[0], oracle.qmm(w, s, b, x1, 1, n, k, bits, g))
    assert np.array_equal(both[1], oracle.qmm(w, s, b, x2, 1, n, k, bits, g))


def test_split_form_equals_direct_form(oracle):
    # cpu_qmm_reference (tests/qmm_gpu_correctness.rs:73-108) vs qmm_oracle: same sum, f32 rounding apart
    from tests.ref_setups import legacy_qmm_inputs
    from metaltile_amd import DType
    m, n, k = 8, 16, 512
    w, s, b, x, g = legacy_qmm_inputs(m, n, k, DType.F32)
    direct = oracle.qmm(w, s, b, x, m, n, k, 4, g)
    split = oracle.qmm_split(w, s, b, x, m, n, k, 4, g)
    ref = oracle.np_qmm_f64(w, s, b, x, m, n, k, 4, g).reshape(-1)
    assert np.max(np.abs(direct - ref) / np.maximum(np.abs(ref), 1.0)) < 1e-5
    assert np.max(np.abs(split - ref) / np.maximum(np.abs(ref), 1.0)) < 1e-5
    assert ref.min() > 100.0  # the legacy inputs give large positive sums


def test_mma_variant_rounds_weights(oracle):
    rng = np.random.default_rng(21)
    m, n, k, g, bits = 4, 8, 128, 64, 4
    codes, s, b, x = _rand_case(rng, n, k, bits, g, m)
    w = oracle.pack_codes(codes, bits)
    for dt in (F16, BF16):
        wd = oracle.round_through(oracle.np_dequant(w, s, b, n, k, bits, g).reshape(-1), dt).reshape(n, k)
        want = x.reshape(m, k).astype(np.float64) @ wd.astype(np.float64).T
        got = oracle.qmm_mma(w, s, b, x, m, n, k, bits, g, dt).reshape(m, n)
        assert np.max(np.abs(got - want)) < 1e-9
    exact = oracle.qmm_f64(w, s, b, x, m, n, k, bits, g)
    assert np.max(np.abs(oracle.qmm_mma(w, s, b, x, m, n, k, bits, g, F32) - exact)) < 1e-12


def test_csr_expert_resolution(oracle):
    # moe.rs:376-385: first e with t < off[e+1], default 0
    off = [0, 2, 5, 6]
    assert [oracle.csr_expert(off, 3, t) for t in range(8)] == [0, 0, 1, 1, 1, 2, 0, 0]
    assert [oracle.csr_expert([0, 0, 3, 3], 3, t) for t in range(4)] == [1, 1, 1, 0]


def test_gather_identities(oracle):
    rng = np.random.default_rng(33)
    E, N, K, g, bits, T = 4, 12, 128, 32, 4, 9
    codes = rng.integers(0, 16, size=(E * N, K), dtype=np.uint8)
    w = oracle.pack_codes(codes, bits)
    s = (0.02 * np.abs(rng.standard_normal(E * N * K // g)) + 1e-3).astype(np.float32)
    b = (-8 * s).astype(np.float32)
    x = rng.standard_normal(T * K).astype(np.float32)
    off = np.array([0, 3, 3, 7, 9], dtype=np.uint32)
    idx = np.array([0, 0, 0, 2, 2, 2, 2, 3, 3], dtype=np.uint32)
    y_csr = oracle.gather_qmm(x, w, s, b, T, K, N, E, bits, g, expert_offsets=off).reshape(T, N)
    y_idx = oracle.gather_qmm(x, w, s, b, T, K, N, E, bits, g, indices=idx).reshape(T, N)
    assert np.array_equal(y_csr, y_idx)                      # CSR == indices after expansion
    wpe, spe = N * K * bits // 32, N * K // g
    for t in range(T):                                       # each row == plain qmv on its slab
        e = int(idx[t])
        want = oracle.qmm(w[e * wpe:(e + 1) * wpe], s[e * spe:(e + 1) * spe], b[e * spe:(e + 1) * spe],
                          x[t * K:(t + 1) * K], 1, N, K, bits, g)
        assert np.array_equal(y_idx[t], want)
    perm = rng.permutation(T)                                # permuting rows permutes outputs
    y_perm = oracle.gather_qmm(x.reshape(T, K)[perm].ravel(), w, s, b, T, K, N, E, bits, g,
                               indices=idx[perm]).reshape(T, N)
    assert np.array_equal(y_perm, y_idx[perm])
    # expert-indexed(e) == row of the gather with that expert (dequant_gemv_expert_indexed.rs:47-53)
    e = 2
    y_e = oracle.expert_indexed(w, s, b, x[:K], e, N, K, g)
    assert np.array_equal(y_e, oracle.gather_qmm(x[:K], w, s, b, 1, K, N, E, bits, g,
                                                 indices=np.array([e], np.uint32)))
    # f64 variant agrees with numpy on the slab
    y64 = oracle.gather_qmm(x, w, s, b, T, K, N, E, bits, g, indices=idx, f64=True).reshape(T, N)
    ref = oracle.np_qmm_f64(w[2 * wpe:3 * wpe], s[2 * spe:3 * spe], b[2 * spe:3 * spe], x[3 * K:4 * K], 1, N, K, bits, g)
    assert np.max(np.abs(y64[3] - ref.reshape(-1))) < 1e-9


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_affine_quantize_round_trip(oracle, bits):
    # quantized.rs:5283-5284 ramp; round trip within one step (affine_int2_gpu_correctness.rs:134-144)
    g = 64 if bits in (2, 4, 8) else 32
    n_groups = 8
    i = np.arange(n_groups * g)
    v = (((i % 37).astype(np.float32) - 18.0) * np.float32(0.05)).astype(np.float32)
    codes, s, b = oracle.affine_quantize(v, g, bits, F32)
    grp = v.reshape(n_groups, g)
    assert np.allclose(b, grp.min(axis=1)) and np.allclose(s, (grp.max(axis=1) - grp.min(axis=1)) / ((1 << bits) - 1))
    assert codes.max() <= (1 << bits) - 1
    w = oracle.pack_codes(codes.reshape(1, -1), bits)
    back = oracle.affine_dequantize(w, s, b, v.size, g, bits)
    assert np.max(np.abs(back - v) / np.repeat(s, g)) <= 0.5 + 1e-4
    # constant group -> scale 1, bias = the constant, all codes 0
    c, s1, b1 = oracle.affine_quantize(np.full(g, 0.25, np.float32), g, bits, F32)
    assert s1[0] == 1.0 and b1[0] == 0.25 and not c.any()


def test_bench_stats_reference_values(oracle):
    # stats.rs:57-84
    st = oracle.bench_stats([1.0, 2.0, 3.0, 4.0, 10.0])
    assert (st["min_us"], st["median_us"], st["p95_us"], st["p99_us"]) == (1.0, 3.0, 10.0, 10.0)
    assert st["stddev_us"] > 0
    slow = oracle.bench_stats([250.0] * 5 + [120.0] * 5)
    fast = oracle.bench_stats([250.0] * 4 + [120.0] * 6)
    assert slow["median_us"] - fast["median_us"] >= 100.0 and slow["min_us"] == fast["min_us"] == 120.0
    assert abs(st["mean_us"] - 4.0) < 1e-12 and abs(st["stddev_us"] - np.std([1, 2, 3, 4, 10])) < 1e-12


@pytest.mark.parametrize("bits", [4, 8])
def test_rms_norm_qgemv_against_numpy_and_closed_forms(oracle, bits):
    """Fused RMSNorm + GEMV: (a) equals a library matmul of the independently unpacked weight
    matrix with a numpy-normalised row; (b) a constant row c with unit norm weights has
    inv_rms = 1/sqrt(c^2+eps) in closed form, so the output is qmv(w, ones) * c * inv_rms;
    (c) scaling x by 4 leaves the output unchanged when eps = 0 (a dropped 1/in_dim or a
    missing square root breaks this); (d) eps >> mean(x^2) gives out ~ qmv(x*nw)/sqrt(eps)."""
    rng = np.random.default_rng(4242 + bits)
    n, k, g = 12, 256, 64
    codes, s, b, x = _rand_case(rng, n, k, bits, g, 1)
    nw = (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    w = oracle.pack_codes(codes, bits)
    eps = np.float32(1e-5)
    out32, out64, normed = oracle.rms_norm_qgemv(w, s, b, x, nw, k, g, n, bits, eps)
    # (a) numpy in f64 throughout
    xd, nwd = x.astype(np.float64), nw.astype(np.float64)
    inv = 1.0 / np.sqrt(np.mean(xd * xd) + float(eps))
    wd = oracle.np_dequant(w, s, b, n, k, bits, g).astype(np.float64).reshape(n, k)
    ref = wd @ (xd * nwd * inv)
    assert np.max(np.abs(normed - xd * nwd * inv)) < 1e-5
    assert np.max(np.abs(out64 - ref)) < 1e-4
    assert np.max(np.abs(out32 - ref)) < 5e-4
    assert np.max(np.abs(ref)) > 0.3
    # (b) constant row, unit weights
    c = np.float32(0.75)
    xc, ones = np.full(k, c, dtype=np.float32), np.ones(k, dtype=np.float32)
    o32, o64, _ = oracle.rms_norm_qgemv(w, s, b, xc, ones, k, g, n, bits, eps)
    rowsum = oracle.qmm_f64(w, s, b, ones, 1, n, k, bits, g)
    assert np.max(np.abs(o64 - rowsum * float(c) / np.sqrt(float(c) ** 2 + float(eps)))) < 1e-4
    # (c) scale invariance at eps = 0
    a32, a64, _ = oracle.rms_norm_qgemv(w, s, b, x, nw, k, g, n, bits, np.float32(0.0))
    b32, b64, _ = oracle.rms_norm_qgemv(w, s, b, 4.0 * x, nw, k, g, n, bits, np.float32(0.0))
    assert np.max(np.abs(a64 - b64)) < 1e-5
    # (d) large eps
    big = np.float32(1e6)
    d32, d64, _ = oracle.rms_norm_qgemv(w, s, b, x, nw, k, g, n, bits, big)
    plain = oracle.qmm_f64(w, s, b, x * nw, 1, n, k, bits, g)
    assert np.max(np.abs(d64 * 1e3 - plain)) < 1e-4 * max(1.0, np.max(np.abs(plain)))


def test_gated_rms_norm_qgemv_against_numpy_and_closed_forms(oracle):
    """Fused gated RMSNorm + 4-bit GEMV (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:322-366): (a) equals a
    library matmul of the independently unpacked weight matrix with a numpy-gated, numpy-normalised activation (the
    gate through the library's logistic function); (b) one row whose gate is the same everywhere is that gate times
    the pinned RMSNorm GEMV; (c) z = 0 gives zero; (d) silu(ln 3) = 0.75 ln 3; (e) scaling ONE row of y leaves the
    output unchanged at eps = 0 (a sum of squares over all rows, or a division by hv * dv, breaks this); (f) the norm
    weights repeat per row (indexing them by r * dv + d instead of d breaks (a) already: they differ along d)."""
    from scipy.special import expit
    rng = np.random.default_rng(515)
    hv, dv, n, g = 4, 96, 12, 64
    k = hv * dv
    codes, s, b, _ = _rand_case(rng, n, k, 4, g, 1)
    w = oracle.pack_codes(codes, 4)
    y = (rng.standard_normal((hv, dv)) * np.array([0.3, 1.0, 2.5, 7.0])[:, None]).astype(np.float32)
    z = (1.5 * rng.standard_normal((hv, dv))).astype(np.float32)
    nw = (1.0 + 0.2 * rng.standard_normal(dv)).astype(np.float32)
    eps = np.float32(1e-5)
    out32, out64, inner = oracle.gated_rms_norm_qgemv(w, s, b, y, z, nw, hv, dv, g, n, eps)
    # (a) numpy in f64 throughout
    yd, zd, nwd = y.astype(np.float64), z.astype(np.float64), nw.astype(np.float64)
    inv = 1.0 / np.sqrt(np.mean(yd * yd, axis=1, keepdims=True) + float(eps))
    ref_inner = (yd * inv * nwd[None, :] * (zd * expit(zd))).reshape(-1)
    wd = oracle.np_dequant(w, s, b, n, k, 4, g).astype(np.float64).reshape(n, k)
    ref = wd @ ref_inner
    assert np.max(np.abs(inner - ref_inner)) < 1e-5 * max(1.0, np.max(np.abs(ref_inner)))
    assert np.max(np.abs(out64 - ref)) < 1e-4 and np.max(np.abs(out32 - ref)) < 1e-3
    assert np.max(np.abs(ref)) > 0.3
    # (b) one row, constant gate: silu(z0) x rms_norm_qgemv
    z0 = np.float32(0.8)
    y1 = rng.standard_normal(k).astype(np.float32)
    nwk = (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    _, g64, _ = oracle.gated_rms_norm_qgemv(w, s, b, y1, np.full(k, z0, np.float32), nwk, 1, k, g, n, eps)
    _, r64, _ = oracle.rms_norm_qgemv(w, s, b, y1, nwk, k, g, n, 4, eps)
    assert np.max(np.abs(g64 - r64 * float(z0) * float(expit(np.float64(z0))))) < 1e-4
    # (c) closed gates
    o32, o64, _ = oracle.gated_rms_norm_qgemv(w, s, b, y, np.zeros_like(z), nw, hv, dv, g, n, eps)
    assert not o32.any() and not o64.any()
    # (d) silu(ln 3) = ln 3 / (1 + 1/3)
    _, _, one = oracle.gated_rms_norm_qgemv(w, s, b, np.ones_like(y), np.full_like(z, np.log(3.0)), np.ones_like(nw), hv, dv, g, n,
                                            np.float32(0.0))
    assert np.max(np.abs(one - 0.75 * np.log(3.0))) < 1e-6
    # (e) per-row scale invariance at eps = 0
    y4 = y.copy()
    y4[2] *= 4.0
    _, a64, _ = oracle.gated_rms_norm_qgemv(w, s, b, y, z, nw, hv, dv, g, n, np.float32(0.0))
    _, b64, _ = oracle.gated_rms_norm_qgemv(w, s, b, y4, z, nw, hv, dv, g, n, np.float32(0.0))
    assert np.max(np.abs(a64 - b64)) < 1e-5


def _ref_source(n, seed, scale, off):
    """The deterministic generator of the reference's test (gated_rms_norm_qgemv.rs:308-318): xorshift64 on a u64,
    ((s % 20000) as f32 / 20000 - 0.5) * scale + off in f32."""
    out = np.empty(n, dtype=np.float32)
    s, m = seed, (1 << 64) - 1
    for i in range(n):
        s ^= (s << 13) & m
        s ^= s >> 7
        s ^= (s << 17) & m
        out[i] = (np.float32(s % 20000) / np.float32(20000.0) - np.float32(0.5)) * np.float32(scale) + np.float32(off)
    return out


def _ref_quantize_int4_rows(rows, g):
    """The reference test's per-row quantiser (gated_rms_norm_qgemv.rs:283-305): scale = (max - min) / 15 (1 for a flat
    group), bias = min, q = round((v - min) / scale) clamped to 0..15, half away from zero."""
    n, k = rows.shape
    grp = rows.reshape(n, k // g, g)
    mn, mx = grp.min(axis=2), grp.max(axis=2)
    rng_ = mx - mn
    scale = np.where(np.abs(rng_) < 1e-10, np.float32(1.0), rng_ / np.float32(15.0)).astype(np.float32)
    t = (grp - mn[:, :, None]) / scale[:, :, None]
    q = np.clip(np.floor(t + np.float32(0.5)), 0, 15).astype(np.uint8)   # t >= 0: half away from zero == floor(t + 0.5)
    return q.reshape(n, k), scale.reshape(-1), mn.astype(np.float32).reshape(-1)


def test_gated_rms_norm_qgemv_on_the_reference_test_setup(oracle):
    """The reference's own test (gated_rms_norm_qgemv.rs:372-432: hv 4, dv 128, out_dim 512, g 64, eps 1e-5, inputs from
    its xorshift generator and its per-row quantiser) holds no numbers, only generators: restated here, with the
    expectation composed of pieces pinned elsewhere (the gated, normalised activation from numpy, the dot from the
    pinned plain GEMV oracle), as the reference states the kernel's contract (:62-72)."""
    from scipy.special import expit
    hv, dv, n, g = 4, 128, 512, 64
    k = hv * dv
    y = _ref_source(k, 0xA1, 2.0, 0.1)
    z = oracle.round_through(_ref_source(k, 0xD4, 1.5, 0.0), 2)
    nw = oracle.round_through(_ref_source(dv, 0xB2, 0.4, 1.0), 2)
    assert abs(float(y.mean()) - 0.1) < 0.05 and 1.9 < float(y.max() - y.min()) <= 2.0   # the generator's range
    codes, s, b = _ref_quantize_int4_rows(_ref_source(n * k, 0xC3, 3.0, 0.0).reshape(n, k), g)
    s, b = oracle.round_through(s, 2), oracle.round_through(b, 2)
    w = oracle.pack_codes(codes, 4)
    out32, out64, inner = oracle.gated_rms_norm_qgemv(w, s, b, y, z, nw, hv, dv, g, n, np.float32(1e-5))
    yd, zd = y.astype(np.float64).reshape(hv, dv), z.astype(np.float64).reshape(hv, dv)
    ref_inner = (yd / np.sqrt(np.mean(yd * yd, axis=1, keepdims=True) + 1e-5) * nw.astype(np.float64)[None, :] * zd * expit(zd)).reshape(-1)
    assert np.max(np.abs(inner - ref_inner)) < 1e-5
    plain = oracle.qmm_f64(w, s, b, ref_inner.astype(np.float32), 1, n, k, 4, g).reshape(-1)
    assert np.max(np.abs(out64 - plain)) < 1e-3 and np.max(np.abs(out32 - plain)) < 5e-3   # the reference's f32 band: 5e-3
    assert np.max(np.abs(plain)) > 1.0


@pytest.mark.parametrize("bits,hidden,g", [(2, 256, 64), (4, 256, 64), (8, 256, 64), (3, 64, 32), (5, 64, 32), (6, 64, 32)])
def test_dequant_gather_brute_force_on_the_reference_table(oracle, bits, hidden, g):
    """The reference test's table (crates/metaltile-std/src/ffai/dequant_gather.rs:187-215: 8 rows from its bit-stream
    generator, scales 0.02 + (i % 7) * 0.01, biases ((i % 5) - 2) * 0.05, rows 3 0 7 1 4 4): every output element
    against the code re-derived from the generator's formula (not read back from the packed words) times its group's
    scale plus bias; a repeated row, and a row order that is not the table's."""
    vocab, ids = 8, np.array([3, 0, 7, 1, 4, 4], dtype=np.uint32)
    ng = hidden // g
    w = oracle.synth_bitstream_w(vocab, hidden, bits)
    s = (0.02 + (np.arange(vocab * ng) % 7) * 0.01).astype(np.float32)
    b = (((np.arange(vocab * ng) % 5).astype(np.float32) - 2.0) * 0.05).astype(np.float32)
    out = oracle.dequant_gather(w, s, b, ids, vocab, hidden, g, bits)
    assert out.shape == (ids.size, hidden)
    for t, r in enumerate(ids.tolist()):
        for d in range(hidden):
            code = (((r * hidden + d) * 2654435761 + d) & 0xFFFFFFFF) & ((1 << bits) - 1)
            want = np.float32(code) * s[r * ng + d // g] + b[r * ng + d // g]
            assert out[t, d] == want, (t, d)
    assert np.array_equal(out[4], out[5]) and not np.array_equal(out[0], out[1])


def _np_topk(logits, k, mode):
    """Independent restatement: stable descending argsort + library softmax."""
    from scipy.special import softmax
    z = np.asarray(logits, dtype=np.float64)
    order = np.argsort(-z, axis=1, kind="stable")[:, :k]
    zs = np.take_along_axis(z, order, axis=1)
    w = softmax(zs, axis=1) if mode == 1 else np.take_along_axis(softmax(z, axis=1), order, axis=1)
    return order.astype(np.uint32), w


@pytest.mark.parametrize("mode", [1, 0])
def test_moe_router_topk_against_numpy(oracle, mode):
    # the reference test's logits (moe_gpu_correctness.rs:103-106) and a random draw
    n_rows, n_exp, k = 8, 64, 4
    i = np.arange(n_rows * n_exp, dtype=np.float32)
    logits = np.fmod(i * np.float32(0.13), np.float32(7.0)) - np.float32(3.5) + i * np.float32(0.001)
    for lg, (r, e, kk) in ((logits, (n_rows, n_exp, k)),
                           (np.random.default_rng(3).standard_normal(16 * 128).astype(np.float32), (16, 128, 8))):
        idx, w = oracle.moe_router_topk(lg, r, e, kk, mode)
        ridx, rw = _np_topk(lg.reshape(r, e), kk, mode)
        assert np.array_equal(idx.reshape(r, kk), ridx)
        assert np.max(np.abs(w.reshape(r, kk) - rw)) < 1e-6
        if mode == 1:
            assert np.allclose(w.reshape(r, kk).sum(axis=1), 1.0, atol=1e-6)
        else:
            assert np.all(w.reshape(r, kk).sum(axis=1) < 1.0)


def test_moe_router_topk_reference_edge_cases(oracle):
    # tie -> smaller index first (moe_gpu_correctness.rs:316-335)
    z = np.zeros(8, dtype=np.float32)
    z[2] = z[5] = 3.0
    idx, _ = oracle.moe_router_topk(z, 1, 8, 2)
    assert idx.tolist() == [2, 5]
    # k = 1 -> weight exactly 1 (:288-313)
    idx, w = oracle.moe_router_topk(np.arange(32, dtype=np.float32), 1, 32, 1)
    assert idx.tolist() == [31] and w.tolist() == [1.0]
    # NaN never chosen, +Inf first, -Inf not chosen, no duplicates (:524-597)
    n_exp, k = 16, 4
    lg = np.tile(np.arange(n_exp, dtype=np.float32) * np.float32(0.1), 4)
    lg[5] = np.nan
    lg[n_exp + 7] = np.inf
    lg[2 * n_exp + 3] = -np.inf
    lg[3 * n_exp + 2] = np.nan
    lg[3 * n_exp + 11] = np.inf
    idx, _ = oracle.moe_router_topk(lg, 4, n_exp, k)
    idx = idx.reshape(4, k)
    assert all(len(set(r.tolist())) == k for r in idx)
    assert idx[1, 0] == 7 and idx[3, 0] == 11
    assert 3 not in idx[2] and 5 not in idx[0] and 2 not in idx[3]


def test_moe_unpermute_permute_sort(oracle):
    rng = np.random.default_rng(9)
    T, k, E, H = 12, 3, 7, 40
    logits = rng.standard_normal(T * E).astype(np.float32)
    idx, w = oracle.moe_router_topk(logits, T, E, k)
    sti, inv, offs = oracle.moe_sort_by_expert(idx, T, k, E)
    flat = idx.astype(np.int64)
    # sorted positions are grouped by expert in CSR order, stably
    assert np.all(np.diff(flat[np.argsort(inv)]) >= 0)
    assert offs[0] == 0 and offs[-1] == T * k
    for e in range(E):
        seg = np.argsort(inv)[offs[e]:offs[e + 1]]
        assert np.all(flat[seg] == e) and np.all(np.diff(seg) > 0)
    assert np.array_equal(sti, (np.argsort(inv) // k).astype(np.uint32))
    tokens = rng.standard_normal(T * H).astype(np.float32)
    perm = oracle.moe_permute(tokens, sti, H).reshape(T * k, H)
    for t in range(T):
        for j in range(k):
            assert np.array_equal(perm[inv[t * k + j]], tokens.reshape(T, H)[t])
    # unpermute of the permuted rows gives sum_j w_j * token = token (weights sum to 1)
    out = oracle.moe_unpermute(perm.reshape(-1), inv, w, T, H, k).reshape(T, H)
    ein = np.einsum("tj,tjh->th", w.reshape(T, k).astype(np.float64),
                    perm[inv.reshape(T, k)].astype(np.float64))
    assert np.max(np.abs(out - ein)) < 1e-6
    assert np.max(np.abs(out - tokens.reshape(T, H))) < 1e-5


def test_moe_down_swiglu_accum_against_composition(oracle):
    """The fused MoE decode oracle against numpy silu + the expert-indexed GEMV oracle (pinned
    above) + a numpy slot sum; one slot of weight 1 reduces to that GEMV; zero gates give zero."""
    rng = np.random.default_rng(31)
    E, n, k, g, slots = 6, 20, 256, 64, 8
    codes = rng.integers(0, 16, size=(E * n, k), dtype=np.uint8)
    s = (0.02 * np.abs(rng.standard_normal(E * n * (k // g))) + 1e-3).astype(np.float32)
    b = (-8 * s + rng.standard_normal(s.size).astype(np.float32) * 1e-3).astype(np.float32)
    w = oracle.pack_codes(codes, 4)
    gates = rng.standard_normal((slots, k)).astype(np.float32) * 1.5
    ups = rng.standard_normal((slots, k)).astype(np.float32)
    experts = np.array([3, 1, 5, 0, 2, 4, 1, 3], dtype=np.uint32)
    sw = np.array([0.31, 0.19, 0.12, 0.08, 0.06, 0.05, 0.04, 0.03], dtype=np.float32)
    out32, out64 = oracle.moe_down_swiglu_accum(gates, ups, experts, sw, w, s, b, k, n, g)
    g64 = gates.astype(np.float64)
    inner = (g64 / (1.0 + np.exp(-g64))) * ups.astype(np.float64)
    ref = np.zeros(n)
    for j in range(slots):
        ref += float(sw[j]) * oracle.expert_indexed(w, s, b, inner[j].astype(np.float32), int(experts[j]), n, k, g).astype(np.float64)
    assert np.max(np.abs(out64 - ref)) < 1e-4 and np.max(np.abs(out32 - ref)) < 2e-4
    assert np.max(np.abs(ref)) > 0.05
    one32, _ = oracle.moe_down_swiglu_accum(gates[:1], ups[:1], experts[:1], np.ones(1, dtype=np.float32), w, s, b, k, n, g)
    single = oracle.expert_indexed(w, s, b, inner[0].astype(np.float32), int(experts[0]), n, k, g)
    assert np.max(np.abs(one32 - single)) < 1e-4
    z32, z64 = oracle.moe_down_swiglu_accum(np.zeros_like(gates), ups, experts, sw, w, s, b, k, n, g)
    assert not z32.any() and not z64.any()


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 8])
def test_qvm_against_numpy_and_transposed_qmv(oracle, bits):
    """qvm on the [K, N] layout: (a) numpy f64 x @ dequant(W) with an independently unpacked
    code matrix; (b) equals qmv of the transposed matrix repacked along K (scales transposed
    too) -- a swapped axis in the code or scale indexing breaks one of the two."""
    rng = np.random.default_rng(800 + bits)
    m, n, k, g = 2, 64, 128, 32
    codes = rng.integers(0, 1 << bits, size=(k, n), dtype=np.uint8)      # [K, N]
    s = (0.02 * np.abs(rng.standard_normal((k // g, n))) + 1e-3).astype(np.float32)
    b = (rng.standard_normal((k // g, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = oracle.pack_codes(codes, bits)                                    # rows = K, packed along N
    assert np.array_equal(oracle.np_unpack_codes(w, k, n, bits), codes)
    out32, out64 = oracle.qvm(w, s, b, x, m, n, k, bits, g)
    wd = codes.astype(np.float32) * np.repeat(s, g, axis=0) + np.repeat(b, g, axis=0)   # f32 products, as the oracle forms them
    ref = x.astype(np.float64) @ wd.astype(np.float64)
    assert np.max(np.abs(out64.reshape(m, n) - ref)) < 1e-9
    assert np.max(np.abs(out32.reshape(m, n) - ref)) < 2e-4
    assert np.max(np.abs(ref)) > 0.3
    wt = oracle.pack_codes(np.ascontiguousarray(codes.T), bits)          # [N, K]
    via_qmv = oracle.qmm_f64(wt, np.ascontiguousarray(s.T), np.ascontiguousarray(b.T), x, m, n, k, bits, g)
    assert np.max(np.abs(via_qmv.reshape(m, n) - ref)) < 1e-9
