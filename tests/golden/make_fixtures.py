"""Writes tests/golden/qmatmul_vectors.npz: small input/expected-output vectors
for the affine-quantized matmul family.

The reference keeps no stored outputs for this path (its tests recompute expected
values from closed-form inputs), so these vectors are produced here, by code that
shares nothing with the C oracle or the GPU library: codes are packed with Python
big integers (LSB-first bit string cut into little-endian 32-bit words, the layout
at crates/metaltile-std/src/mlx/quantized.rs:5393-5396 and, for widths that
straddle words, crates/metaltile-std/src/ffai/dequant_gemv.rs:437-441), element
values are rounded to f16 by numpy and to bf16 by integer arithmetic, and expected
outputs are f64 sums of (scale*q + bias)*x over the unpacked integers.

Run:  python tests/golden/make_fixtures.py      (deterministic; rewrites the file)
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def to_bf16_values(v):
    u = np.asarray(v, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32)


def round_to(v, dt):
    v = np.asarray(v, np.float32)
    if dt == "f16":
        return v.astype(np.float16).astype(np.float32)
    if dt == "bf16":
        return to_bf16_values(v)
    return v


def pack_row(codes, bits):
    acc = 0
    for i, q in enumerate(codes):
        acc |= int(q) << (i * bits)
    nwords = len(codes) * bits // 32
    return [(acc >> (32 * j)) & 0xFFFFFFFF for j in range(nwords)]


def make(rng, dt, bits, G, M, N, K, E=1):
    rows = E * N
    codes = rng.integers(0, 1 << bits, size=(rows, K))
    w = np.array([pack_row(r, bits) for r in codes], dtype=np.uint32).reshape(-1)
    ng = rows * (K // G)
    scale = round_to(0.02 * np.abs(rng.standard_normal(ng)) + 1e-3, dt)
    bias = round_to(-(1 << (bits - 1)) * scale + 1e-3 * rng.standard_normal(ng), dt)
    x = round_to(rng.standard_normal(M * K), dt)
    what = (scale.astype(np.float64).reshape(rows, K // G).repeat(G, axis=1) * codes
            + bias.astype(np.float64).reshape(rows, K // G).repeat(G, axis=1))
    return codes, w, scale, bias, x, what.reshape(E, N, K)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    names = []
    i = 0
    for dt in ("f32", "f16", "bf16"):
        for bits in (2, 3, 4, 5, 6, 8):
            G = (32, 64, 128)[i % 3]
            M = (1, 2, 3, 4)[i % 4]
            N = (8, 5, 16)[i % 3]
            K = 2 * G if bits in (3, 5, 6) else (256, 512)[i % 2]
            _, w, s, b, x, what = make(rng, dt, bits, G, M, N, K)
            exp = x.astype(np.float64).reshape(M, K) @ what[0].T
            tag = f"qmm_{dt}_b{bits}_g{G}_m{M}_n{N}_k{K}"
            names.append(tag)
            out.update({f"{tag}/w": w, f"{tag}/scales": s, f"{tag}/biases": b, f"{tag}/x": x,
                        f"{tag}/expected": exp.reshape(-1)})
            i += 1
    # gather: 4 experts, 7 rows, one empty expert; both routing views of the same assignment
    for dt in ("f16", "bf16"):
        E, N, K, G, bits, T = 4, 8, 256, 64, 4, 7
        _, w, s, b, x, what = make(rng, dt, bits, G, T, N, K, E=E)
        indices = np.array([0, 0, 1, 1, 1, 3, 3], dtype=np.uint32)      # expert 2 gets no rows
        offsets = np.array([0, 2, 5, 5, 7], dtype=np.uint32)
        xr = x.astype(np.float64).reshape(T, K)
        exp = np.stack([what[indices[t]] @ xr[t] for t in range(T)])
        tag = f"gather_{dt}_b{bits}_g{G}_t{T}_n{N}_k{K}_e{E}"
        names.append(tag)
        out.update({f"{tag}/w": w, f"{tag}/scales": s, f"{tag}/biases": b, f"{tag}/x": x,
                    f"{tag}/indices": indices, f"{tag}/offsets": offsets, f"{tag}/expected": exp.reshape(-1)})
    # a hand-checkable vector: one row, 32 four-bit codes 0..15,0..15, scale 0.5, bias -4, x = 1
    codes = np.array(list(range(16)) * 2)
    w = np.array(pack_row(codes, 4), dtype=np.uint32)
    assert [hex(v) for v in w[:2]] == ["0x76543210", "0xfedcba98"]
    tag = "qmm_f32_b4_g32_m1_n1_k32_handcheck"
    names.append(tag)
    out.update({f"{tag}/w": w, f"{tag}/scales": np.float32([0.5]), f"{tag}/biases": np.float32([-4.0]),
                f"{tag}/x": np.ones(32, np.float32), f"{tag}/expected": np.float64([0.5 * 240 - 4 * 32])})
    out["names"] = np.array(names)
    path = os.path.join(HERE, "qmatmul_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(names), "cases")


if __name__ == "__main__":
    main()
