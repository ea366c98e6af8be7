"""Seeded synthetic inputs in the packed affine format, for tests and benches.

Value distributions are those the benchmark configurations state: codes uniform
over 0..2^bits-1, scale = 0.02*|N(0,1)| + 1e-3, bias = -8*scale + N(0, sigma=1e-3)
(or -(2^(bits-1))*scale for the bit-width sweep), x ~ N(0,1). Values are drawn in
f32 and rounded once to the element dtype; the same bytes go to the GPU and to
whatever checks it.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np

from .dtypes import DType, pack_f32, round_through


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    """[rows, K] codes -> u32 words, LSB-first little-endian bit stream per row."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    rows, k = codes.shape
    if (k * bits) % 32:
        raise ValueError("K*bits must be a multiple of 32")
    if bits in (2, 4, 8):
        pf = 32 // bits
        c = codes.reshape(rows, k // pf, pf).astype(np.uint32)
        shifts = (np.arange(pf, dtype=np.uint32) * np.uint32(bits))
        return np.bitwise_or.reduce(c << shifts, axis=2).astype(np.uint32).reshape(-1)
    bit = ((codes[:, :, None] >> np.arange(bits, dtype=np.uint8)) & 1).astype(np.uint8)
    packed = np.packbits(bit.reshape(rows, k * bits), axis=1, bitorder="little")
    return packed.view("<u4").reshape(-1).copy()


@dataclass
class QCase:
    """One quantized matrix (or a stack of E of them) plus activations."""
    dtype: DType
    bits: int
    group_size: int
    M: int
    N: int
    K: int
    E: int
    w: np.ndarray          # u32 [E*N*K*bits/32]
    scales_f: np.ndarray   # f32 values already rounded through dtype, [E*N*K/G]
    biases_f: np.ndarray
    x_f: np.ndarray        # [M*K]

    @property
    def scales_bytes(self) -> bytes:
        return pack_f32(self.scales_f, self.dtype)

    @property
    def biases_bytes(self) -> bytes:
        return pack_f32(self.biases_f, self.dtype)

    @property
    def x_bytes(self) -> bytes:
        return pack_f32(self.x_f, self.dtype)


def make_case(seed: int, dtype: DType, bits: int, group_size: int, M: int, N: int, K: int,
              E: int = 1, bias_rule: str = "minus8") -> QCase:
    rng = np.random.default_rng(seed)
    rows = E * N
    codes = rng.integers(0, 1 << bits, size=(rows, K), dtype=np.uint8)
    w = pack_codes(codes, bits)
    ng = rows * (K // group_size)
    scale = (np.float32(0.02) * np.abs(rng.standard_normal(ng, dtype=np.float32)) + np.float32(1e-3)).astype(np.float32)
    if bias_rule == "minus8":
        bias = (np.float32(-8.0) * scale + rng.standard_normal(ng, dtype=np.float32) * np.float32(1e-3)).astype(np.float32)
    elif bias_rule == "midpoint":
        bias = (np.float32(-(1 << (bits - 1))) * scale).astype(np.float32)
    else:
        raise ValueError(bias_rule)
    x = rng.standard_normal(M * K, dtype=np.float32)
    return QCase(dtype, bits, group_size, M, N, K, E, w, round_through(scale, dtype),
                 round_through(bias, dtype), round_through(x, dtype))


def top2_routing(seed: int, tokens: int, n_experts: int, top_k: int = 2):
    """Per token, `top_k` distinct experts drawn uniformly. Returns (pair_token,
    pair_expert) sorted by expert (stable), i.e. the row order of the CSR view,
    and expert_offsets[E+1]."""
    rng = np.random.default_rng(seed)
    tok, exp = [], []
    for t in range(tokens):
        for e in rng.choice(n_experts, size=top_k, replace=False):
            tok.append(t)
            exp.append(int(e))
    tok, exp = np.array(tok, np.uint32), np.array(exp, np.uint32)
    order = np.argsort(exp, kind="stable")
    tok, exp = tok[order], exp[order]
    counts = np.bincount(exp, minlength=n_experts)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    return tok, exp, offsets


def qmv_bytes(N: int, K: int, bits: int, group_size: int, M: int, elem_size: int) -> int:
    """Algorithmic bytes of one launch: packed weights + scales + biases + x + out
    (the reference's `qmb`, crates/metaltile-std/src/mlx/quantized.rs:5804)."""
    return N * K * bits // 8 + 2 * N * (K // group_size) * elem_size + M * K * elem_size + M * N * elem_size
