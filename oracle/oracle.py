"""ctypes loader for the CPU oracle (oracle/mtq_oracle.c) plus an independent
numpy restatement used to pin it.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and bench.py's
cpu_baseline leg. The product package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmtq_oracle.so")

F32, F16, BF16 = 0, 1, 2

_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "mtq_oracle.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.mtq_oracle_f32_to_bf16.restype = C.c_uint16
        _lib.mtq_oracle_f32_to_bf16.argtypes = [C.c_float]
        _lib.mtq_oracle_f32_to_f16.restype = C.c_uint16
        _lib.mtq_oracle_f32_to_f16.argtypes = [C.c_float]
        _lib.mtq_oracle_bf16_to_f32.restype = C.c_float
        _lib.mtq_oracle_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.mtq_oracle_f16_to_f32.restype = C.c_float
        _lib.mtq_oracle_f16_to_f32.argtypes = [C.c_uint16]
        _lib.mtq_oracle_csr_expert.restype = C.c_uint32
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


_sz = C.c_size_t


def pack_f32(vals, dt: int) -> bytes:
    v = _f32(vals).ravel()
    out = np.empty(v.size * (4 if dt == F32 else 2), dtype=np.uint8)
    lib().mtq_oracle_pack_f32(_p(v), _sz(v.size), C.c_int(dt), _p(out))
    return out.tobytes()


def unpack_f32(data: bytes, dt: int) -> np.ndarray:
    n = len(data) // (4 if dt == F32 else 2)
    raw = np.frombuffer(data, dtype=np.uint8).copy()
    out = np.empty(n, dtype=np.float32)
    lib().mtq_oracle_unpack_f32(_p(raw), _sz(n), C.c_int(dt), _p(out))
    return out


def round_through(vals, dt: int) -> np.ndarray:
    v = _f32(vals).copy()
    lib().mtq_oracle_round_through(_p(v), _sz(v.size), C.c_int(dt))
    return v


def synth_packed_w(n: int, k: int, bits: int) -> np.ndarray:
    out = np.empty(n * k * bits // 32, dtype=np.uint32)
    lib().mtq_oracle_synth_packed_w(_sz(n), _sz(k), C.c_uint32(bits), _p(out))
    return out


def synth_bitstream_w(out_dim: int, in_dim: int, bits: int) -> np.ndarray:
    out = np.empty(out_dim * in_dim * bits // 32, dtype=np.uint32)
    lib().mtq_oracle_synth_bitstream_w(_sz(out_dim), _sz(in_dim), C.c_uint32(bits), _p(out))
    return out


def synth_stacked_w(n_experts: int, out_dim: int, in_dim: int) -> np.ndarray:
    out = np.empty(n_experts * out_dim * in_dim // 8, dtype=np.uint32)
    lib().mtq_oracle_synth_stacked_w(_sz(n_experts), _sz(out_dim), _sz(in_dim), _p(out))
    return out


def unpack_codes(w, n: int, k: int, bits: int) -> np.ndarray:
    w = _u32(w)
    out = np.empty(n * k, dtype=np.uint8)
    lib().mtq_oracle_unpack_codes(_p(w), _sz(n), _sz(k), C.c_uint32(bits), _p(out))
    return out.reshape(n, k)


def pack_codes(codes, bits: int) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    n, k = codes.shape
    out = np.empty(n * k * bits // 32, dtype=np.uint32)
    lib().mtq_oracle_pack_codes(_p(codes), _sz(n), _sz(k), C.c_uint32(bits), _p(out))
    return out


def qmm(w, scales, biases, x, m, n, k, bits, group_size, threads: int = 1) -> np.ndarray:
    """f32-sequential reference oracle (qmm_oracle)."""
    w, scales, biases, x = _u32(w), _f32(scales), _f32(biases), _f32(x)
    out = np.empty(m * n, dtype=np.float32)
    lib().mtq_oracle_qmm(_p(w), _p(scales), _p(biases), _p(x), _sz(m), _sz(n), _sz(k),
                         C.c_uint32(bits), _sz(group_size), _p(out), C.c_int(threads))
    return out


def qmm_f64(w, scales, biases, x, m, n, k, bits, group_size, threads: int = 1) -> np.ndarray:
    w, scales, biases, x = _u32(w), _f32(scales), _f32(biases), _f32(x)
    out = np.empty(m * n, dtype=np.float64)
    lib().mtq_oracle_qmm_f64(_p(w), _p(scales), _p(biases), _p(x), _sz(m), _sz(n), _sz(k),
                             C.c_uint32(bits), _sz(group_size), _p(out), C.c_int(threads))
    return out


def qmm_split(w, scales, biases, x, m, n, k, bits, group_size) -> np.ndarray:
    w, scales, biases, x = _u32(w), _f32(scales), _f32(biases), _f32(x)
    out = np.empty(m * n, dtype=np.float32)
    lib().mtq_oracle_qmm_split(_p(w), _p(scales), _p(biases), _p(x), _sz(m), _sz(n), _sz(k),
                               C.c_uint32(bits), _sz(group_size), _p(out))
    return out


def qmm_mma(w, scales, biases, x, m, n, k, bits, group_size, dt: int, threads: int = 1) -> np.ndarray:
    w, scales, biases, x = _u32(w), _f32(scales), _f32(biases), _f32(x)
    out = np.empty(m * n, dtype=np.float64)
    lib().mtq_oracle_qmm_mma(_p(w), _p(scales), _p(biases), _p(x), _sz(m), _sz(n), _sz(k),
                             C.c_uint32(bits), _sz(group_size), C.c_int(dt), _p(out), C.c_int(threads))
    return out


def csr_expert(expert_offsets, n_experts: int, t: int) -> int:
    off = _u32(expert_offsets)
    return int(lib().mtq_oracle_csr_expert(_p(off), _sz(n_experts), C.c_uint32(t)))


def gather_qmm(x, weight_packed, scales, biases, t_rows, k_in, m_out, n_experts, bits, group_size,
               expert_offsets=None, indices=None, f64: bool = False, threads: int = 1) -> np.ndarray:
    x, w, s, b = _f32(x), _u32(weight_packed), _f32(scales), _f32(biases)
    off = _u32(expert_offsets) if expert_offsets is not None else None
    idx = _u32(indices) if indices is not None else None
    out = np.empty(t_rows * m_out, dtype=np.float64 if f64 else np.float32)
    lib().mtq_oracle_gather_qmm(_p(x), _p(w), _p(s), _p(b), _p(off) if off is not None else None,
                                _p(idx) if idx is not None else None, _sz(t_rows), _sz(k_in),
                                _sz(m_out), _sz(n_experts), C.c_uint32(bits), _sz(group_size),
                                None if f64 else _p(out), _p(out) if f64 else None, C.c_int(threads))
    return out


def expert_indexed(weight, scales, biases, inp, expert, out_dim, in_dim, group_size) -> np.ndarray:
    w, s, b, x = _u32(weight), _f32(scales), _f32(biases), _f32(inp)
    out = np.empty(out_dim, dtype=np.float32)
    lib().mtq_oracle_expert_indexed(_p(w), _p(s), _p(b), _p(x), _sz(expert), _sz(out_dim), _sz(in_dim),
                                    _sz(group_size), _p(out))
    return out


def rms_norm_qgemv(w, scales, biases, x, norm_weight, in_dim, group_size, out_dim, bits, eps):
    """Returns (out f32 sequential, out f64-accumulated, normalised activation f32)."""
    w, scales, biases, x, norm_weight = _u32(w), _f32(scales), _f32(biases), _f32(x), _f32(norm_weight)
    out = np.empty(out_dim, dtype=np.float32)
    out64 = np.empty(out_dim, dtype=np.float64)
    normed = np.empty(in_dim, dtype=np.float32)
    lib().mtq_oracle_rms_norm_qgemv(_p(w), _p(scales), _p(biases), _p(x), _p(norm_weight), _sz(in_dim), _sz(group_size),
                                    _sz(out_dim), C.c_uint32(bits), C.c_float(eps), _p(out), _p(out64), _p(normed))
    return out, out64, normed


def gated_rms_norm_qgemv(w, scales, biases, y, z, norm_weight, hv, dv, group_size, out_dim, eps):
    """4-bit codes; y, z [hv, dv], norm_weight [dv]. Returns (out f32 sequential, out f64-accumulated, the gated,
    normalised activation f32 [hv * dv])."""
    w, scales, biases, y, z, norm_weight = _u32(w), _f32(scales), _f32(biases), _f32(y), _f32(z), _f32(norm_weight)
    assert y.size == hv * dv and z.size == hv * dv and norm_weight.size == dv
    out = np.empty(out_dim, dtype=np.float32)
    out64 = np.empty(out_dim, dtype=np.float64)
    inner = np.empty(hv * dv, dtype=np.float32)
    lib().mtq_oracle_gated_rms_norm_qgemv(_p(w), _p(scales), _p(biases), _p(y), _p(z), _p(norm_weight), _sz(hv), _sz(dv),
                                          _sz(group_size), _sz(out_dim), C.c_float(eps), _p(out), _p(out64), _p(inner))
    return out, out64, inner


def qvm(w, scales, biases, x, m, n, k, bits, group_size):
    """W [K, N] packed along N, scales / biases [K/G, N]. Returns (f32 sequential, f64-accumulated), each [m, n]."""
    w, scales, biases, x = _u32(w), _f32(scales), _f32(biases), _f32(x)
    out = np.empty(m * n, dtype=np.float32)
    out64 = np.empty(m * n, dtype=np.float64)
    lib().mtq_oracle_qvm(_p(w), _p(scales), _p(biases), _p(x), _sz(m), _sz(n), _sz(k), C.c_uint32(bits), _sz(group_size),
                         _p(out), _p(out64))
    return out, out64


def moe_router_topk(logits, n_rows: int, n_experts: int, k: int, norm_topk_prob: int = 1):
    logits = _f32(logits)
    idx = np.empty(n_rows * k, dtype=np.uint32)
    w = np.empty(n_rows * k, dtype=np.float32)
    lib().mtq_oracle_moe_router_topk(_p(logits), _sz(n_rows), _sz(n_experts), _sz(k), C.c_int(norm_topk_prob), _p(idx), _p(w))
    return idx, w


def moe_unpermute(expert_outputs, inv_perm, weights, n_tokens: int, hidden: int, k: int) -> np.ndarray:
    eo, ip, w = _f32(expert_outputs), _u32(inv_perm), _f32(weights)
    out = np.empty(n_tokens * hidden, dtype=np.float32)
    lib().mtq_oracle_moe_unpermute(_p(eo), _p(ip), _p(w), _sz(n_tokens), _sz(hidden), _sz(k), _p(out))
    return out


def moe_permute(tokens, sort_token_idx, hidden: int) -> np.ndarray:
    """permuted[p, :] = tokens[sort_token_idx[p], :] (crates/metaltile-std/src/ffai/moe.rs:282-302); any dtype."""
    t = np.asarray(tokens).reshape(-1, hidden)
    return t[np.asarray(sort_token_idx, dtype=np.int64)].reshape(-1)


def moe_sort_by_expert(indices, n_tokens: int, k: int, n_experts: int):
    """The caller-side sort the reference describes (crates/metaltile-std/src/ffai/moe.rs:256-275):
    a stable argsort of the flattened (token * k + slot) expert ids. Returns sort_token_idx [n*k]
    (source token of each sorted position), inv_perm [n, k] (sorted position of each (token, slot))
    and expert_offsets [E + 1] (CSR bounds of each expert's rows)."""
    flat = np.asarray(indices, dtype=np.int64).reshape(-1)
    order = np.argsort(flat, kind="stable")
    inv = np.empty_like(order)
    inv[order] = np.arange(order.size)
    offsets = np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=n_experts))])
    return (order // k).astype(np.uint32), inv.astype(np.uint32), offsets.astype(np.uint32)


def moe_down_swiglu_accum(gates, ups, experts, slot_w, weights, scales, biases, in_dim, out_dim, group_size):
    """gates / ups: [n_slots, in_dim]. Returns (f32 chain, f64-accumulated)."""
    gates, ups, slot_w = _f32(gates), _f32(ups), _f32(slot_w)
    experts, weights, scales, biases = _u32(experts), _u32(weights), _f32(scales), _f32(biases)
    n_slots = experts.size
    out = np.empty(out_dim, dtype=np.float32)
    out64 = np.empty(out_dim, dtype=np.float64)
    lib().mtq_oracle_moe_down_swiglu_accum(_p(gates), _p(ups), _p(experts), _p(slot_w), _sz(n_slots), _p(weights), _p(scales),
                                           _p(biases), _sz(in_dim), _sz(out_dim), _sz(group_size), _p(out), _p(out64))
    return out, out64


def affine_quantize(v, group_size: int, bits: int, dt: int):
    v = _f32(v).ravel()
    ng = v.size // group_size
    codes = np.empty(v.size, dtype=np.uint8)
    scales = np.empty(ng, dtype=np.float32)
    biases = np.empty(ng, dtype=np.float32)
    lib().mtq_oracle_affine_quantize(_p(v), _sz(ng), _sz(group_size), C.c_uint32(bits), C.c_int(dt),
                                     _p(codes), _p(scales), _p(biases))
    return codes, scales, biases


def affine_dequantize(w, scales, biases, n_elem: int, group_size: int, bits: int) -> np.ndarray:
    w, s, b = _u32(w), _f32(scales), _f32(biases)
    out = np.empty(n_elem, dtype=np.float32)
    lib().mtq_oracle_affine_dequantize(_p(w), _p(s), _p(b), _sz(n_elem), _sz(group_size),
                                       C.c_uint32(bits), _p(out))
    return out


def dequant_gather(weight, scales, biases, indices, vocab: int, hidden: int, group_size: int, bits: int) -> np.ndarray:
    """out[t, :] = row indices[t] of the dequantised table [vocab, hidden]: the affine dequantiser over the whole table
    (each row a bit stream of hidden codes, groups along the row) and a row take. Reference:
    crates/metaltile-std/src/ffai/dequant_gather.rs:148-185 (its CPU form), :56-93 (kernel)."""
    table = affine_dequantize(weight, scales, biases, vocab * hidden, group_size, bits).reshape(vocab, hidden)
    return table[np.asarray(indices, dtype=np.int64)]


def bench_stats(samples) -> dict:
    s = np.ascontiguousarray(samples, dtype=np.float64)
    out = np.empty(7, dtype=np.float64)
    lib().mtq_oracle_bench_stats(_p(s), _sz(s.size), _p(out))
    keys = ["min_us", "mean_us", "median_us", "p95_us", "p99_us", "stddev_us", "cv_pct"]
    return dict(zip(keys, out.tolist()))


# ---------------------------------------------------------------------------
# Independent numpy path (no shared code with the C file): used to pin it.
# ---------------------------------------------------------------------------

def np_unpack_codes(w, n: int, k: int, bits: int) -> np.ndarray:
    """Bit-stream reader written against the format definition: code j of a row
    occupies bits [j*bits, (j+1)*bits) of the row's little-endian bit string."""
    w = _u32(w).reshape(n, -1)
    bitsarr = np.unpackbits(w.view(np.uint8).reshape(n, -1), axis=1, bitorder="little")
    bitsarr = bitsarr[:, : k * bits].reshape(n, k, bits).astype(np.uint32)
    weights = (1 << np.arange(bits, dtype=np.uint32))
    return (bitsarr * weights).sum(axis=2).astype(np.uint8)


def np_dequant(w, scales, biases, n: int, k: int, bits: int, group_size: int) -> np.ndarray:
    q = np_unpack_codes(w, n, k, bits).astype(np.float32)
    s = np.repeat(_f32(scales).reshape(n, k // group_size), group_size, axis=1)
    b = np.repeat(_f32(biases).reshape(n, k // group_size), group_size, axis=1)
    return (q * s + b).astype(np.float32)  # f32 multiply then add, as the reference


def np_qmm_f64(w, scales, biases, x, m, n, k, bits, group_size) -> np.ndarray:
    """Y = X @ dequant(W).T with numpy's f64 matmul."""
    wd = np_dequant(w, scales, biases, n, k, bits, group_size).astype(np.float64)
    return _f32(x).reshape(m, k).astype(np.float64) @ wd.T
