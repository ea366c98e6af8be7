"""Typed operator entry points on resident device buffers.

Thin wrappers over mtq_qmv / mtq_qmm / mtq_gather_qmv_* of the C-ABI; argument
meaning follows the reference kernels they replace (see include/mtq.h). All
launches are asynchronous on the library stream; `GpuBuffer.read_*` waits.
"""
from __future__ import annotations

import ctypes as C

from . import _lib
from .dtypes import DType
from .runtime import GpuBuffer, _ensure_init


def _p(b):
    return b.ptr if isinstance(b, GpuBuffer) else int(b)


def qmv(dtype: DType, bits: int, group_size: int, w, scales, biases, x, out, M: int, N: int, K: int):
    lib = _ensure_init()
    _lib.check(lib.mtq_qmv(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases), _p(x), _p(out), M, N, K))


def qmm(dtype: DType, bits: int, group_size: int, w, scales, biases, x, out, M: int, N: int, K: int):
    lib = _ensure_init()
    _lib.check(lib.mtq_qmm(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases), _p(x), _p(out), M, N, K))


def gather_qmv_csr(dtype, bits, group_size, x, w, scales, biases, expert_offsets, out, T, N, K, E):
    lib = _ensure_init()
    _lib.check(lib.mtq_gather_qmv_csr(int(dtype), bits, group_size, _p(x), _p(w), _p(scales), _p(biases),
                                      _p(expert_offsets), _p(out), T, N, K, E))


def gather_qmv_indices(dtype, bits, group_size, x, w, scales, biases, indices, out, T, N, K, E):
    lib = _ensure_init()
    _lib.check(lib.mtq_gather_qmv_indices(int(dtype), bits, group_size, _p(x), _p(w), _p(scales), _p(biases),
                                          _p(indices), _p(out), T, N, K, E))


def gather_qmv_single(dtype, bits, group_size, w, scales, biases, inp, expert_index, out, N, K, E):
    lib = _ensure_init()
    _lib.check(lib.mtq_gather_qmv_single(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases),
                                         _p(inp), _p(expert_index), _p(out), N, K, E))


def qvm(dtype, bits, group_size, w, scales, biases, x, out, M, N, K):
    """out[M, N] = x[M, K] @ w_hat, w packed [K, N*bits/32], scales / biases [K/G, N]."""
    lib = _ensure_init()
    _lib.check(lib.mtq_qvm(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases), _p(x), _p(out), M, N, K))


def qvm_noalloc(dtype, bits, group_size, w, scales, biases, x, out, M, N, K):
    """qvm through the library's built-in 4 MiB scratch array: no device allocation in the call."""
    lib = _ensure_init()
    _lib.check(lib.mtq_qvm_noalloc(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases), _p(x), _p(out), M, N, K))


def qmv_batched(dtype, bits, group_size, ws, scales, biases, x, outs, Ns, K):
    """2..4 weight matrices (lists of buffers) against one activation row, one launch."""
    lib = _ensure_init()
    n = len(ws)
    arr = lambda bufs: (C.c_void_p * n)(*[_p(b) for b in bufs])
    _lib.check(lib.mtq_qmv_batched(int(dtype), bits, group_size, n, arr(ws), arr(scales), arr(biases), _p(x), arr(outs),
                                   (C.c_uint32 * n)(*Ns), K))


def qmm_batched(dtype, bits, group_size, ws, scales, biases, x, outs, Ns, M, K):
    """1..4 weight matrices (lists of buffers) against the same M activation rows; outs[j] is [M, Ns[j]]."""
    lib = _ensure_init()
    n = len(ws)
    arr = lambda bufs: (C.c_void_p * n)(*[_p(b) for b in bufs])
    _lib.check(lib.mtq_qmm_batched(int(dtype), bits, group_size, n, arr(ws), arr(scales), arr(biases), _p(x), arr(outs),
                                   (C.c_uint32 * n)(*Ns), M, K))


def rms_norm_qmv(dtype, bits, group_size, x, norm_weight, w, scales, biases, out, eps_buf, N, K):
    """out = qmv(w_hat, rms_norm(x) * norm_weight); eps_buf is a device buffer holding one f32."""
    lib = _ensure_init()
    _lib.check(lib.mtq_rms_norm_qmv(int(dtype), bits, group_size, _p(x), _p(norm_weight), _p(w), _p(scales), _p(biases),
                                    _p(out), _p(eps_buf), N, K))


def gated_rms_norm_qmv(dtype, group_size, y, z, norm_weight, eps_buf, w, scales, biases, out, hv, dv, N):
    """out = qmv(w_hat, flat(rms_norm(y[r]) * norm_weight * silu(z[r]) for r in range(hv))), 4-bit codes; y is f32
    [hv, dv] for every dtype, eps_buf a device buffer holding one f32."""
    lib = _ensure_init()
    _lib.check(lib.mtq_gated_rms_norm_qmv(int(dtype), group_size, _p(y), _p(z), _p(norm_weight), _p(eps_buf), _p(w), _p(scales),
                                          _p(biases), _p(out), hv, dv, N))


def moe_router_topk(dtype, router_logits, indices_out, weights_out, n_rows, n_experts, k, norm_topk_prob=1):
    lib = _ensure_init()
    _lib.check(lib.mtq_moe_router_topk(int(dtype), _p(router_logits), _p(indices_out), _p(weights_out), n_rows, n_experts, k,
                                       norm_topk_prob))


def moe_sort_by_expert(indices, n_tokens, k, n_experts, sort_token_idx, inv_perm, expert_offsets):
    lib = _ensure_init()
    _lib.check(lib.mtq_moe_sort_by_expert(_p(indices), n_tokens, k, n_experts, _p(sort_token_idx), _p(inv_perm),
                                          _p(expert_offsets)))


def moe_permute(dtype, tokens, sort_token_idx, permuted, n_tokens, n_permuted, hidden):
    lib = _ensure_init()
    _lib.check(lib.mtq_moe_permute(int(dtype), _p(tokens), _p(sort_token_idx), _p(permuted), n_tokens, n_permuted, hidden))


def moe_unpermute(dtype, expert_outputs, inv_perm, top_k_weights, out, n_tokens, n_permuted, hidden, k):
    lib = _ensure_init()
    _lib.check(lib.mtq_moe_unpermute(int(dtype), _p(expert_outputs), _p(inv_perm), _p(top_k_weights), _p(out), n_tokens,
                                     n_permuted, hidden, k))


def moe_down_swiglu_accum(dtype, group_size, gates, ups, expert_indices, slot_weights, w, scales, biases, out, in_dim, out_dim,
                          n_experts):
    """gates / ups: lists of 1..8 device buffers T[in_dim] (one per routed slot)."""
    lib = _ensure_init()
    n = len(gates)
    arr = lambda bufs: (C.c_void_p * n)(*[_p(b) for b in bufs])
    _lib.check(lib.mtq_moe_down_swiglu_accum(int(dtype), group_size, n, arr(gates), arr(ups), _p(expert_indices),
                                             _p(slot_weights), _p(w), _p(scales), _p(biases), _p(out), in_dim, out_dim, n_experts))


def affine_quantize(dtype, bits, group_size, w, out, scales, biases, n_elem):
    """w: T[n_elem] -> out: packed u32 words, scales / biases: T[n_elem / group_size]."""
    lib = _ensure_init()
    _lib.check(lib.mtq_affine_quantize(int(dtype), bits, group_size, _p(w), _p(out), _p(scales), _p(biases), n_elem))


def affine_dequantize(dtype, bits, group_size, w, scales, biases, out, n_elem):
    """w: packed u32 words + scales / biases -> out: T[n_elem]."""
    lib = _ensure_init()
    _lib.check(lib.mtq_affine_dequantize(int(dtype), bits, group_size, _p(w), _p(scales), _p(biases), _p(out), n_elem))


def dequant_gather(dtype, bits, group_size, weight, scales, biases, indices, out, n_tokens, hidden, vocab):
    """out[t, :] = dequantised row indices[t] of the packed table [vocab, hidden]."""
    lib = _ensure_init()
    _lib.check(lib.mtq_dequant_gather(int(dtype), bits, group_size, _p(weight), _p(scales), _p(biases), _p(indices), _p(out),
                                      n_tokens, hidden, vocab))


def timed(fn, *args, **kw) -> float:
    """Run one op with GPU timestamps attached to its kernel; returns microseconds."""
    lib = _ensure_init()
    _lib.check(lib.mtq_timed_begin())
    fn(*args, **kw)
    us = C.c_double(0.0)
    _lib.check(lib.mtq_timed_last_us(C.byref(us)))
    return us.value


def sync():
    _lib.check(_ensure_init().mtq_sync())


PLAN_OPS = {"qmv": 0, "qmm": 1, "qmm_mma": 2, "qvm": 3, "gather_csr": 4, "gather_indices": 5, "gather_single": 6, "rms_norm_qmv": 7}


def plan(op: str, dtype, bits: int, group_size: int, M: int = 1, N: int = 0, K: int = 0, E: int = 1, T: int = 0):
    """What the call would launch, without a device (mtq_plan): (rc, [(kernel, grid, block, lds_bytes)], scratch_bytes).
    rc is the code the typed entry point would return as far as shapes decide it; no exception is raised."""
    lib = _lib.load()
    info = _lib.MtqPlanInfo()
    rc = lib.mtq_plan(PLAN_OPS[op], int(dtype), bits, group_size, M, N, K, E, T, info)
    launches = [(l.kernel.decode(), tuple(l.grid), tuple(l.block), int(l.lds_bytes))
                for l in info.launch[:min(info.n_launches, _lib.PLAN_MAX_LAUNCHES)]]
    return rc, launches, int(info.scratch_bytes), info.n_launches
