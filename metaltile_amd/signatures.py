"""Binding order of the reference kernels this backend serves.

For each kernel name: tensor parameters in signature order, constexprs in
signature order, and which parameters are outputs (declared `mut` or named
out / output, crates/metaltile-macros/src/legacy/sig_parser.rs:43-48,85).
Sources: crates/metaltile-std/src/mlx/quantized.rs:8-16, 343-352, 4273-4285;
ffai/dequant_gemv.rs:52-62; ffai/dequant_gemv_expert_indexed.rs:58-68;
ffai/moe.rs:358-370, 2256-2268; mlx/quantized.rs:3575-3581, 3629-3635 (affine
quantise / dequantise); ffai/gated_rms_norm_qgemv.rs:90-103; ffai/batched_qkv_qmm.rs:49-68; ffai/batched_4_qmm.rs:61-85; ffai/dequant_gather.rs:47-55.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple


@dataclass(frozen=True)
class KernelSignature:
    name: str
    bits: int
    params: Tuple[str, ...]
    constexprs: Tuple[str, ...]
    outputs: Tuple[str, ...]


_QM = ("w", "scales", "biases", "x", "out")
_DG = ("weight", "scales", "biases", "input", "output")
_EX = ("weights_stacked", "scales_stacked", "biases_stacked", "input", "expert_index", "output")
_GC = ("x", "weight_packed", "scales", "biases", "expert_offsets", "out")
_GI = ("x", "w", "scales", "biases", "indices", "out")

KERNEL_SIGNATURES: Dict[str, KernelSignature] = {}


def _add(name, bits, params, consts, outs):
    KERNEL_SIGNATURES[name] = KernelSignature(name, bits, params, consts, outs)


for _n, _b in (("mt_qmv", 4), ("mt_qmv_int8_fast", 8)):
    _add(_n, _b, _QM, ("k", "gs_per_row"), ("out",))
for _n, _b in (("mt_qmm", 4), ("mt_qmm_bm2", 4), ("mt_qmm_bm4", 4), ("mt_qmm_int8_fast", 8),
               ("mt_qmm_bm2_int8_fast", 8), ("mt_qmm_bm4_int8_fast", 8), ("mt_qmm_mma", 4),
               ("mt_qmm_mma_m16", 4), ("mt_qmm_mma_int8", 8), ("mt_qmm_mma_m16_int8", 8),
               ("mt_qmm_mma_int2", 2), ("mt_qmm_mma_b3", 3), ("mt_qmm_mma_b5", 5), ("mt_qmm_mma_b6", 6)):
    _add(_n, _b, _QM, ("k", "n", "gs_per_row"), ("out",))
for _b in (3, 4, 5, 6, 8):
    _add(f"mt_qmv_b{_b}", _b, _QM, ("k", "n", "group_size"), ("out",))
    _add(f"mt_qmm_b{_b}", _b, _QM, ("k", "n", "group_size"), ("out",))
for _b in (2, 3, 4, 5, 6, 8):
    _add(f"dequant_gemv_int{_b}", _b, _DG, ("in_dim", "group_size"), ("output",))
_add("dequant_gemv_int4_fast", 4, _DG, ("in_dim", "group_size"), ("output",))
_add("dequant_gemv_int4_expert_indexed", 4, _EX, ("in_dim", "out_dim", "group_size"), ("output",))
for _n, _b in (("mt_moe_gather_qmm_int4", 4), ("mt_moe_gather_qmm_int4_m8", 4),
               ("mt_moe_gather_qmm_int4_m16", 4), ("mt_moe_gather_qmm_int4_m32", 4),
               ("mt_moe_gather_qmm_b3", 3), ("mt_moe_gather_qmm_b5", 5), ("mt_moe_gather_qmm_b6", 6),
               ("mt_moe_gather_qmm_b8", 8)):
    _add(_n, _b, _GC, ("k_in", "m_out", "n_experts", "group_size"), ("out",))
for _n, _b in (("mt_moe_gather_qmm_mma_int4", 4), ("mt_moe_gather_qmm_mma_int4_bm16", 4),
               ("mt_moe_gather_qmm_mma_int8", 8), ("mt_moe_gather_qmm_mma_b3", 3),
               ("mt_moe_gather_qmm_mma_b5", 5), ("mt_moe_gather_qmm_mma_b6", 6),
               ("mt_moe_gather_qmm_mma_b8", 8)):
    _add(_n, _b, _GI, ("m_total", "n_out", "k_in", "group_size"), ("out",))
for _b in (2, 3, 4, 5, 6, 8):
    _add(f"mt_affine_quantize_int{_b}", _b, ("w", "out", "scales", "biases"), ("group_size",),
         ("out", "scales", "biases"))
    _add(f"mt_affine_dequantize_int{_b}", _b, ("w", "scales", "biases", "out"), ("group_size",), ("out",))
for _b in (2, 3, 4, 5, 6, 8):
    _add(f"dequant_gather_int{_b}", _b, ("weight", "scales", "biases", "indices", "out"), ("hidden", "group_size"), ("out",))
_QKV = ("x", "w_q", "scales_q", "biases_q", "w_k", "scales_k", "biases_k", "w_v", "scales_v", "biases_v", "out")
for _n in ("ffai_batched_qkv_qgemv", "ffai_batched_qkv_qgemv_fast"):
    _add(_n, 4, _QKV, ("out_q", "out_k", "out_v", "in_dim", "group_size"), ("out",))
_add("ffai_batched_4_qgemv_fast", 4,
     ("x", "w_a", "scales_a", "biases_a", "w_b", "scales_b", "biases_b", "w_c", "scales_c", "biases_c",
      "w_d", "scales_d", "biases_d", "a_out", "b_out", "c_out", "d_out"),
     ("out_a", "out_b", "out_c", "out_d", "in_dim", "group_size"), ("a_out", "b_out", "c_out", "d_out"))
_add("ffai_batched_qkv_qmm_fast", 4, _QKV[:-1] + ("q_buf", "k_buf", "v_buf"),
     ("out_q", "out_k", "out_v", "in_dim", "group_size"), ("q_buf", "k_buf", "v_buf"))
_add("ffai_batched_4_qmm_fast", 4,
     ("x", "w_a", "scales_a", "biases_a", "w_b", "scales_b", "biases_b", "w_c", "scales_c", "biases_c",
      "w_d", "scales_d", "biases_d", "a_buf", "b_buf", "c_buf", "d_buf"),
     ("out_a", "out_b", "out_c", "out_d", "in_dim", "group_size"), ("a_buf", "b_buf", "c_buf", "d_buf"))
for _n, _b in (("ffai_rms_norm_qgemv", 4), ("ffai_rms_norm_qgemv_fast", 4), ("ffai_rms_norm_qgemv_int8_fast", 8)):
    _add(_n, _b, ("x", "norm_weight", "weight", "scales", "biases", "output", "eps_buf"), ("in_dim", "group_size"), ("output",))
_add("ffai_gated_rms_norm_qgemv_int4_fast", 4,
     ("y", "z", "norm_weight", "eps_buf", "q_weight", "q_scales", "q_biases", "out"),
     ("hv", "dv", "out_dim", "group_size"), ("out",))
_add("mt_moe_router_topk", 0, ("router_logits", "indices_out", "weights_out"), ("n_experts", "k", "norm_topk_prob"),
     ("indices_out", "weights_out"))
_add("mt_moe_permute", 0, ("tokens", "sort_token_idx", "permuted"), ("hidden",), ("permuted",))
_add("mt_moe_unpermute", 0, ("expert_outputs", "inv_perm", "top_k_weights", "out"), ("hidden", "k"), ("out",))
_add("ffai_moe_down_swiglu_accum_int4_chain8", 4,
     tuple(n for k in range(8) for n in (f"gate_{k}", f"up_{k}")) + ("expert_indices", "slot_weights", "weights_stacked",
                                                                      "scales_stacked", "biases_stacked", "output"),
     ("in_dim", "out_dim", "group_size"), ("output",))
for _b in (3, 4, 5, 6, 8):
    _add(f"mt_qvm_b{_b}", _b, ("w", "scales", "biases", "x", "out"), ("k", "n", "group_size"), ("out",))
_add("mt_qvm_int4_fast", 4, ("w", "scales", "biases", "x", "out"), ("k", "n", "gs_per_col"), ("out",))
