"""Thin wrappers, same names and argument order as the reference's
sglang/custom-esimd-kernels/python/custom_esimd_kernels_sglang/ops.py."""
import torch

_ops = torch.ops.custom_esimd_kernels_sglang
_ops_gemm = torch.ops.custom_esimd_kernels


def esimd_gemv_q4_k(input, weight, weight_scale, weight_min, output):
    """input [M, K] fp16, weight [N, K/2] uint8 interleaved nibbles, weight_scale /
    weight_min [N, K/32] fp16, output [M, N] fp16; w = scale * nibble - min."""
    return _ops.esimd_gemv_q4_k(input, weight, weight_scale, weight_min, output)


def q4_k_repack(qweight, ql, weight_scale, weight_min):
    return _ops.q4_k_repack(qweight, ql, weight_scale, weight_min)


def q4_k_dequant(weight, weight_scale, weight_min, output):
    return _ops.q4_k_dequant(weight, weight_scale, weight_min, output)


# other GGUF formats, S/python/custom_esimd_kernels_sglang/ops.py (esimd_gemv_q4_0 ... esimd_gemv_q6_k_m)
def esimd_gemv_q4_0(input, weight, weight_scale, output):
    """weight [N, K/2] uint8 interleaved nibbles, weight_scale [N, K/32] fp16; w = (nib - 8) * scale."""
    return _ops.esimd_gemv_q4_0(input, weight, weight_scale, output)


def esimd_gemm_q4_0(input, weight, weight_scale, output):
    return _ops.esimd_gemm_q4_0(input, weight, weight_scale, output)


def esimd_gemv_q8_0(input, weight, weight_scale, output):
    """weight [N, K] int8, weight_scale [N, K/32] fp16; w = qs * scale."""
    return _ops.esimd_gemv_q8_0(input, weight, weight_scale, output)


def esimd_gemv_q8_0_m(input, weight, weight_scale, output):
    return _ops.esimd_gemv_q8_0_m(input, weight, weight_scale, output)


def esimd_gemv_q5_k(input, ql, qh, weight_scale, weight_min, output):
    return _ops.esimd_gemv_q5_k(input, ql, qh, weight_scale, weight_min, output)


def esimd_gemv_q6_k(input, ql, qh, weight_scale, output):
    return _ops.esimd_gemv_q6_k(input, ql, qh, weight_scale, output)


def esimd_gemv_q6_k_m(input, ql, qh, weight_scale, output):
    return _ops.esimd_gemv_q6_k_m(input, ql, qh, weight_scale, output)


# weight preparation on the device (the reference does these in torch at load time)
def q4_0_repack(qweight, weight, weight_scale):
    return _ops.q4_0_repack(qweight, weight, weight_scale)


def q8_0_repack(qweight, weight, weight_scale):
    return _ops.q8_0_repack(qweight, weight, weight_scale)


def q5_k_repack(qweight, ql, qh, weight_scale, weight_min):
    return _ops.q5_k_repack(qweight, ql, qh, weight_scale, weight_min)


def q6_k_repack(qweight, ql, qh, weight_scale):
    return _ops.q6_k_repack(qweight, ql, qh, weight_scale)


def q5_k_repack_plain(qweight, ql, qh, weight_scale, weight_min):
    return _ops.q5_k_repack_plain(qweight, ql, qh, weight_scale, weight_min)


def q6_k_repack_plain(qweight, ql, qh, weight_scale):
    return _ops.q6_k_repack_plain(qweight, ql, qh, weight_scale)


def q4_0_dequant(weight, weight_scale, output):
    return _ops.q4_0_dequant(weight, weight_scale, output)


def q8_0_dequant(weight, weight_scale, output):
    return _ops.q8_0_dequant(weight, weight_scale, output)


def q5_k_dequant(ql, qh, weight_scale, weight_min, output):
    return _ops.q5_k_dequant(ql, qh, weight_scale, weight_min, output)


def q6_k_dequant(ql, qh, weight_scale, output):
    return _ops.q6_k_dequant(ql, qh, weight_scale, output)


def esimd_gemv_fp8_pern(input, weight, weight_scale, output, N, K):
    return _ops.esimd_gemv_fp8_pern(input, weight, weight_scale, output, N, K)


def esimd_gemv_fp8_pert(input, weight, weight_scale, output):
    return _ops.esimd_gemv_fp8_pert(input, weight, weight_scale, output)


def esimd_gemv_int4(input, weight, weight_scale, output):
    return _ops.esimd_gemv_int4(input, weight, weight_scale, output)


def esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1):
    return _ops.esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1)


def esimd_gemm_fp8_pert(input, weight, weight_scale, output):
    return _ops_gemm.esimd_gemm_fp8_pert(input, weight, weight_scale, output)


def esimd_gemm_int4_pgrp(input, weight, weight_scale, output):
    return _ops_gemm.esimd_gemm_int4_pgrp(input, weight, weight_scale, output)


# FP8 MoE prefill with per-expert scalar scales (torch.ops.moe_fp8_prefill_ops),
# S/python/custom_esimd_kernels_sglang/ops.py:1656-1675
_moe_fp8_prefill = torch.ops.moe_fp8_prefill_ops


def moe_prefill_full_fp8(hidden_states, topk_weights, topk_ids, w13, w13_scale, w2, w2_scale, top_k, num_experts):
    return _moe_fp8_prefill.moe_prefill_full_fp8(hidden_states, topk_weights, topk_ids, w13, w13_scale, w2, w2_scale,
                                                 top_k, num_experts)


# fused GGUF k-quant MoE decode stages, S/python/custom_esimd_kernels_sglang/ops.py:250-298
def esimd_moe_up_q4k(x, gate_ql, gate_sc, gate_mn, up_ql, up_sc, up_mn, sel, inter, n_tokens, hidden, intermediate,
                     top_k):
    return _ops.esimd_moe_up_q4k(x, gate_ql, gate_sc, gate_mn, up_ql, up_sc, up_mn, sel, inter, n_tokens, hidden,
                                 intermediate, top_k)


def esimd_moe_down_q5k(inter, ql, qh, sc, mn, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k):
    return _ops.esimd_moe_down_q5k(inter, ql, qh, sc, mn, sel, topk_w, out_partial, n_tokens, hidden, intermediate,
                                   top_k)


def esimd_moe_down_q6k(inter, ql, qh, sc, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k):
    return _ops.esimd_moe_down_q6k(inter, ql, qh, sc, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k)


# The names below are what the reference's SGLang package re-exports besides the GGUF ones
# (S/python/custom_esimd_kernels_sglang/__init__.py:69-147) and this library registers under
# torch.ops.custom_esimd_kernels_sglang: the fused FP8 GEMVs, the norm + GEMV family and the MoE helpers the
# patched GGUF path takes through its name lookup (esimd_moe_silu_mul, esimd_moe_gather;
# sglang/patches/sglang_for_multi_arc.patch:2134-2138).  Same argument order as the reference's wrappers
# (S/python/custom_esimd_kernels_sglang/ops.py:26-90, 421-600, 638-735).
def esimd_gemv_fp8_pern_fused2(input, w0, s0, o0, N0, w1, s1, o1, N1, K):
    return _ops.esimd_gemv_fp8_pern_fused2(input, w0, s0, o0, N0, w1, s1, o1, N1, K)


def esimd_gemv_fp8_pern_fused3(input, w0, s0, o0, N0, w1, s1, o1, N1, w2, s2, o2, N2, K):
    return _ops.esimd_gemv_fp8_pern_fused3(input, w0, s0, o0, N0, w1, s1, o1, N1, w2, s2, o2, N2, K)


def esimd_gemv_fp8_pert_fused2(input, w0, s0, o0, w1, s1, o1):
    return _ops.esimd_gemv_fp8_pert_fused2(input, w0, s0, o0, w1, s1, o1)


def esimd_gemv_fp8_pert_fused3(input, w0, s0, o0, w1, s1, o1, w2, s2, o2):
    return _ops.esimd_gemv_fp8_pert_fused3(input, w0, s0, o0, w1, s1, o1, w2, s2, o2)


def esimd_fused_add_rms_norm(hidden_states, residual, weight, eps):
    """residual = hidden_states + residual (in place); hidden_states = rmsnorm(residual) * weight."""
    return _ops.esimd_fused_add_rms_norm(hidden_states, residual, weight, eps)


def esimd_rms_norm_gated(x, z, weight, output, eps):
    """output = rmsnorm(x) * weight * silu(z); x, z [rows, V], weight [V]."""
    return _ops.esimd_rms_norm_gated(x, z, weight, output, eps)


def esimd_fused_add_rms_norm_batched(hidden_states, residual, weight, eps):
    return _ops.esimd_fused_add_rms_norm_batched(hidden_states, residual, weight, eps)


def esimd_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                    normed_out, eps):
    return _ops.esimd_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale,
                                                output, normed_out, eps)


def esimd_resadd_norm_gemv_int4_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                     normed_out, eps):
    return _ops.esimd_resadd_norm_gemv_int4_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale,
                                                 output, normed_out, eps)


def esimd_resadd_norm_gemv2_fp8_pert(hidden_states, residual, norm_weight, w0, s0, o0, w1, s1, o1, eps):
    return _ops.esimd_resadd_norm_gemv2_fp8_pert(hidden_states, residual, norm_weight, w0, s0, o0, w1, s1, o1, eps)


def esimd_norm_gemv_fp8_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    return _ops.esimd_norm_gemv_fp8_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps)


def esimd_norm_gemv_int4_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    return _ops.esimd_norm_gemv_int4_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps)


def esimd_moe_topk(router_logits, top_values, top_indices, T):
    """router_logits [T, E], top_values [T, K] (output, logits dtype), top_indices [T, K] int32 (output)."""
    return _ops.esimd_moe_topk(router_logits, top_values, top_indices, T)


def esimd_moe_scatter_fused(hidden_states, top_values, top_indices, scattered_hidden, scattered_weights,
                            topk_ids, expert_start, max_tokens_out, K, topk, T, num_experts):
    return _ops.esimd_moe_scatter_fused(hidden_states, top_values, top_indices, scattered_hidden,
                                        scattered_weights, topk_ids, expert_start, max_tokens_out,
                                        K, topk, T, num_experts)


def esimd_moe_silu_mul(input, output, N_gate_up, N_half, total_rows):
    return _ops.esimd_moe_silu_mul(input, output, N_gate_up, N_half, total_rows)


def esimd_moe_gather(moe_output, topk_ids, scattered_weights, final_hidden, K, topk, T):
    return _ops.esimd_moe_gather(moe_output, topk_ids, scattered_weights, final_hidden, K, topk, T)


# MoE batch helpers of torch.ops.moe_ops that the reference package re-exports
_moe = torch.ops.moe_ops
def moe_router_forward(x, weight, scale):
    """Router logits on per-tensor FP8 weights: x [n_tokens, hidden], weight [num_experts, hidden] fp8,
    scale [num_experts] fp32 -> [n_tokens, num_experts] (S/python/custom_esimd_kernels_sglang/ops.py:926-938)."""
    return _moe.moe_router_forward(x, weight, scale)


def moe_batch_topk(logits, top_k, norm=True):
    """(top_values [n_tokens, top_k], top_indices [n_tokens, top_k] int32) (S/python/custom_esimd_kernels_sglang/ops.py:941-953)."""
    return _moe.moe_topk(logits, top_k, norm)


def moe_accumulate(partials, top_k, num_shared_experts):
    """Unweighted sum of each token's top_k + shared rows: partials [n_tokens * (top_k + shared), hidden]
    -> [n_tokens, hidden] (S/python/custom_esimd_kernels_sglang/ops.py:1015-1025)."""
    return _moe.moe_accumulate(partials, top_k, num_shared_experts)


def moe_forward_full(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight, shared_gate_up_scale,
                     down_weight, down_scale, shared_down_weight, shared_down_scale, shared_expert_gate_weight,
                     top_k, num_shared_experts, n_routed_experts):
    """The fused decode MoE forward on K-major per-tensor FP8 weights (torch.ops.moe_ops.moe_forward_full)."""
    return _moe.moe_forward_full(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight,
                                 shared_gate_up_scale, down_weight, down_scale, shared_down_weight,
                                 shared_down_scale, shared_expert_gate_weight, top_k, num_shared_experts,
                                 n_routed_experts)


# Imported at module level by the patched SGLang's XPU attention backend
# (sglang/patches/sglang_for_multi_arc.patch:684); paged attention is outside the quantized-linear path:
# the name exists so that module imports, and raises when called.
from mi355x_qlinear.not_provided import NotProvided as _NotProvided  # noqa: E402

eagle_page_attn_decode = _NotProvided("eagle_page_attn_decode", "an attention backend other than xpu")
