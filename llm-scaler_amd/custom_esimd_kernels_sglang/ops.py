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
