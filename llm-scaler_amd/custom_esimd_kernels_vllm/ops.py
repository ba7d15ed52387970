"""Thin 1:1 wrappers over torch.ops, same names and argument order as the
reference's vllm/custom-esimd-kernels-vllm/python/custom_esimd_kernels_vllm/ops.py.
Layouts are documented there and in include/mi355x_qlinear.h; bf16 activations
are accepted wherever the reference takes fp16."""
import torch

_ops = torch.ops.custom_esimd_kernels_vllm


def esimd_gemv_fp8_pern(input, weight, weight_scale, output, N, K):
    """input [M, K], weight [N, K] e4m3, weight_scale [N] fp16 or fp32, output [M, N]."""
    return _ops.esimd_gemv_fp8_pern(input, weight, weight_scale, output, N, K)


def esimd_gemv_fp8_pern_fused2(input, w0, s0, o0, N0, w1, s1, o1, N1, K):
    return _ops.esimd_gemv_fp8_pern_fused2(input, w0, s0, o0, N0, w1, s1, o1, N1, K)


def esimd_gemv_fp8_pern_fused3(input, w0, s0, o0, N0, w1, s1, o1, N1, w2, s2, o2, N2, K):
    return _ops.esimd_gemv_fp8_pern_fused3(input, w0, s0, o0, N0, w1, s1, o1, N1, w2, s2, o2, N2, K)


def esimd_gemv_fp8_pert(input, weight, weight_scale, output):
    """weight_scale: fp32 scalar tensor on the device (read by the kernel, no host sync)."""
    return _ops.esimd_gemv_fp8_pert(input, weight, weight_scale, output)


def esimd_gemv_fp8_pert_bmg(input, weight, weight_scale, output):
    return _ops.esimd_gemv_fp8_pert_bmg(input, weight, weight_scale, output)


def esimd_gemv_fp8_pert_fused2(input, w0, s0, o0, w1, s1, o1):
    return _ops.esimd_gemv_fp8_pert_fused2(input, w0, s0, o0, w1, s1, o1)


def esimd_gemv_fp8_pert_fused3(input, w0, s0, o0, w1, s1, o1, w2, s2, o2):
    return _ops.esimd_gemv_fp8_pert_fused3(input, w0, s0, o0, w1, s1, o1, w2, s2, o2)


def esimd_gemm_fp8_pert(input, weight, weight_scale, output):
    return _ops.esimd_gemm_fp8_pert(input, weight, weight_scale, output)


def esimd_gemm_fp8_blockscale(input, weight, weight_scale, output, block_n=128, block_k=128):
    """weight_scale [ceil(N/128), K/128] fp32 (weight_scale_inv); activations are not quantized."""
    return _ops.esimd_gemm_fp8_blockscale(input, weight, weight_scale, output, block_n, block_k)


def esimd_gemv_fp8_blockscale_fused2(input, w0, s0, o0, w1, s1, o1, block_n=128, block_k=128):
    return _ops.esimd_gemv_fp8_blockscale_fused2(input, w0, s0, o0, w1, s1, o1, block_n, block_k)


def esimd_gemv_int4(input, weight, weight_scale, output):
    """weight [N, K/2] uint8 (or [N, K/8] int32), low nibble = even k, stored value + 8;
    weight_scale [N, K/128] fp16."""
    return _ops.esimd_gemv_int4(input, weight, weight_scale, output)


def esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1):
    return _ops.esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1)


def int4_dequant(weight, weight_scale, weight_zp, output):
    return _ops.int4_dequant(weight, weight_scale, weight_zp, output)


def fp8_dequant(weight, weight_scale, output, mode):
    return _ops.fp8_dequant(weight, weight_scale, output, mode)


def e4m3_decode(codes, output):
    return _ops.e4m3_decode(codes, output)
