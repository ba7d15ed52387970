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


def esimd_gemv_fp8_blockscale_fp16_fused2(input, w0, s0, o0, w1, o1, block_n=128, block_k=128):
    return _ops.esimd_gemv_fp8_blockscale_fp16_fused2(input, w0, s0, o0, w1, o1, block_n, block_k)


def esimd_gemv_fp16(input, weight, output):
    """input [M, K], weight [N, K] (16-bit, contiguous), output [M, N]."""
    return _ops.esimd_gemv_fp16(input, weight, output)


def esimd_gemv_fp16_gelu_mul(input, weight, output):
    """weight [2N, K], gate rows first; output [M, N] = gelu_tanh(gate) * up."""
    return _ops.esimd_gemv_fp16_gelu_mul(input, weight, output)


def esimd_gemv_int4(input, weight, weight_scale, output):
    """weight [N, K/2] uint8 (or [N, K/8] int32), low nibble = even k, stored value + 8;
    weight_scale [N, K/128] fp16."""
    return _ops.esimd_gemv_int4(input, weight, weight_scale, output)


def esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1):
    return _ops.esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1)


def esimd_gemm_int4_pgrp(input, weight, weight_scale, output):
    """input [M, K], weight [N, K/2] uint8 (low nibble = even k, value + 8), weight_scale [N, K/128]
    fp16, output [M, N]; any M (the reference's kernel stops at 64 rows)."""
    return _ops.esimd_gemm_int4_pgrp(input, weight, weight_scale, output)


def esimd_gemm_int4_pgrp_zp(input, weight, weight_scale, weight_zp, output):
    """Asymmetric sibling: weight_zp [N, K/128] uint8 in 0..15."""
    return _ops.esimd_gemm_int4_pgrp_zp(input, weight, weight_scale, weight_zp, output)


def int4_gemm_w4a16(x, qweight, bias, scales, qzeros, group_size, g_idx=None):
    """The GPTQ / AWQ / sym_int4 linear call of the patched vLLM
    (vllm/patches/vllm_for_multi_arc.patch:5492-5500): qweight logical [K/8, N] int32, scales [K/128, N]
    fp16, qzeros [K/128, N/8] int32 or one value; returns a new [M, N] tensor."""
    return _ops.int4_gemm_w4a16(x, qweight, bias, scales, qzeros, group_size, g_idx)


def w4a16_prepare(qweight, scales, qzeros, group_size, zero_bias=0):
    """Load-time conversion of those operands into (weight [N, K/8], scale [N, K/128], zp [N, K/128]) for
    esimd_gemm_int4_pgrp_zp / esimd_gemv_int4."""
    return _ops.w4a16_prepare(qweight, scales, qzeros, group_size, zero_bias)


def int4_dequant(weight, weight_scale, weight_zp, output):
    return _ops.int4_dequant(weight, weight_scale, weight_zp, output)


def fp8_dequant(weight, weight_scale, output, mode):
    return _ops.fp8_dequant(weight, weight_scale, output, mode)


def e4m3_decode(codes, output):
    return _ops.e4m3_decode(codes, output)


# ---- MoE ----
_moe = torch.ops.moe_ops


def esimd_moe_topk(router_logits, top_values, top_indices, T):
    """router_logits [T, E], top_values [T, K] (output, logits dtype), top_indices [T, K] int32 (output)."""
    return _ops.esimd_moe_topk(router_logits, top_values, top_indices, T)


def esimd_moe_scatter(hidden_states, router_top_value, sorted_token_ids, scattered_hidden, scattered_weights,
                      K, topk, total_expanded):
    return _ops.esimd_moe_scatter(hidden_states, router_top_value, sorted_token_ids, scattered_hidden,
                                  scattered_weights, K, topk, total_expanded)


def esimd_moe_scatter_fused(hidden_states, top_values, top_indices, scattered_hidden, scattered_weights,
                            topk_ids, expert_start, max_tokens_out, K, topk, T, num_experts):
    return _ops.esimd_moe_scatter_fused(hidden_states, top_values, top_indices, scattered_hidden,
                                        scattered_weights, topk_ids, expert_start, max_tokens_out,
                                        K, topk, T, num_experts)


def esimd_moe_silu_mul(input, output, N_gate_up, N_half, total_rows):
    return _ops.esimd_moe_silu_mul(input, output, N_gate_up, N_half, total_rows)


def esimd_moe_gelu_tanh_mul(input, output, N_gate_up, N_half, total_rows):
    """GELU_tanh(gate) * up activation."""
    return _ops.esimd_moe_gelu_tanh_mul(input, output, N_gate_up, N_half, total_rows)


def esimd_moe_gather(moe_output, topk_ids, scattered_weights, final_hidden, K, topk, T):
    return _ops.esimd_moe_gather(moe_output, topk_ids, scattered_weights, final_hidden, K, topk, T)


def esimd_moe_gemm_fp8_blockscale(input, weight, weight_scale, output, expert_idx, N, K, num_experts,
                                  block_n=128, block_k=128):
    """input [total_tokens, K] (expert-grouped rows), weight [E, N, K] e4m3, weight_scale
    [E, ceil(N/128), K/128] fp32, expert_idx [E+1] start offsets; activations stay 16 bit."""
    return _ops.esimd_moe_gemm_fp8_blockscale(input, weight, weight_scale, output, expert_idx,
                                              N, K, num_experts, block_n, block_k)


def moe_topk(logits, top_k, norm=True):
    return _moe.moe_topk(logits, top_k, norm)


def moe_sort(top_ids, num_experts, sorted_pairs, expert_start, inv, sorted_token=None, max_count=None):
    return _ops.moe_sort(top_ids, num_experts, sorted_pairs, expert_start, inv, sorted_token, max_count)


def act_quant_fp8(x, q, scale):
    return _ops.act_quant_fp8(x, q, scale)


def moe_gemm_fp8_block(a, a_scale, row_map, weight, weight_scale, expert_start, output, N, K,
                       num_experts, fuse_silu_mul=False):
    """Grouped block-FP8 GEMM; a_scale None -> 16-bit activations (w8a16), else e4m3 activations
    with per-row per-128 scales.  Optional row gather, fused SiLU*mul, fp32 output."""
    return _ops.moe_gemm_fp8_block(a, a_scale, row_map, weight, weight_scale, expert_start, output,
                                   N, K, num_experts, fuse_silu_mul)


def moe_gate_up_fp8_routed(xq, xs, top_ids, weight, weight_scale, expert_start, inv, sorted_pairs, output,
                           num_experts):
    """moe_sort and the gate_up moe_gemm_fp8_block (e4m3 activations, fused SiLU*mul) in one launch,
    for up to 8192 (token, route) pairs; expert_start / inv / sorted_pairs are written for later stages."""
    return _ops.moe_gate_up_fp8_routed(xq, xs, top_ids, weight, weight_scale, expert_start, inv, sorted_pairs,
                                       output, num_experts)


def moe_combine(y, inv, top_w, output, top_k):
    return _ops.moe_combine(y, inv, top_w, output, top_k)


def moe_forward_fp8_block(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale, output,
                          top_k, act_quant=True):
    return _ops.moe_forward_fp8_block(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                      output, top_k, act_quant)


def moe_forward_full_fp8_block(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight,
                               shared_gate_up_scale, down_weight, down_scale, shared_down_weight,
                               shared_down_scale, shared_expert_gate_weight, top_k, num_shared_experts,
                               n_routed_experts):
    """Allocates the output and runs torch.ops.moe_ops.moe_forward_full_fp8_block
    (V/python/custom_esimd_kernels_vllm/ops.py:1092-1125)."""
    output = torch.empty_like(x)
    return torch.ops.moe_ops.moe_forward_full_fp8_block(
        x, logits, output, gate_up_weight, gate_up_scale, shared_gate_up_weight, shared_gate_up_scale,
        down_weight, down_scale, shared_down_weight, shared_down_scale, shared_expert_gate_weight,
        top_k, num_shared_experts, n_routed_experts)


# ---- per-expert-scale FP8 MoE with the tanh-GELU gate (V/python/custom_esimd_kernels_vllm/ops.py:1693-1800)
def moe_forward_full_gelu_tanh(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale, top_k,
                               n_routed_experts):
    return _moe.moe_forward_full_gelu_tanh(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                           top_k, n_routed_experts)


def moe_forward_full_fp8_grouped(x, gate_up_weight, gate_up_scale, down_weight, down_scale, routing_weights,
                                 expert_offsets, expert_tokens, top_k, n_routed_experts):
    return _moe.moe_forward_full_fp8_grouped(x, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                             routing_weights, expert_offsets, expert_tokens, top_k,
                                             n_routed_experts)


def moe_forward_full_gelu_tanh_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight,
                                      down_scale, top_k, n_routed_experts):
    return _moe.moe_forward_full_gelu_tanh_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale,
                                                  down_weight, down_scale, top_k, n_routed_experts)


def moe_forward_full_gelu_tanh_routed_decode(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale,
                                             down_weight, down_scale, top_k, n_routed_experts):
    return _moe.moe_forward_full_gelu_tanh_routed_decode(x, topk_weights, topk_indices, gate_up_weight,
                                                         gate_up_scale, down_weight, down_scale, top_k,
                                                         n_routed_experts)


def moe_forward_full_gelu_tanh_decode(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                      per_expert_scale, top_k, n_routed_experts):
    return _moe.moe_forward_full_gelu_tanh_decode(x, logits, gate_up_weight, gate_up_scale, down_weight,
                                                  down_scale, per_expert_scale, top_k, n_routed_experts)


def moe_forward_full(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight, shared_gate_up_scale,
                     down_weight, down_scale, shared_down_weight, shared_down_scale, shared_expert_gate_weight,
                     top_k, num_shared_experts, n_routed_experts):
    """V/python/custom_esimd_kernels_vllm/ops.py:1063-1090."""
    return _moe.moe_forward_full(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight,
                                 shared_gate_up_scale, down_weight, down_scale, shared_down_weight,
                                 shared_down_scale, shared_expert_gate_weight, top_k, num_shared_experts,
                                 n_routed_experts)

def moe_router_forward(x, weight, scale):
    """Router logits on per-tensor FP8 weights: x [n_tokens, hidden], weight [num_experts, hidden] fp8,
    scale [num_experts] fp32 -> [n_tokens, num_experts] (V/python/custom_esimd_kernels_vllm/ops.py:931-943)."""
    return _moe.moe_router_forward(x, weight, scale)


def moe_batch_topk(logits, top_k, norm=True):
    """(top_values [n_tokens, top_k], top_indices [n_tokens, top_k] int32) (V/python/custom_esimd_kernels_vllm/ops.py:946-958)."""
    return _moe.moe_topk(logits, top_k, norm)


def moe_accumulate(partials, top_k, num_shared_experts):
    """Unweighted sum of each token's top_k + shared rows: partials [n_tokens * (top_k + shared), hidden]
    -> [n_tokens, hidden] (V/python/custom_esimd_kernels_vllm/ops.py:1020-1030)."""
    return _moe.moe_accumulate(partials, top_k, num_shared_experts)



def precompute_moe_route(topk_weights, topk_ids, num_experts):
    """Same contract as the reference helper: (sorted_rows, sorted_weights, rows_per_expert),
    stable by expert; computed on the device by the sort kernel."""
    T, k = topk_ids.shape
    dev = topk_ids.device
    ids = topk_ids.to(torch.int32).contiguous()
    pairs = torch.empty(T * k, dtype=torch.int32, device=dev)
    start = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(T * k, dtype=torch.int32, device=dev)
    tok = torch.empty(T * k, dtype=torch.int32, device=dev)
    moe_sort(ids, num_experts, pairs, start, inv, tok, None)
    return tok.to(torch.int64), topk_weights.reshape(-1)[pairs.long()].contiguous(), (start[1:] - start[:-1]).contiguous()


# decode fusions: RMS norm (+ residual add / SiLU gate) + GEMV
# (V/python/custom_esimd_kernels_vllm/ops.py:340-560)
def esimd_fused_add_rms_norm(hidden_states, residual, weight, eps):
    """residual = hidden_states + residual (in place); hidden_states = rmsnorm(residual) * weight."""
    return _ops.esimd_fused_add_rms_norm(hidden_states, residual, weight, eps)


def esimd_fused_scaled_add_rms_norm(hidden_states, residual, weight, eps, scalar):
    """residual = (hidden_states + residual) * scalar (in place); hidden_states = rmsnorm(residual) * weight."""
    return _ops.esimd_fused_scaled_add_rms_norm(hidden_states, residual, weight, eps, scalar)


def esimd_fused_add_rms_norm_batched(hidden_states, residual, weight, eps):
    return _ops.esimd_fused_add_rms_norm_batched(hidden_states, residual, weight, eps)


def esimd_rms_norm_gated(x, z, weight, output, eps):
    """output = rmsnorm(x) * weight * silu(z); x, z [rows, V], weight [V]."""
    return _ops.esimd_rms_norm_gated(x, z, weight, output, eps)


def esimd_rms_norm(input, output, weight, eps):
    return _ops.esimd_rms_norm(input, output, weight, eps)


def esimd_resadd_norm_gemv_int4_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                     normed_out, eps):
    return _ops.esimd_resadd_norm_gemv_int4_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale,
                                                 output, normed_out, eps)


def esimd_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                    normed_out, eps):
    return _ops.esimd_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale,
                                                output, normed_out, eps)


def esimd_resadd_norm_gemv2_fp8_pert(hidden_states, residual, norm_weight, w0, s0, o0, w1, s1, o1, eps):
    return _ops.esimd_resadd_norm_gemv2_fp8_pert(hidden_states, residual, norm_weight, w0, s0, o0, w1, s1, o1, eps)


def esimd_scaled_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, qkv_weight, qkv_scale, qkv_out, eps,
                                           scalar):
    return _ops.esimd_scaled_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, qkv_weight, qkv_scale,
                                                       qkv_out, eps, scalar)


def esimd_norm_gemv_norm_fp16(residual, scale_with_root, proj_w, pre_ff_w, router_logits, moe_input, eps):
    return _ops.esimd_norm_gemv_norm_fp16(residual, scale_with_root, proj_w, pre_ff_w, router_logits, moe_input, eps)


def esimd_norm_add_norm(h2_raw, h1, w1, w2, out, eps1, eps2):
    return _ops.esimd_norm_add_norm(h2_raw, h1, w1, w2, out, eps1, eps2)


def esimd_accum_norm_add_norm(routed_output, h1, w1, w2, out, top_k, eps1, eps2):
    return _ops.esimd_accum_norm_add_norm(routed_output, h1, w1, w2, out, top_k, eps1, eps2)


def esimd_norm_gemv_int4_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    return _ops.esimd_norm_gemv_int4_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps)


def esimd_norm_gemv_fp8_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    return _ops.esimd_norm_gemv_fp8_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps)


def esimd_norm_gemv_fp8_blockscale(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    return _ops.esimd_norm_gemv_fp8_blockscale(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps)


def q4_0_quantize(input, out_qweight, out_scale):
    """torch.ops.custom_esimd_kernels_vllm.q4_0_quantize (the reference registers it from its
    q4_0_quant_ops module): [M, K] fp16/bf16 -> int32 [M, K/8] + fp16 scale [M, K/128]."""
    return _ops.q4_0_quantize(input, out_qweight, out_scale)


# Read unguarded by the patched callers but outside the quantized-linear path (attention, GDN, RoPE and
# INT4-MoE fusions): the names exist so the callers import, and raise when called
# (vllm/patches/vllm_for_multi_arc.patch:3149, :3159-3160, :8518-8520, :10011-10014).
from mi355x_qlinear.not_provided import NotProvided as _NotProvided  # noqa: E402

esimd_qkv_split_norm_rope = _NotProvided("esimd_qkv_split_norm_rope", "DISABLE_ESIMD_QKV=1")
esimd_qkv_split_norm_rope_v = _NotProvided("esimd_qkv_split_norm_rope_v", "DISABLE_ESIMD_QKV_FUSED=1")
esimd_gdn_conv_fused = _NotProvided("esimd_gdn_conv_fused", "DISABLE_ESIMD_GDN_CONV=1")
esimd_gdn_conv_fused_seq = _NotProvided("esimd_gdn_conv_fused_seq", "DISABLE_ESIMD_GDN_CONV=1")
moe_forward_full_cutlass_nmajor_int4 = _NotProvided("moe_forward_full_cutlass_nmajor_int4", "DISABLE_ESIMD_INT4=1 (sym_int4 MoE models)")
moe_forward_tiny_cutlass_nmajor_int4_full_fp16_shared_from_logits = _NotProvided(
    "moe_forward_tiny_cutlass_nmajor_int4_full_fp16_shared_from_logits", "DISABLE_ESIMD_INT4=1 (sym_int4 MoE models)")
