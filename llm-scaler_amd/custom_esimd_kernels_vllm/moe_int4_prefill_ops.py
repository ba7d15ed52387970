"""Stand-in for the reference's compiled `custom_esimd_kernels_vllm.moe_int4_prefill_ops` extension: the
patched vLLM imports it for its side effect of registering
`torch.ops.moe_int4_prefill_ops.moe_prefill_gather_forward_v2`, which groups tokens by expert for the FP8
grouped MoE ops too (vllm/patches/vllm_for_multi_arc.patch:8218-8240).  Only the weight-format-agnostic
ops of that namespace are provided (the gather and the softmax top-k); the INT4 prefill GEMMs are not."""
import torch

import mi355x_qlinear  # noqa: F401  (registers torch.ops.moe_int4_prefill_ops)


def __getattr__(name):
    return getattr(torch.ops.moe_int4_prefill_ops, name)
