"""Stand-in for the reference's compiled `custom_esimd_kernels_vllm.moe_ops` module
(vllm/custom-esimd-kernels-vllm/python/custom_esimd_kernels_vllm/__init__.py:12-13): importing it
makes torch.ops.moe_ops.* available, and its attributes are those ops (callers use e.g.
`custom_esimd_kernels_vllm.moe_ops.moe_forward_full_v2`)."""
import torch

import mi355x_qlinear  # noqa: F401  (registers torch.ops.moe_ops)


def __getattr__(name):
    return getattr(torch.ops.moe_ops, name)
