"""Stand-in for the reference's compiled `custom_esimd_kernels_sglang.moe_ops` extension
(sglang/custom-esimd-kernels/setup.py:318): importing it makes torch.ops.moe_ops.* available, and
its attributes are those ops (the patched SGLang runner takes
`custom_esimd_kernels_sglang.moe_ops.moe_forward_full_silu_routed_sglang`,
sglang/patches/sglang_for_multi_arc.patch:1166-1186)."""
import torch

import mi355x_qlinear  # noqa: F401  (registers torch.ops.moe_ops)


def __getattr__(name):
    return getattr(torch.ops.moe_ops, name)
