"""Stand-in for the reference's compiled `custom_esimd_kernels_sglang.moe_fp8_prefill_ops` extension
(sglang/custom-esimd-kernels/setup.py:343): the patched SGLang imports it for its side effect of
registering torch.ops.moe_fp8_prefill_ops.* and then takes `moe_prefill_full_fp8` from there
(sglang/patches/sglang_for_multi_arc.patch:1413-1416)."""
import torch

import mi355x_qlinear  # noqa: F401  (registers torch.ops.moe_fp8_prefill_ops)


def __getattr__(name):
    return getattr(torch.ops.moe_fp8_prefill_ops, name)
