"""Stand-in for the reference's compiled `custom_esimd_kernels_vllm.eagle_ops` module
(vllm/custom-esimd-kernels-vllm/python/custom_esimd_kernels_vllm/__init__.py:14-16).  The patched
vLLM binds `_esimd.eagle_ops.page_attn_decode` at import time
(vllm/patches/vllm_for_multi_arc.patch:3205); paged attention is not part of the quantized-linear
path, so the name exists and raises when called."""
from mi355x_qlinear.not_provided import NotProvided

page_attn_decode = NotProvided("eagle_ops.page_attn_decode", "DISABLE_ESIMD_PA=1 and DISABLE_ESIMD_PAGE_ATTN=1")
