"""Drop-in for the reference's `custom_esimd_kernels_vllm` Python package
(vllm/custom-esimd-kernels-vllm/python/custom_esimd_kernels_vllm/__init__.py):
importing it registers the torch.ops and re-exports the thin wrappers."""
import mi355x_qlinear  # noqa: F401  (registers torch.ops.* for ROCm tensors)

from .ops import *  # noqa: F401,F403
from . import moe_ops  # noqa: F401,E402
from . import moe_int4_prefill_ops  # noqa: F401,E402
from . import eagle_ops  # noqa: F401,E402
