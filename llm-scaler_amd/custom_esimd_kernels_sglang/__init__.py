"""Drop-in for the reference's `custom_esimd_kernels_sglang` Python package
(sglang/custom-esimd-kernels/python/custom_esimd_kernels_sglang/__init__.py)."""
import mi355x_qlinear  # noqa: F401

from .ops import *  # noqa: F401,F403
