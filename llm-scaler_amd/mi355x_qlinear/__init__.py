"""Host side of the gfx950 quantized-linear kernels.

`capi` loads libmi355x_qlinear.so (built in-tree by `make -C csrc`) through
ctypes; `ops` registers the torch.ops schemas that the reference's vLLM / SGLang
patches call, with implementations that forward device pointers to the C ABI.
There is no CPU or eager fallback: without the built library every op raises.
"""
from . import capi  # noqa: F401
from . import ops  # noqa: F401
