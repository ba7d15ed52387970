"""Names the reference's patched callers read from the kernel packages without a guard, for kernels
that are not part of the quantized-linear path (attention, GDN, RoPE, INT4-MoE fusions).

The patched vLLM binds them at import time (`esimd_qkv_split_norm_rope = _esimd.esimd_qkv_split_norm_rope`,
vllm/patches/vllm_for_multi_arc.patch:3149, :3159-3160, :3205), so the names have to exist for the
caller's module to import at all.  Each one is a callable that computes nothing and raises: there is no
fallback arithmetic behind it, and the message names the caller-side switch that keeps the call site
from being reached.
"""


class NotProvided:
    """Callable placeholder: `name` is not built on MI355X; `switch` is the environment variable of the
    reference's caller that routes around the call site."""

    def __init__(self, name, switch):
        self.__name__ = name
        self.__qualname__ = name
        self.switch = switch

    def __call__(self, *args, **kwargs):
        raise RuntimeError(
            f"{self.__name__} is not provided on MI355X (it is outside the quantized-linear path); "
            f"set {self.switch} so the caller takes its stock path")

    def __repr__(self):
        return f"<not provided on MI355X: {self.__name__} ({self.switch})>"
