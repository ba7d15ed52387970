"""ctypes binding of the C ABI declared in include/mi355x_qlinear.h.

The header is the single source of truth: its prototypes are parsed at import
and turned into ctypes signatures, so a symbol that the header declares but the
library does not export fails here, loudly.
"""
from __future__ import annotations

import ctypes
import os
import re

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG_ROOT = os.path.dirname(_HERE)
HEADER = os.path.join(os.path.dirname(_PKG_ROOT), "include", "mi355x_qlinear.h")
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "libmi355x_qlinear.so")

MI_ERRORS = {-1: "invalid argument (null pointer or bad enum)",
             -2: "unsupported shape or divisibility",
             -3: "kernel launch failed",
             -4: "size beyond the fixed capacity of this no-allocation entry point",
             -5: "the static scratch is claimed by another stream on this GPU"}

DT_F16, DT_BF16 = 0, 1
_ACT_DT = {torch.float16: DT_F16, torch.bfloat16: DT_BF16}

_PROTO = re.compile(r"^int\s+(mi_\w+)\s*\(([^;]*?)\)\s*;", re.S | re.M)


def parse_header(path: str = HEADER):
    """-> {name: [ctypes type per parameter]} for every `int mi_*(...)` prototype."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for name, params in _PROTO.findall(text):
        types = []
        for p in params.split(","):
            p = " ".join(p.split())
            if p == "void":                       # f(void): no parameters
                continue
            if "*" in p:
                types.append(ctypes.c_void_p)
            elif p.startswith("long long") or p.startswith("int64_t"):
                types.append(ctypes.c_longlong)
            elif p.startswith("float"):
                types.append(ctypes.c_float)
            elif p.startswith("int"):
                types.append(ctypes.c_int)
            else:
                raise RuntimeError(f"mi355x_qlinear: cannot map parameter '{p}' of {name}")
        protos[name] = types
    return protos


_lib = None


def lib():
    """The loaded shared library; raises ImportError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"mi355x_qlinear: {LIB_PATH} is missing - build it with "
                f"`make -C {os.path.join(_PKG_ROOT, 'csrc')}` (hipcc, gfx950). "
                "There is no fallback path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, types in parse_header().items():
            try:
                fn = getattr(handle, name)
            except AttributeError as e:
                raise ImportError(f"mi355x_qlinear: {LIB_PATH} does not export {name}") from e
            fn.argtypes = types
            fn.restype = ctypes.c_int
        _lib = handle
    return _lib


def _device_ptr(t) -> int:
    # a host address handed to a kernel is a GPU memory fault, not an error code: refuse it here
    if not t.is_cuda:
        raise RuntimeError(f"mi355x_qlinear: every tensor operand must live on a ROCm device, got one on {t.device}")
    return t.data_ptr()


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return None
    return ctypes.c_void_p(_device_ptr(t))


def ptr_array(tensors):
    arr = (ctypes.c_void_p * len(tensors))(*[0 if t is None else _device_ptr(t) for t in tensors])
    return arr


def int_array(vals):
    return (ctypes.c_int * len(vals))(*[int(v) for v in vals])


def act_dtype(t: torch.Tensor) -> int:
    try:
        return _ACT_DT[t.dtype]
    except KeyError:
        raise RuntimeError(f"mi355x_qlinear: activations must be fp16 or bf16, got {t.dtype}") from None


def stream_of(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def call(name: str, anchor: torch.Tensor, *args):
    """Run C entry `name` on `anchor`'s device and current stream; the stream
    argument (always last in the ABI) is appended here."""
    fn = getattr(lib(), name)
    if not anchor.is_cuda:
        raise RuntimeError(f"{name}: tensors must live on a ROCm device, got {anchor.device}")
    with torch.cuda.device(anchor.device):
        rc = fn(*args, stream_of(anchor))
    if rc != 0:
        raise RuntimeError(f"{name} failed: {MI_ERRORS.get(rc, rc)}")
