"""torch.ops registration: the reference's op names, argument order and layouts.

Schemas follow the reference's registration files
(vllm/custom-esimd-kernels-vllm/csrc/xpu/torch_extension.cc:8-61,
torch_extension_gemm.cc:11-40, torch_extension_moe.cc:11-57,
sglang/custom-esimd-kernels/csrc/xpu/torch_extension.cc:65-69) so that the vLLM
and SGLang call sites work unchanged.  The reference registers for the XPU
dispatch key; here the implementations are registered for CUDA, which is the key
ROCm tensors dispatch on.  Conventions kept from the reference: the caller
pre-allocates every output, the op writes it in place on the current stream and
returns that same tensor, and nothing synchronises.

Ops whose names end in a suffix the reference does not have (`*_zp`, `*_m`,
`esimd_gemm_q4_k`, `q4_k_repack`, `*_dequant*`) are siblings added for shapes and
operands the reference's kernels do not take; the reference-named ops keep their
exact signatures.
"""
from __future__ import annotations

import ctypes

import torch

from . import capi

_FP8_TYPES = (torch.float8_e4m3fn, torch.uint8)

_libs = {}


def _library(ns: str) -> torch.library.Library:
    if ns not in _libs:
        _libs[ns] = torch.library.Library(ns, "FRAGMENT")
    return _libs[ns]


_DEFINED = {}        # namespace -> names of the operators defined here


def _define(ns: str, schema: str, impl, meta=None):
    lib = _library(ns)
    lib.define(schema)
    name = schema.split("(", 1)[0]
    _DEFINED.setdefault(ns, []).append(name)
    lib.impl(name, impl, "CUDA")
    if meta is not None:
        lib.impl(name, meta, "Meta")


def _chk(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def _chk_fp8(w: torch.Tensor, who: str):
    _chk(w.dtype in _FP8_TYPES,
         f"{who}: weight must be float8_e4m3fn (or uint8 holding E4M3 bits), got {w.dtype}")
    _chk(w.is_contiguous(), f"{who}: weight must be contiguous")


def _chk_act(x: torch.Tensor, out: torch.Tensor, who: str):
    _chk(x.dtype in (torch.float16, torch.bfloat16), f"{who}: input must be fp16 or bf16, got {x.dtype}")
    _chk(out.dtype == x.dtype, f"{who}: output dtype {out.dtype} must match input dtype {x.dtype}")
    _chk(x.is_contiguous() and out.is_contiguous(), f"{who}: input and output must be contiguous")


# --------------------------------------------------------------------------
# Prefill route (M > 64, K % 128 == 0) of the FP8 and Q4_K ops: the tiled matrix-core GEMM.  The
# re-tiled activations live in a workspace from torch's caching allocator, so that the op stays
# capturable in a HIP graph.
# --------------------------------------------------------------------------
_SC_PERN, _SC_PERT, _SC_BLOCK = 0, 1, 2


def _tiled_workspace(x, M, K):
    need = ctypes.c_longlong(0)
    rc = capi.lib().mi_gemm_tiled_workspace(M, K, ctypes.byref(need))
    if rc != 0:
        raise RuntimeError(f"mi_gemm_tiled_workspace: {capi.MI_ERRORS.get(rc, rc)}")
    return torch.empty(need.value, dtype=torch.uint8, device=x.device), need.value


def _prefill_route(M, K):
    return M > 64 and K % 128 == 0


def _fp8_tiled_multi(x, ws, ss, os_, Ns, M, K, mode, scale_f16):
    buf, nbytes = _tiled_workspace(x, M, K)
    for w, s, o, N in zip(ws, ss, os_, Ns):
        capi.call("mi_gemm_fp8_tiled_ws", x, capi.ptr(x), capi.ptr(w), capi.ptr(s), mode, 1 if scale_f16 else 0,
                  capi.ptr(o), capi.ptr(buf), nbytes, M, int(N), K, capi.act_dtype(x))
    return os_[0]


# --------------------------------------------------------------------------
# FP8 per-channel  (esimd_gemv_fp8_pern, _fused2, _fused3)
# --------------------------------------------------------------------------
def _fp8_pern_multi(x, ws, ss, os_, Ns, K, who):
    K = int(K)
    _chk(K > 0 and x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    M = x.numel() // K
    sdt = ss[0].dtype
    for w, s, o, N in zip(ws, ss, os_, Ns):
        _chk_fp8(w, who)
        _chk_act(x, o, who)
        _chk(w.numel() == int(N) * K, f"{who}: weight has {w.numel()} elements, expected N*K={int(N) * K}")
        _chk(s.dtype == sdt and sdt in (torch.float16, torch.float32),
             f"{who}: weight_scale must be fp16 or fp32 (all the same), got {s.dtype}")
        _chk(s.numel() == int(N), f"{who}: weight_scale must have N={int(N)} entries")
        _chk(o.numel() == M * int(N), f"{who}: output has {o.numel()} elements, expected M*N={M * int(N)}")
    if _prefill_route(M, K):
        return _fp8_tiled_multi(x, ws, ss, os_, Ns, M, K, _SC_PERN, sdt == torch.float16)
    capi.call("mi_gemm_fp8_pern_multi", x, capi.ptr(x), len(ws), capi.ptr_array(ws), capi.ptr_array(ss),
              capi.ptr_array(os_), capi.int_array(Ns), M, K, capi.act_dtype(x),
              1 if sdt == torch.float16 else 0)
    return os_[0]


def esimd_gemv_fp8_pern(input, weight, weight_scale, output, N, K):
    return _fp8_pern_multi(input, [weight], [weight_scale], [output], [N], K, "esimd_gemv_fp8_pern")


def esimd_gemv_fp8_pern_fused2(input, w0, s0, o0, N0, w1, s1, o1, N1, K):
    return _fp8_pern_multi(input, [w0, w1], [s0, s1], [o0, o1], [N0, N1], K, "esimd_gemv_fp8_pern_fused2")


def esimd_gemv_fp8_pern_fused3(input, w0, s0, o0, N0, w1, s1, o1, N1, w2, s2, o2, N2, K):
    return _fp8_pern_multi(input, [w0, w1, w2], [s0, s1, s2], [o0, o1, o2], [N0, N1, N2], K,
                           "esimd_gemv_fp8_pern_fused3")


# --------------------------------------------------------------------------
# FP8 per-tensor  (esimd_gemv_fp8_pert, _fused2/3, _bmg, esimd_gemm_fp8_pert)
# --------------------------------------------------------------------------
def _fp8_pert_multi(x, ws, ss, os_, who):
    _chk(ws[0].dim() == 2, f"{who}: weight must be [N, K]")
    K = ws[0].shape[1]
    _chk(x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    M = x.numel() // K
    Ns = []
    for w, s, o in zip(ws, ss, os_):
        _chk_fp8(w, who)
        _chk_act(x, o, who)
        _chk(w.dim() == 2 and w.shape[1] == K, f"{who}: all weights must be [N, K={K}]")
        _chk(s.dtype == torch.float32 and s.numel() >= 1, f"{who}: weight_scale must be an fp32 scalar tensor")
        _chk(o.numel() == M * w.shape[0], f"{who}: output has {o.numel()} elements, expected {M * w.shape[0]}")
        Ns.append(w.shape[0])
    if _prefill_route(M, K):
        return _fp8_tiled_multi(x, ws, ss, os_, Ns, M, K, _SC_PERT, False)
    capi.call("mi_gemm_fp8_pert_multi", x, capi.ptr(x), len(ws), capi.ptr_array(ws), capi.ptr_array(ss),
              capi.ptr_array(os_), capi.int_array(Ns), M, K, capi.act_dtype(x))
    return os_[0]


def esimd_gemv_fp8_pert(input, weight, weight_scale, output):
    return _fp8_pert_multi(input, [weight], [weight_scale], [output], "esimd_gemv_fp8_pert")


def esimd_gemv_fp8_pert_bmg(input, weight, weight_scale, output):
    return _fp8_pert_multi(input, [weight], [weight_scale], [output], "esimd_gemv_fp8_pert_bmg")


def esimd_gemm_fp8_pert(input, weight, weight_scale, output):
    return _fp8_pert_multi(input, [weight], [weight_scale], [output], "esimd_gemm_fp8_pert")


def esimd_gemv_fp8_pert_fused2(input, w0, s0, o0, w1, s1, o1):
    return _fp8_pert_multi(input, [w0, w1], [s0, s1], [o0, o1], "esimd_gemv_fp8_pert_fused2")


def esimd_gemv_fp8_pert_fused3(input, w0, s0, o0, w1, s1, o1, w2, s2, o2):
    return _fp8_pert_multi(input, [w0, w1, w2], [s0, s1, s2], [o0, o1, o2], "esimd_gemv_fp8_pert_fused3")


# --------------------------------------------------------------------------
# FP8 128x128 block scale  (esimd_gemm_fp8_blockscale, esimd_gemv_fp8_blockscale_fused2)
# --------------------------------------------------------------------------
def _fp8_block_multi(x, ws, ss, os_, block_n, block_k, who):
    _chk(int(block_n) == 128 and int(block_k) == 128, f"{who}: only block_n == block_k == 128 is supported")
    _chk(x.dim() == 2, f"{who}: input must be [M, K]")
    M, K = x.shape
    _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
    Ns = []
    for w, s, o in zip(ws, ss, os_):
        _chk_fp8(w, who)
        _chk_act(x, o, who)
        _chk(w.dim() == 2 and w.shape[1] == K, f"{who}: weight must be [N, K={K}]")
        N = w.shape[0]
        _chk(s.dtype == torch.float32 and s.is_contiguous(), f"{who}: weight_scale must be contiguous fp32")
        _chk(tuple(s.shape) == ((N + 127) // 128, K // 128),
             f"{who}: weight_scale must be [ceil(N/128), K/128] = {((N + 127) // 128, K // 128)}, got {tuple(s.shape)}")
        _chk(o.numel() == M * N, f"{who}: output must be [M, N]")
        Ns.append(N)
    if _prefill_route(M, K):
        return _fp8_tiled_multi(x, ws, ss, os_, Ns, M, K, _SC_BLOCK, False)
    capi.call("mi_gemm_fp8_blockscale_multi", x, capi.ptr(x), len(ws), capi.ptr_array(ws), capi.ptr_array(ss),
              capi.ptr_array(os_), capi.int_array(Ns), M, K, capi.act_dtype(x))
    return os_[0]


def esimd_gemm_fp8_blockscale(input, weight, weight_scale, output, block_n, block_k):
    return _fp8_block_multi(input, [weight], [weight_scale], [output], block_n, block_k,
                            "esimd_gemm_fp8_blockscale")


def esimd_gemv_fp8_blockscale_fused2(input, w0, s0, o0, w1, s1, o1, block_n, block_k):
    return _fp8_block_multi(input, [w0, w1], [s0, s1], [o0, o1], block_n, block_k,
                            "esimd_gemv_fp8_blockscale_fused2")


# --------------------------------------------------------------------------
# 16-bit weights beside the quantized ones (esimd_gemv_fp16, _gelu_mul, the fp16 half of
# esimd_gemv_fp8_blockscale_fp16_fused2)
# --------------------------------------------------------------------------
def _gemv_w16(x, w, out, gelu, who):
    _chk(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, f"{who}: input [M, K], weight [N, K], output [M, N]")
    _chk_act(x, out, who)
    _chk(w.dtype == x.dtype and w.is_contiguous(), f"{who}: weight must be contiguous and share the input dtype")
    M, K = x.shape
    rows = w.shape[0]
    _chk(w.shape[1] == K and K % 8 == 0, f"{who}: weight must be [N, K={K}] with K a multiple of 8")
    _chk(not gelu or rows % 2 == 0, f"{who}: the gate-up weight must have an even number of rows")
    N = rows // 2 if gelu else rows
    _chk(tuple(out.shape) == (M, N), f"{who}: output must be [M, N] = {(M, N)}, got {tuple(out.shape)}")
    capi.call("mi_gemv_w16", x, capi.ptr(x), capi.ptr(w), capi.ptr(out), M, N, K, 1 if gelu else 0, capi.act_dtype(x))
    return out


def esimd_gemv_fp16(input, weight, output):
    """out = input @ weight^T on 16-bit weights (V/csrc/xpu/torch_extension.cc:27-28); bf16 accepted too."""
    return _gemv_w16(input, weight, output, False, "esimd_gemv_fp16")


def esimd_gemv_fp16_gelu_mul(input, weight, output):
    """weight [2N, K], gate rows first: out = gelu_tanh(input @ gate^T) * (input @ up^T)
    (V/csrc/xpu/torch_extension.cc:30-33)."""
    return _gemv_w16(input, weight, output, True, "esimd_gemv_fp16_gelu_mul")


def esimd_gemv_fp8_blockscale_fp16_fused2(input, w0, s0, o0, w1, o1, block_n, block_k):
    """A block-scaled FP8 weight and a 16-bit weight sharing the input
    (V/csrc/xpu/torch_extension_gemm.cc:37-41).  Two launches here: the formats do not share a kernel."""
    who = "esimd_gemv_fp8_blockscale_fp16_fused2"
    _fp8_block_multi(input, [w0], [s0], [o0], block_n, block_k, who)
    _gemv_w16(input, w1, o1, False, who)
    return o0


# --------------------------------------------------------------------------
# INT4 group-128  (esimd_gemv_int4, _fused2, esimd_gemm_int4_pgrp [+ _zp sibling])
# --------------------------------------------------------------------------
def _int4_nk(w: torch.Tensor, who: str):
    """Accepts the uint8 [N, K/2] and the int32 [N, K/8] view of the same bytes."""
    _chk(w.dim() == 2 and w.is_contiguous(), f"{who}: weight must be a contiguous 2-D tensor")
    if w.dtype == torch.uint8:
        return w.shape[0], w.shape[1] * 2
    if w.dtype == torch.int32:
        return w.shape[0], w.shape[1] * 8
    raise RuntimeError(f"{who}: weight must be uint8 [N, K/2] or int32 [N, K/8], got {w.dtype}")


def _chk_int4(x, w, s, zp, o, who):
    N, K = _int4_nk(w, who)
    _chk_act(x, o, who)
    _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of the group size 128")
    _chk(x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    M = x.numel() // K
    _chk(s.dtype == torch.float16 and s.is_contiguous() and s.numel() == N * (K // 128),
         f"{who}: weight_scale must be contiguous fp16 [N, K/128]")
    if zp is not None:
        _chk(zp.dtype == torch.uint8 and zp.is_contiguous() and zp.numel() == N * (K // 128),
             f"{who}: weight_zp must be contiguous uint8 [N, K/128] with values 0..15")
    _chk(o.numel() == M * N, f"{who}: output has {o.numel()} elements, expected M*N={M * N}")
    return M, N, K


def _int4_multi(x, ws, ss, zps, os_, who):
    Ns, M, K = [], None, None
    for w, s, zp, o in zip(ws, ss, zps, os_):
        m, n, k = _chk_int4(x, w, s, zp, o, who)
        _chk(K is None or k == K, f"{who}: all weights must share K")
        M, K = m, k
        Ns.append(n)
    zarr = capi.ptr_array(zps) if any(z is not None for z in zps) else None
    capi.call("mi_gemv_int4_multi", x, capi.ptr(x), len(ws), capi.ptr_array(ws), capi.ptr_array(ss), zarr,
              capi.ptr_array(os_), capi.int_array(Ns), M, K, capi.act_dtype(x))
    return os_[0]


def esimd_gemv_int4(input, weight, weight_scale, output):
    return _int4_multi(input, [weight], [weight_scale], [None], [output], "esimd_gemv_int4")


def esimd_gemv_int4_fused2(input, w0, s0, o0, w1, s1, o1):
    return _int4_multi(input, [w0, w1], [s0, s1], [None, None], [o0, o1], "esimd_gemv_int4_fused2")


def _gemm_int4(x, w, s, zp, o, who):
    M, N, K = _chk_int4(x, w, s, zp, o, who)
    # the prefill kernel re-tiles the activations into a workspace; it comes from torch's
    # caching allocator so that the op stays capturable in a HIP graph
    need = ctypes.c_longlong(0)
    rc = capi.lib().mi_gemm_int4_workspace(M, N, K, ctypes.byref(need))
    if rc != 0:
        raise RuntimeError(f"{who}: {capi.MI_ERRORS.get(rc, rc)}")
    ws = torch.empty(need.value, dtype=torch.uint8, device=x.device) if need.value else None
    capi.call("mi_gemm_int4_ws", x, capi.ptr(x), capi.ptr(w), capi.ptr(s), capi.ptr(zp), capi.ptr(o),
              capi.ptr(ws), need.value, M, N, K, capi.act_dtype(x))
    return o


def esimd_gemm_int4_pgrp(input, weight, weight_scale, output):
    """Symmetric (implicit zero-point 8) group-128 int4 GEMM for any M."""
    return _gemm_int4(input, weight, weight_scale, None, output, "esimd_gemm_int4_pgrp")


def esimd_gemm_int4_pgrp_zp(input, weight, weight_scale, weight_zp, output):
    """Asymmetric sibling: weight_zp [N, K/128] uint8 with values 0..15; w = (nibble - zp) * scale."""
    return _gemm_int4(input, weight, weight_scale, weight_zp, output, "esimd_gemm_int4_pgrp_zp")


# --------------------------------------------------------------------------
# GGUF Q4_K  (esimd_gemv_q4_k + siblings)
# --------------------------------------------------------------------------
def _chk_q4k(x, w, s, mn, o, who):
    _chk(w.dtype == torch.uint8 and w.dim() == 2 and w.is_contiguous(), f"{who}: weight must be contiguous uint8 [N, K/2]")
    N, K = w.shape[0], w.shape[1] * 2
    _chk(K % 32 == 0, f"{who}: K={K} must be a multiple of 32")
    _chk(x.dtype == torch.float16 and o.dtype == torch.float16, f"{who}: input and output must be fp16")
    _chk(x.is_contiguous() and o.is_contiguous(), f"{who}: input and output must be contiguous")
    for t, nm in ((s, "weight_scale"), (mn, "weight_min")):
        _chk(t.dtype == torch.float16 and t.is_contiguous() and t.numel() == N * (K // 32),
             f"{who}: {nm} must be contiguous fp16 [N, K/32]")
    _chk(x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    M = x.numel() // K
    _chk(o.numel() == M * N, f"{who}: output has {o.numel()} elements, expected M*N={M * N}")
    return M, N, K


def esimd_gemv_q4_k(input, weight, weight_scale, weight_min, output):
    M, N, K = _chk_q4k(input, weight, weight_scale, weight_min, output, "esimd_gemv_q4_k")
    if _prefill_route(M, K):
        buf, nbytes = _tiled_workspace(input, M, K)
        capi.call("mi_gemm_q4k_tiled_ws", input, capi.ptr(input), capi.ptr(weight), capi.ptr(weight_scale),
                  capi.ptr(weight_min), capi.ptr(output), capi.ptr(buf), nbytes, M, N, K)
        return output
    capi.call("mi_gemv_q4k", input, capi.ptr(input), capi.ptr(weight), capi.ptr(weight_scale),
              capi.ptr(weight_min), capi.ptr(output), M, N, K)
    return output


def q4_k_repack(qweight, ql, weight_scale, weight_min):
    """Raw GGUF super-blocks [N, K/256*144] uint8 -> (ql, scale, min), written in place."""
    who = "q4_k_repack"
    _chk(qweight.dtype == torch.uint8 and qweight.dim() == 2 and qweight.is_contiguous(),
         f"{who}: qweight must be contiguous uint8 [N, nsb*144]")
    _chk(qweight.shape[1] % 144 == 0, f"{who}: row length {qweight.shape[1]} is not a multiple of 144")
    N, K = qweight.shape[0], qweight.shape[1] // 144 * 256
    _chk(ql.dtype == torch.uint8 and ql.is_contiguous() and ql.numel() == N * K // 2, f"{who}: ql must be uint8 [N, K/2]")
    for t in (weight_scale, weight_min):
        _chk(t.dtype == torch.float16 and t.is_contiguous() and t.numel() == N * K // 32,
             f"{who}: scale / min must be fp16 [N, K/32]")
    capi.call("mi_q4k_repack", qweight, capi.ptr(qweight), capi.ptr(ql), capi.ptr(weight_scale),
              capi.ptr(weight_min), N, K)
    return ql


def q4_k_dequant(weight, weight_scale, weight_min, output):
    who = "q4_k_dequant"
    _chk(weight.dtype == torch.uint8 and weight.dim() == 2 and weight.is_contiguous(), f"{who}: weight must be uint8 [N, K/2]")
    N, K = weight.shape[0], weight.shape[1] * 2
    _chk(K % 32 == 0, f"{who}: K must be a multiple of 32")
    _chk(output.dtype == torch.float16 and output.is_contiguous() and output.numel() == N * K,
         f"{who}: output must be contiguous fp16 [N, K]")
    capi.call("mi_dequant_q4k", weight, capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(weight_min),
              capi.ptr(output), N, K)
    return output


# --------------------------------------------------------------------------
# Other GGUF formats: Q4_0, Q8_0, Q5_K, Q6_K (S/csrc/xpu/torch_extension.cc:48-106)
# and the group-128 Q4_0 quantizer (V/csrc/xpu/torch_extension_q4_0.cc:27-75)
# --------------------------------------------------------------------------
def _chk_gguf_io(x, o, N, K, who):
    _chk(x.dtype == torch.float16 and o.dtype == torch.float16, f"{who}: input and output must be fp16")
    _chk(x.is_contiguous() and o.is_contiguous(), f"{who}: input and output must be contiguous")
    _chk(x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    M = x.numel() // K
    _chk(o.numel() == M * N, f"{who}: output has {o.numel()} elements, expected M*N={M * N}")
    return M


def _chk_u8(t, shape, nm, who, dtypes=(torch.uint8,)):
    _chk(t.dtype in dtypes and t.is_contiguous() and tuple(t.shape) == tuple(shape),
         f"{who}: {nm} must be contiguous {'/'.join(str(d) for d in dtypes)} {list(shape)}, got {t.dtype} {list(t.shape)}")


def _chk_f16(t, numel, nm, who):
    _chk(t.dtype == torch.float16 and t.is_contiguous() and t.numel() == numel,
         f"{who}: {nm} must be contiguous fp16 with {numel} elements")


def _gemv_q4_0(input, weight, weight_scale, output, who):
    _chk(weight.dtype == torch.uint8 and weight.dim() == 2 and weight.is_contiguous(),
         f"{who}: weight must be contiguous uint8 [N, K/2]")
    N, K = weight.shape[0], weight.shape[1] * 2
    _chk(K % 32 == 0, f"{who}: K={K} must be a multiple of 32")
    _chk_f16(weight_scale, N * (K // 32), "weight_scale [N, K/32]", who)
    M = _chk_gguf_io(input, output, N, K, who)
    capi.call("mi_gemv_q4_0", input, capi.ptr(input), capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(output), M, N, K)
    return output


def esimd_gemv_q4_0(input, weight, weight_scale, output):
    """weight [N, K/2] uint8 interleaved nibbles, scale [N, K/32] fp16; w = (nib - 8) * scale."""
    return _gemv_q4_0(input, weight, weight_scale, output, "esimd_gemv_q4_0")


def esimd_gemm_q4_0(input, weight, weight_scale, output):
    """The reference's M >= 2 op on the same layout; one kernel family serves both here."""
    return _gemv_q4_0(input, weight, weight_scale, output, "esimd_gemm_q4_0")


def _gemv_q8_0(input, weight, weight_scale, output, who):
    _chk(weight.dtype in (torch.int8, torch.uint8) and weight.dim() == 2 and weight.is_contiguous(),
         f"{who}: weight must be contiguous int8 [N, K]")
    N, K = weight.shape
    _chk(K % 32 == 0, f"{who}: K={K} must be a multiple of 32")
    _chk_f16(weight_scale, N * (K // 32), "weight_scale [N, K/32]", who)
    M = _chk_gguf_io(input, output, N, K, who)
    capi.call("mi_gemv_q8_0", input, capi.ptr(input), capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(output), M, N, K)
    return output


def esimd_gemv_q8_0(input, weight, weight_scale, output):
    """weight [N, K] int8, scale [N, K/32] fp16; w = qs * scale."""
    return _gemv_q8_0(input, weight, weight_scale, output, "esimd_gemv_q8_0")


def esimd_gemv_q8_0_m(input, weight, weight_scale, output):
    return _gemv_q8_0(input, weight, weight_scale, output, "esimd_gemv_q8_0_m")


def esimd_gemv_q5_k(input, ql, qh, weight_scale, weight_min, output):
    """ql [N, K/2], qh [N, K/8] (tile-shuffled fifth bits), scale / min [N, K/32] fp16."""
    who = "esimd_gemv_q5_k"
    _chk(ql.dtype == torch.uint8 and ql.dim() == 2 and ql.is_contiguous(), f"{who}: ql must be contiguous uint8 [N, K/2]")
    N, K = ql.shape[0], ql.shape[1] * 2
    _chk(K % 512 == 0, f"{who}: K={K} must be a multiple of 512")
    _chk_u8(qh, (N, K // 8), "qh", who)
    _chk_f16(weight_scale, N * (K // 32), "weight_scale [N, K/32]", who)
    _chk_f16(weight_min, N * (K // 32), "weight_min [N, K/32]", who)
    M = _chk_gguf_io(input, output, N, K, who)
    capi.call("mi_gemv_q5k", input, capi.ptr(input), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale),
              capi.ptr(weight_min), capi.ptr(output), M, N, K)
    return output


# routed decode GEMVs of a GGUF MoE layer (esimd_moe_up_q4k, esimd_moe_down_q5k / _q6k)
def _chk_moe_gguf(x, sel, n_tokens, top_k, who):
    _chk(x.dtype == torch.float16 and x.is_contiguous(), f"{who}: activations must be contiguous fp16")
    _chk(sel.dtype == torch.int32 and sel.is_contiguous() and sel.numel() >= int(n_tokens) * int(top_k),
         f"{who}: sel must be contiguous int32 [n_tokens * top_k]")
    _chk(int(n_tokens) * int(top_k) <= 65535, f"{who}: at most 65535 routes per call")


def _chk_stack(t, dtype, shape, name, who):
    _chk(t.dtype == dtype and t.is_contiguous() and tuple(t.shape) == tuple(shape),
         f"{who}: {name} must be contiguous {dtype} {list(shape)}, got {t.dtype} {list(t.shape)}")


def esimd_moe_up_q4k(x, gate_ql, gate_sc, gate_mn, up_ql, up_sc, up_mn, sel, inter, n_tokens, hidden, intermediate,
                     top_k):
    """inter[r] = silu(x[t] @ Wg[e]^T) * (x[t] @ Wu[e]^T), r = t * top_k + j, e = sel[r]; Q4_K stacks
    gate_ql / up_ql [E, I, H/2] uint8, scale / min [E, I, H/32] fp16
    (S/csrc/xpu/torch_extension.cc:86-91).  One routed GEMV launch over both matrices, then SiLU * up on
    their fp16 results."""
    who = "esimd_moe_up_q4k"
    T, H, I, k = int(n_tokens), int(hidden), int(intermediate), int(top_k)
    _chk_moe_gguf(x, sel, T, k, who)
    _chk(gate_ql.dim() == 3 and H % 32 == 0, f"{who}: gate_ql must be [E, I, H/2], H a multiple of 32")
    E = gate_ql.shape[0]
    for q, sc, mn, nm in ((gate_ql, gate_sc, gate_mn, "gate"), (up_ql, up_sc, up_mn, "up")):
        _chk_stack(q, torch.uint8, (E, I, H // 2), nm + "_ql", who)
        _chk_stack(sc, torch.float16, (E, I, H // 32), nm + "_sc", who)
        _chk_stack(mn, torch.float16, (E, I, H // 32), nm + "_mn", who)
    P = T * k
    _chk(x.numel() >= T * H and inter.dtype == torch.float16 and inter.is_contiguous() and inter.numel() >= P * I,
         f"{who}: x must be [n_tokens, hidden], inter fp16 [n_tokens * top_k, intermediate]")
    if P == 0:
        return inter
    gu = torch.empty(P, 2 * I, dtype=torch.float16, device=x.device)
    capi.call("mi_moe_gguf_gemv", x, 2, capi.ptr(x), k, 2, capi.ptr_array([gate_ql, up_ql]), None,
              capi.ptr_array([gate_sc, up_sc]), capi.ptr_array([gate_mn, up_mn]), capi.ptr_array([gu, gu[:, I:]]),
              2 * I, capi.ptr(sel), None, P, E, I, H)
    capi.call("mi_moe_silu_mul", gu, capi.ptr(gu), capi.ptr(inter), 2 * I, I, P, capi.DT_F16)
    return inter


def _moe_down_gguf(fmt, inter, ql, qh, sc, mn, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k, who):
    T, H, I, k = int(n_tokens), int(hidden), int(intermediate), int(top_k)
    _chk_moe_gguf(inter, sel, T, k, who)
    _chk(ql.dim() == 3 and I % 32 == 0, f"{who}: ql must be [E, hidden, intermediate/2], intermediate a multiple of 32")
    E = ql.shape[0]
    _chk_stack(ql, torch.uint8, (E, H, I // 2), "ql", who)
    if fmt == 5:
        _chk_stack(qh, torch.uint8, (E, H, I // 8), "qh", who)
        _chk_stack(sc, torch.float16, (E, H, I // 32), "sc", who)
        _chk_stack(mn, torch.float16, (E, H, I // 32), "mn", who)
    else:
        _chk_stack(qh, torch.uint8, (E, H, I // 4), "qh", who)
        _chk_stack(sc, torch.float16, (E, H, I // 16), "sc", who)
    P = T * k
    _chk(inter.numel() >= P * I and topk_w.dtype == torch.float16 and topk_w.is_contiguous() and topk_w.numel() >= P,
         f"{who}: inter must be [n_tokens * top_k, intermediate], topk_w fp16 [n_tokens * top_k]")
    _chk(out_partial.dtype == torch.float16 and out_partial.is_contiguous() and out_partial.numel() >= P * H,
         f"{who}: out_partial must be contiguous fp16 [n_tokens * top_k, hidden]")
    if P == 0:
        return out_partial
    capi.call("mi_moe_gguf_gemv", inter, fmt, capi.ptr(inter), 1, 1, capi.ptr_array([ql]), capi.ptr_array([qh]),
              capi.ptr_array([sc]), capi.ptr_array([mn]) if mn is not None else None, capi.ptr_array([out_partial]),
              H, capi.ptr(sel), capi.ptr(topk_w), P, E, H, I)
    return out_partial


def esimd_moe_down_q5k(inter, ql, qh, sc, mn, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k):
    """out_partial[r] = topk_w[r] * (inter[r] @ Wd[sel[r]]^T) on the Q5_K stack ql [E, H, I/2], qh [E, H, I/8]
    in ELEMENT order (byte j bit b = fifth bit of element 8j + b; not the tile shuffle of the dense GEMV),
    scale / min [E, H, I/32] fp16 (S/csrc/xpu/torch_extension.cc:93-97, moe_kquant_GEMV.h:109-157); I % 32 == 0;
    the caller sums each token's top_k rows."""
    return _moe_down_gguf(5, inter, ql, qh, sc, mn, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k,
                          "esimd_moe_down_q5k")


def esimd_moe_down_q6k(inter, ql, qh, sc, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k):
    """The same on the Q6_K stack ql [E, H, I/2], qh [E, H, I/4] in ELEMENT order (byte j 2-bit field p = top
    bits of element 4j + p), scale [E, H, I/16] fp16 (S/csrc/xpu/torch_extension.cc:98-101,
    moe_kquant_GEMV.h:159-209)."""
    return _moe_down_gguf(6, inter, ql, qh, sc, None, sel, topk_w, out_partial, n_tokens, hidden, intermediate, top_k,
                          "esimd_moe_down_q6k")


# grouped GGUF MoE GEMMs over chunks of expert-sorted rows (the reference's pybind module
# moe_grouped_gguf_xpu: moe_up_q4k_ggemv, moe_down_q5k_ggemv, moe_down_q6k_ggemv)
def _chk_chunks(chunks, who):
    _chk(chunks.dim() == 2 and chunks.size(1) == 3, f"{who}: chunks [num_chunks,3]")
    _chk(chunks.dtype == torch.int32 and chunks.is_contiguous(), f"{who}: chunks must be contiguous int32")


def moe_up_q4k_ggemv(expert_states, gate_ql, gate_sc, gate_mn, up_ql, up_sc, up_mn, gate_buf, chunks, hidden_size,
                     intermediate_size, tok_ids=None, smallm=False):
    """gate_buf[t0 + m, 0:I] = x_m @ Wg[e]^T and gate_buf[t0 + m, I:2I] = x_m @ Wu[e]^T for every chunk
    {e, t0, nt} of `chunks` and m < min(nt, 64) (16 with smallm), where x_m is row tok_ids[t0 + m] of
    `expert_states` (row t0 + m when tok_ids is empty or None).  Q4_K stacks gate_ql / up_ql [E, I, H/2] uint8,
    scale / min [E, I, H/32] fp16; fp16 activations and output; chunks with nt <= 0 are skipped
    (S/csrc/moe_grouped/moe_grouped_entry.sycl:24-60, moe_q4k_ggemv.h:47-201).  Returns gate_buf."""
    who = "moe_up_q4k_ggemv"
    H, I = int(hidden_size), int(intermediate_size)
    _chk_chunks(chunks, who)
    _chk(gate_ql.dim() == 3 and H % 32 == 0, f"{who}: gate_ql must be [E, I, H/2], H a multiple of 32")
    E = gate_ql.shape[0]
    for q, sc, mn, nm in ((gate_ql, gate_sc, gate_mn, "gate"), (up_ql, up_sc, up_mn, "up")):
        _chk_stack(q, torch.uint8, (E, I, H // 2), nm + "_ql", who)
        _chk_stack(sc, torch.float16, (E, I, H // 32), nm + "_sc", who)
        _chk_stack(mn, torch.float16, (E, I, H // 32), nm + "_mn", who)
    _chk(expert_states.dtype == torch.float16 and expert_states.is_contiguous() and expert_states.dim() == 2
         and expert_states.shape[1] == H, f"{who}: expert_states must be contiguous fp16 [rows, hidden]")
    _chk(gate_buf.dtype == torch.float16 and gate_buf.is_contiguous() and gate_buf.dim() == 2
         and gate_buf.shape[1] == 2 * I, f"{who}: gate_buf must be contiguous fp16 [total, 2 * intermediate]")
    total = gate_buf.shape[0]
    has_ids = tok_ids is not None and tok_ids.numel() > 0
    if has_ids:
        _chk(tok_ids.dtype == torch.int32 and tok_ids.is_contiguous() and tok_ids.numel() >= total,
             f"{who}: tok_ids must be contiguous int32 with one entry per row of gate_buf")
    if chunks.size(0) == 0 or total == 0:
        return gate_buf
    capi.call("mi_moe_gguf_grouped", expert_states, 2, capi.ptr(expert_states), expert_states.shape[0],
              capi.ptr(tok_ids) if has_ids else None, 2, capi.ptr_array([gate_ql, up_ql]), None,
              capi.ptr_array([gate_sc, up_sc]), capi.ptr_array([gate_mn, up_mn]), capi.ptr(gate_buf), 2 * I, total,
              capi.ptr(chunks), chunks.size(0), E, I, H, 1 if smallm else 0)
    return gate_buf


def _moe_down_grouped(fmt, intermediate, w_ql, w_qh, w_scale, w_min, expert_output, chunks, intermediate_size,
                      hidden_size, smallm, who):
    I, H = int(intermediate_size), int(hidden_size)
    _chk_chunks(chunks, who)
    _chk(w_ql.dim() == 3 and I % 32 == 0, f"{who}: w_ql must be [E, hidden, intermediate/2], intermediate a multiple of 32")
    E = w_ql.shape[0]
    _chk_stack(w_ql, torch.uint8, (E, H, I // 2), "w_ql", who)
    if fmt == 5:
        _chk_stack(w_qh, torch.uint8, (E, H, I // 8), "w_qh", who)
        _chk_stack(w_scale, torch.float16, (E, H, I // 32), "w_scale", who)
        _chk_stack(w_min, torch.float16, (E, H, I // 32), "w_min", who)
    else:
        _chk_stack(w_qh, torch.uint8, (E, H, I // 4), "w_qh", who)
        _chk_stack(w_scale, torch.float16, (E, H, I // 16), "w_scale", who)
    _chk(intermediate.dtype == torch.float16 and intermediate.is_contiguous() and intermediate.dim() == 2
         and intermediate.shape[1] == I, f"{who}: intermediate must be contiguous fp16 [total, intermediate]")
    _chk(expert_output.dtype == torch.float16 and expert_output.is_contiguous() and expert_output.dim() == 2
         and expert_output.shape[1] == H, f"{who}: expert_output must be contiguous fp16 [total, hidden]")
    total = expert_output.shape[0]
    _chk(intermediate.shape[0] >= total, f"{who}: intermediate has fewer rows than expert_output")
    if chunks.size(0) == 0 or total == 0:
        return expert_output
    capi.call("mi_moe_gguf_grouped", intermediate, fmt, capi.ptr(intermediate), intermediate.shape[0], None, 1,
              capi.ptr_array([w_ql]), capi.ptr_array([w_qh]), capi.ptr_array([w_scale]),
              capi.ptr_array([w_min]) if fmt == 5 else None, capi.ptr(expert_output), H, total, capi.ptr(chunks),
              chunks.size(0), E, H, I, 1 if smallm else 0)
    return expert_output


def moe_down_q5k_ggemv(intermediate, w_ql, w_qh, w_scale, w_min, expert_output, chunks, intermediate_size,
                       hidden_size, smallm=False):
    """expert_output[t0 + m] = intermediate[t0 + m] @ Wd[e]^T for every chunk {e, t0, nt}, m < min(nt, 64)
    (16 with smallm), on the Q5_K stack w_ql [E, H, I/2], w_qh [E, H, I/8] in ELEMENT order (byte j bit b =
    fifth bit of element 8j + b), scale / min [E, H, I/32] fp16
    (S/csrc/moe_grouped/moe_grouped_entry.sycl:62-84, moe_q5k_down_ggemv.h:26-191).  Returns expert_output."""
    return _moe_down_grouped(5, intermediate, w_ql, w_qh, w_scale, w_min, expert_output, chunks, intermediate_size,
                             hidden_size, smallm, "moe_down_q5k_ggemv")


def moe_down_q6k_ggemv(intermediate, w_ql, w_qh, w_scale, expert_output, chunks, intermediate_size, hidden_size,
                       smallm=False):
    """The same on the Q6_K stack w_ql [E, H, I/2], w_qh [E, H, I/4] in ELEMENT order (byte j 2-bit field p =
    top bits of element 4j + p), scale [E, H, I/16] fp16
    (S/csrc/moe_grouped/moe_grouped_entry.sycl:86-106, moe_q6k_down_ggemv.h)."""
    return _moe_down_grouped(6, intermediate, w_ql, w_qh, w_scale, None, expert_output, chunks, intermediate_size,
                             hidden_size, smallm, "moe_down_q6k_ggemv")


def _gemv_q6_k(input, ql, qh, weight_scale, output, who):
    _chk(ql.dtype == torch.uint8 and ql.dim() == 2 and ql.is_contiguous(), f"{who}: ql must be contiguous uint8 [N, K/2]")
    N, K = ql.shape[0], ql.shape[1] * 2
    _chk(K % 512 == 0, f"{who}: K={K} must be a multiple of 512")
    _chk_u8(qh, (N, K // 4), "qh", who)
    _chk_f16(weight_scale, N * (K // 16), "weight_scale [N, K/16]", who)
    M = _chk_gguf_io(input, output, N, K, who)
    capi.call("mi_gemv_q6k", input, capi.ptr(input), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale),
              capi.ptr(output), M, N, K)
    return output


def esimd_gemv_q6_k(input, ql, qh, weight_scale, output):
    """ql [N, K/2], qh [N, K/4] (tile-shuffled top two bits), scale [N, K/16] fp16; w = (v6 - 32) * scale."""
    return _gemv_q6_k(input, ql, qh, weight_scale, output, "esimd_gemv_q6_k")


def esimd_gemv_q6_k_m(input, ql, qh, weight_scale, output):
    return _gemv_q6_k(input, ql, qh, weight_scale, output, "esimd_gemv_q6_k_m")


def _raw_rows(qweight, block_bytes, block_elems, who):
    _chk(qweight.dtype == torch.uint8 and qweight.dim() == 2 and qweight.is_contiguous(),
         f"{who}: qweight must be contiguous uint8 [N, blocks*{block_bytes}]")
    _chk(qweight.shape[1] % block_bytes == 0, f"{who}: row length {qweight.shape[1]} is not a multiple of {block_bytes}")
    return qweight.shape[0], qweight.shape[1] // block_bytes * block_elems


def q4_0_repack(qweight, weight, weight_scale):
    """Raw GGML q4_0 rows [N, K/32*18] -> (weight [N, K/2] interleaved nibbles, scale [N, K/32])."""
    who = "q4_0_repack"
    N, K = _raw_rows(qweight, 18, 32, who)
    _chk_u8(weight, (N, K // 2), "weight", who)
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    capi.call("mi_q4_0_repack", qweight, capi.ptr(qweight), capi.ptr(weight), capi.ptr(weight_scale), N, K)
    return weight


def q8_0_repack(qweight, weight, weight_scale):
    """Raw GGML q8_0 rows [N, K/32*34] -> (weight [N, K] int8, scale [N, K/32])."""
    who = "q8_0_repack"
    N, K = _raw_rows(qweight, 34, 32, who)
    _chk_u8(weight, (N, K), "weight", who, (torch.int8, torch.uint8))
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    capi.call("mi_q8_0_repack", qweight, capi.ptr(qweight), capi.ptr(weight), capi.ptr(weight_scale), N, K)
    return weight


def q5_k_repack(qweight, ql, qh, weight_scale, weight_min):
    """Raw GGML q5_K rows [N, K/256*176] -> (ql, tile-shuffled qh, scale, min)."""
    who = "q5_k_repack"
    N, K = _raw_rows(qweight, 176, 256, who)
    _chk(K % 512 == 0, f"{who}: K={K} must be a multiple of 512")
    _chk_u8(ql, (N, K // 2), "ql", who)
    _chk_u8(qh, (N, K // 8), "qh", who)
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    _chk_f16(weight_min, N * (K // 32), "weight_min", who)
    capi.call("mi_q5k_repack", qweight, capi.ptr(qweight), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale),
              capi.ptr(weight_min), N, K)
    return ql


def q6_k_repack(qweight, ql, qh, weight_scale):
    """Raw GGML q6_K rows [N, K/256*210] -> (ql, tile-shuffled qh, scale [N, K/16])."""
    who = "q6_k_repack"
    N, K = _raw_rows(qweight, 210, 256, who)
    _chk(K % 512 == 0, f"{who}: K={K} must be a multiple of 512")
    _chk_u8(ql, (N, K // 2), "ql", who)
    _chk_u8(qh, (N, K // 4), "qh", who)
    _chk_f16(weight_scale, N * (K // 16), "weight_scale", who)
    capi.call("mi_q6k_repack", qweight, capi.ptr(qweight), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale), N, K)
    return ql


def q5_k_repack_plain(qweight, ql, qh, weight_scale, weight_min):
    """Raw GGML q5_K rows -> (ql, element-order qh [N, K/8]: byte j bit b = element 8j + b, scale, min): the
    representation of the MoE down stacks (sglang_for_multi_arc.patch:2736-2750).  K % 256 == 0."""
    who = "q5_k_repack_plain"
    N, K = _raw_rows(qweight, 176, 256, who)
    _chk_u8(ql, (N, K // 2), "ql", who)
    _chk_u8(qh, (N, K // 8), "qh", who)
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    _chk_f16(weight_min, N * (K // 32), "weight_min", who)
    capi.call("mi_q5k_repack_plain", qweight, capi.ptr(qweight), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale),
              capi.ptr(weight_min), N, K)
    return ql


def q6_k_repack_plain(qweight, ql, qh, weight_scale):
    """Raw GGML q6_K rows -> (ql, element-order qh [N, K/4]: byte j field p = element 4j + p, scale [N, K/16])
    (sglang_for_multi_arc.patch:2753-2765).  K % 256 == 0."""
    who = "q6_k_repack_plain"
    N, K = _raw_rows(qweight, 210, 256, who)
    _chk_u8(ql, (N, K // 2), "ql", who)
    _chk_u8(qh, (N, K // 4), "qh", who)
    _chk_f16(weight_scale, N * (K // 16), "weight_scale", who)
    capi.call("mi_q6k_repack_plain", qweight, capi.ptr(qweight), capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale), N, K)
    return ql


def _chk_dense_out(output, N, K, who):
    _chk(output.dtype == torch.float16 and output.is_contiguous() and output.numel() == N * K,
         f"{who}: output must be contiguous fp16 [N, K]")


def q4_0_dequant(weight, weight_scale, output):
    who = "q4_0_dequant"
    _chk(weight.dtype == torch.uint8 and weight.dim() == 2 and weight.is_contiguous(), f"{who}: weight must be uint8 [N, K/2]")
    N, K = weight.shape[0], weight.shape[1] * 2
    _chk(K % 32 == 0, f"{who}: K must be a multiple of 32")
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    _chk_dense_out(output, N, K, who)
    capi.call("mi_dequant_q4_0", weight, capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(output), N, K)
    return output


def q8_0_dequant(weight, weight_scale, output):
    who = "q8_0_dequant"
    _chk(weight.dtype in (torch.int8, torch.uint8) and weight.dim() == 2 and weight.is_contiguous(),
         f"{who}: weight must be int8 [N, K]")
    N, K = weight.shape
    _chk(K % 32 == 0, f"{who}: K must be a multiple of 32")
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    _chk_dense_out(output, N, K, who)
    capi.call("mi_dequant_q8_0", weight, capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(output), N, K)
    return output


def q5_k_dequant(ql, qh, weight_scale, weight_min, output):
    who = "q5_k_dequant"
    _chk(ql.dtype == torch.uint8 and ql.dim() == 2 and ql.is_contiguous(), f"{who}: ql must be uint8 [N, K/2]")
    N, K = ql.shape[0], ql.shape[1] * 2
    _chk(K % 512 == 0, f"{who}: K must be a multiple of 512")
    _chk_u8(qh, (N, K // 8), "qh", who)
    _chk_f16(weight_scale, N * (K // 32), "weight_scale", who)
    _chk_f16(weight_min, N * (K // 32), "weight_min", who)
    _chk_dense_out(output, N, K, who)
    capi.call("mi_dequant_q5k", ql, capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale), capi.ptr(weight_min),
              capi.ptr(output), N, K)
    return output


def q6_k_dequant(ql, qh, weight_scale, output):
    who = "q6_k_dequant"
    _chk(ql.dtype == torch.uint8 and ql.dim() == 2 and ql.is_contiguous(), f"{who}: ql must be uint8 [N, K/2]")
    N, K = ql.shape[0], ql.shape[1] * 2
    _chk(K % 512 == 0, f"{who}: K must be a multiple of 512")
    _chk_u8(qh, (N, K // 4), "qh", who)
    _chk_f16(weight_scale, N * (K // 16), "weight_scale", who)
    _chk_dense_out(output, N, K, who)
    capi.call("mi_dequant_q6k", ql, capi.ptr(ql), capi.ptr(qh), capi.ptr(weight_scale), capi.ptr(output), N, K)
    return output


def q4_0_quantize(input, out_qweight, out_scale):
    """V/csrc/xpu/torch_extension_q4_0.cc:27-75: [M, K] fp16/bf16 -> int32 [M, K/8] + fp16 scale [M, K/128]."""
    who = "q4_0_quantize"
    _chk(input.dim() == 2, f"{who}: input must be 2D")
    _chk(input.is_contiguous(), f"{who}: input must be contiguous")
    _chk(out_qweight.is_contiguous(), f"{who}: out_qweight must be contiguous")
    _chk(out_scale.is_contiguous(), f"{who}: out_scale must be contiguous")
    _chk(out_qweight.dtype == torch.int32, f"{who}: out_qweight must be int32")
    _chk(out_scale.dtype == torch.float16, f"{who}: out_scale must be float16")
    M, K = input.shape
    _chk(K % 128 == 0, f"{who}: K must be divisible by 128 (got {K})")
    _chk(out_qweight.shape[0] == M, f"{who}: out_qweight row count mismatch")
    _chk(out_qweight.shape[1] == K // 8, f"{who}: out_qweight col count must be K/8")
    _chk(out_scale.shape[0] == M, f"{who}: out_scale row count mismatch")
    _chk(out_scale.shape[1] == K // 128, f"{who}: out_scale col count must be K/128")
    _chk(input.dtype in (torch.float16, torch.bfloat16), f"{who}: input dtype must be bfloat16 or float16 (got {input.dtype})")
    capi.call("mi_q4_0_quantize", input, capi.ptr(input), capi.ptr(out_qweight), capi.ptr(out_scale), M, K,
              capi.act_dtype(input))


# --------------------------------------------------------------------------
# dequant-only siblings
# --------------------------------------------------------------------------
def int4_dequant(weight, weight_scale, weight_zp, output):
    who = "int4_dequant"
    N, K = _int4_nk(weight, who)
    _chk(K % 128 == 0, f"{who}: K must be a multiple of 128")
    _chk(output.dtype in (torch.float16, torch.bfloat16) and output.is_contiguous() and output.numel() == N * K,
         f"{who}: output must be contiguous fp16/bf16 [N, K]")
    _chk(weight_scale.dtype == torch.float16 and weight_scale.numel() == N * K // 128, f"{who}: scale must be fp16 [N, K/128]")
    if weight_zp is not None:
        _chk(weight_zp.dtype == torch.uint8 and weight_zp.numel() == N * K // 128, f"{who}: zp must be uint8 [N, K/128]")
    capi.call("mi_dequant_int4", weight, capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(weight_zp),
              capi.ptr(output), N, K, capi.act_dtype(output))
    return output


def fp8_dequant(weight, weight_scale, output, mode):
    """mode: 'pern' | 'pert' | 'block' -> fp32 [N, K] = e4m3(w) * scale."""
    who = "fp8_dequant"
    _chk_fp8(weight, who)
    _chk(weight.dim() == 2, f"{who}: weight must be [N, K]")
    N, K = weight.shape
    _chk(output.dtype == torch.float32 and output.is_contiguous() and output.numel() == N * K,
         f"{who}: output must be contiguous fp32 [N, K]")
    if mode == "pern":
        _chk(weight_scale.numel() == N and weight_scale.dtype in (torch.float32, torch.float16), f"{who}: scale must be [N]")
        m = 0 if weight_scale.dtype == torch.float32 else 1
    elif mode == "pert":
        _chk(weight_scale.dtype == torch.float32, f"{who}: scale must be fp32")
        m = 2
    elif mode == "block":
        _chk(weight_scale.dtype == torch.float32 and tuple(weight_scale.shape) == ((N + 127) // 128, (K + 127) // 128),
             f"{who}: scale must be fp32 [ceil(N/128), ceil(K/128)]")
        m = 3
    else:
        raise RuntimeError(f"{who}: unknown mode {mode}")
    capi.call("mi_dequant_fp8", weight, capi.ptr(weight), capi.ptr(weight_scale), m, capi.ptr(output), N, K)
    return output


def e4m3_decode(codes, output):
    who = "e4m3_decode"
    _chk(codes.dtype in _FP8_TYPES and codes.is_contiguous(), f"{who}: codes must be contiguous uint8 / float8_e4m3fn")
    _chk(codes.numel() % 8 == 0 and output.numel() == codes.numel(), f"{who}: count must be a multiple of 8")
    _chk(output.dtype in (torch.float16, torch.bfloat16) and output.is_contiguous(), f"{who}: output must be fp16/bf16")
    capi.call("mi_decode_e4m3", codes, capi.ptr(codes), capi.ptr(output), codes.numel(), capi.act_dtype(output))
    return output



# --------------------------------------------------------------------------
# MoE: routing, permutation, grouped GEMM, combine
# --------------------------------------------------------------------------
def esimd_moe_topk(router_logits, top_values, top_indices, T, gate=None):
    """gate (not part of the op's schema) = (x [T, H], gate_weight [H], out fp32 [T]): the same launch also
    writes out[t] = sigmoid(x[t] . gate_weight)."""
    who = "esimd_moe_topk"
    _chk(router_logits.dim() == 2 and router_logits.is_contiguous(), f"{who}: router_logits must be contiguous [T, E]")
    T = int(T)
    _chk(router_logits.shape[0] >= T, f"{who}: T={T} exceeds router_logits rows")
    E = router_logits.shape[1]
    _chk(top_values.dim() == 2 and top_values.dtype == router_logits.dtype and top_values.is_contiguous(),
         f"{who}: top_values must be contiguous [T, K] in the logits dtype")
    K = top_values.shape[1]
    _chk(top_indices.dtype == torch.int32 and top_indices.is_contiguous() and top_indices.numel() >= T * K,
         f"{who}: top_indices must be contiguous int32 [T, K]")
    _chk(E <= 1024 and 1 <= K <= min(64, E), f"{who}: needs E <= 1024 and 1 <= K <= min(64, E)")
    capi.call("mi_moe_topk", router_logits, capi.ptr(router_logits), capi.ptr(top_values),
              capi.ptr(top_indices), T, E, K, 1, None, capi.ptr(gate[0]) if gate else None,
              capi.ptr(gate[1]) if gate else None, capi.ptr(gate[2]) if gate else None,
              gate[0].shape[1] if gate else 0, capi.act_dtype(router_logits))
    return top_values


def moe_topk(logits, top_k, norm, expert_scale=None, gate=None):
    """moe_ops::moe_topk(logits, top_k, norm) -> (weights, ids); outputs are allocated here.
    Not part of the op's schema: expert_scale (fp32 [E]), a factor on the rounded weight of each selected
    expert; gate = (x [T, H], gate_weight [H], out fp32 [T]): the same launch also writes
    out[t] = sigmoid(x[t] . gate_weight)."""
    _chk(logits.dim() == 2 and logits.is_contiguous(), "moe_topk: logits must be contiguous [T, E]")
    T, E = logits.shape
    w = torch.empty(T, int(top_k), dtype=logits.dtype, device=logits.device)
    ids = torch.empty(T, int(top_k), dtype=torch.int32, device=logits.device)
    _chk(E <= 1024 and 1 <= int(top_k) <= min(64, E), "moe_topk: needs E <= 1024 and 1 <= top_k <= min(64, E)")
    gx, gw, go = gate if gate is not None else (None, None, None)
    capi.call("mi_moe_topk", logits, capi.ptr(logits), capi.ptr(w), capi.ptr(ids), T, E, int(top_k),
              1 if norm else 0, capi.ptr(expert_scale), capi.ptr(gx), capi.ptr(gw), capi.ptr(go),
              gx.shape[1] if gx is not None else 0, capi.act_dtype(logits))
    return w, ids


def topk_v2(router_logits, top_values, top_indices, T, num_experts, topk):
    """esimd_topk_v2::topk_v2: esimd_moe_topk with the expert and route counts passed explicitly
    (V/csrc/xpu/torch_extension_topk_v2.cc:12-16)."""
    who = "topk_v2"
    _chk(router_logits.dim() == 2 and router_logits.shape[1] == int(num_experts), f"{who}: router_logits must be [T, num_experts]")
    _chk(top_values.dim() == 2 and top_values.shape[1] == int(topk), f"{who}: top_values must be [T, topk]")
    return esimd_moe_topk(router_logits, top_values, top_indices, T)


def moe_router_forward(x, weight, scale):
    """logits[T, E] = x[T, H] @ (scale[0] * e4m3(weight[E, H]))^T in x's dtype
    (V/csrc/moe_batch/moe.sycl:302-358); runs on the per-tensor FP8 GEMV / small-batch GEMM."""
    who = "moe_router_forward"
    _chk(x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.float16, torch.bfloat16), f"{who}: x must be contiguous fp16 [T, H]")
    _chk(scale.dtype == torch.float32 and scale.numel() >= 1, f"{who}: scale must be float32")
    _chk_fp8(weight, who)
    _chk(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.is_contiguous(), f"{who}: weight must be [num_experts, hidden]")
    out = torch.empty(x.shape[0], weight.shape[0], dtype=x.dtype, device=x.device)
    return esimd_gemm_fp8_pert(x, weight, scale.reshape(-1)[:1], out)


def moe_accumulate(partials, top_k, num_shared_experts):
    """out[t] = sum of the top_k + num_shared_experts consecutive rows of token t, added in fp32 and
    rounded once (V/csrc/moe_batch/moe.sycl:1177-1230)."""
    who = "moe_accumulate"
    _chk(partials.dim() == 2 and partials.is_contiguous() and partials.dtype in (torch.float16, torch.bfloat16),
         f"{who}: partials must be contiguous fp16 [T * rows_per_token, H]")
    rows = int(top_k) + int(num_shared_experts)
    _chk(rows >= 1 and partials.shape[0] % rows == 0, f"{who}: the row count must be a multiple of top_k + num_shared_experts")
    H = partials.shape[1]
    _chk(H % 8 == 0, f"{who}: hidden size must be a multiple of 8")
    T = partials.shape[0] // rows
    out = torch.empty(T, H, dtype=partials.dtype, device=partials.device)
    if T == 0:
        return out
    capi.call("mi_moe_combine", partials, capi.ptr(partials), None, None, capi.ptr(out), H, rows, T, 0,
              capi.act_dtype(partials), 0)
    return out


def moe_sort(top_ids, num_experts, sorted_pairs, expert_start, inv, sorted_token=None, max_count=None):
    """Stable expert sort of the flattened (token, route) pairs; all outputs int32, written in place."""
    who = "moe_sort"
    _chk(top_ids.dim() == 2 and top_ids.dtype == torch.int32 and top_ids.is_contiguous(),
         f"{who}: top_ids must be contiguous int32 [T, K]")
    T, K = top_ids.shape
    E = int(num_experts)
    _chk(1 <= E <= 1024, f"{who}: num_experts must be in 1..1024")
    for t, n, nm in ((sorted_pairs, T * K, "sorted_pairs"), (expert_start, E + 1, "expert_start"), (inv, T * K, "inv")):
        _chk(t.dtype in (torch.int32, torch.uint32) and t.is_contiguous() and t.numel() >= n,
             f"{who}: {nm} must be contiguous int32 with >= {n} entries")
    if sorted_token is not None:
        _chk(sorted_token.dtype == torch.int32 and sorted_token.numel() >= T * K, f"{who}: sorted_token must be int32 [T*K]")
    if max_count is not None:
        _chk(max_count.dtype == torch.int32 and max_count.numel() >= 1, f"{who}: max_count must be int32 [1]")
    capi.call("mi_moe_sort", top_ids, capi.ptr(top_ids), capi.ptr(sorted_pairs), capi.ptr(expert_start),
              capi.ptr(inv), capi.ptr(sorted_token), capi.ptr(max_count), T, K, E)
    return sorted_pairs


def act_quant_fp8(x, q, scale):
    who = "act_quant_fp8"
    _chk(x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.float16, torch.bfloat16), f"{who}: x must be contiguous fp16/bf16 [rows, K]")
    rows, K = x.shape
    _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
    _chk(q.dtype in _FP8_TYPES and q.is_contiguous() and q.numel() == rows * K, f"{who}: q must be e4m3/uint8 [rows, K]")
    _chk(scale.dtype == torch.float32 and scale.is_contiguous() and scale.numel() == rows * (K // 128),
         f"{who}: scale must be fp32 [rows, K/128]")
    capi.call("mi_act_quant_fp8", x, capi.ptr(x), capi.ptr(q), capi.ptr(scale), rows, K, capi.act_dtype(x))
    return q


def _act_mul(input, output, N_gate_up, N_half, total_rows, entry, who):
    _chk_act(input, output, who)
    _chk(int(N_gate_up) == 2 * int(N_half), f"{who}: N_gate_up must be 2 * N_half")
    _chk(input.numel() >= int(total_rows) * int(N_gate_up) and output.numel() >= int(total_rows) * int(N_half),
         f"{who}: tensors too small for total_rows")
    capi.call(entry, input, capi.ptr(input), capi.ptr(output), int(N_gate_up), int(N_half),
              int(total_rows), capi.act_dtype(input))
    return output


def esimd_moe_silu_mul(input, output, N_gate_up, N_half, total_rows):
    return _act_mul(input, output, N_gate_up, N_half, total_rows, "mi_moe_silu_mul", "esimd_moe_silu_mul")


def esimd_moe_gelu_tanh_mul(input, output, N_gate_up, N_half, total_rows):
    """GELU_tanh(gate) * up (V/csrc/xpu/esimd_kernels/moe_ops.h:680-728)."""
    return _act_mul(input, output, N_gate_up, N_half, total_rows, "mi_moe_gelu_tanh_mul", "esimd_moe_gelu_tanh_mul")


def esimd_moe_scatter(hidden_states, router_top_value, sorted_token_ids, scattered_hidden, scattered_weights,
                      K, topk, total_expanded):
    who = "esimd_moe_scatter"
    _chk_act(hidden_states, scattered_hidden, who)
    _chk(int(K) % 8 == 0, f"{who}: K must be a multiple of 8")
    _chk(sorted_token_ids.dtype == torch.int32 and sorted_token_ids.numel() >= int(total_expanded), f"{who}: sorted_token_ids must be int32")
    _chk(router_top_value.dtype == hidden_states.dtype and scattered_weights.dtype == hidden_states.dtype,
         f"{who}: weights must share the activation dtype")
    capi.call("mi_moe_scatter", hidden_states, capi.ptr(hidden_states), capi.ptr(router_top_value),
              capi.ptr(sorted_token_ids), capi.ptr(scattered_hidden), capi.ptr(scattered_weights), int(K),
              int(topk), int(total_expanded))
    return scattered_hidden


def esimd_moe_scatter_fused(hidden_states, top_values, top_indices, scattered_hidden, scattered_weights,
                            topk_ids, expert_start, max_tokens_out, K, topk, T, num_experts):
    """Device-side expert sort + row scatter.  topk_ids receives the reverse map
    (pair -> scattered row), expert_start the E+1 start offsets."""
    who = "esimd_moe_scatter_fused"
    T, topk, K, E = int(T), int(topk), int(K), int(num_experts)
    _chk_act(hidden_states, scattered_hidden, who)
    _chk(top_indices.dtype == torch.int32 and top_indices.is_contiguous() and top_indices.numel() >= T * topk,
         f"{who}: top_indices must be contiguous int32 [T, topk]")
    _chk(expert_start.dtype in (torch.int32, torch.uint32) and expert_start.numel() >= E + 1,
         f"{who}: expert_start must be int32/uint32 [num_experts+1]")
    _chk(topk_ids.dtype == torch.int32 and topk_ids.numel() >= T * topk, f"{who}: topk_ids must be int32 [T*topk]")
    sorted_pairs = torch.empty(T * topk, dtype=torch.int32, device=hidden_states.device)
    ids2d = top_indices.reshape(-1)[:T * topk].reshape(T, topk)
    moe_sort(ids2d, E, sorted_pairs, expert_start, topk_ids, None, max_tokens_out)
    esimd_moe_scatter(hidden_states, top_values, sorted_pairs, scattered_hidden, scattered_weights, K, topk, T * topk)
    return scattered_hidden


def esimd_moe_gather(moe_output, topk_ids, scattered_weights, final_hidden, K, topk, T):
    who = "esimd_moe_gather"
    _chk_act(moe_output, final_hidden, who)
    _chk(int(K) % 8 == 0, f"{who}: K must be a multiple of 8")
    _chk(topk_ids.dtype == torch.int32 and topk_ids.numel() >= int(T) * int(topk), f"{who}: topk_ids must be int32 [T, topk]")
    _chk(scattered_weights.dtype == moe_output.dtype, f"{who}: scattered_weights must share the activation dtype")
    capi.call("mi_moe_combine", moe_output, capi.ptr(moe_output), capi.ptr(topk_ids), capi.ptr(scattered_weights),
              capi.ptr(final_hidden), int(K), int(topk), int(T), 1, capi.act_dtype(moe_output), 0)
    return final_hidden


_ACT_NONE, _ACT_SILU, _ACT_GELU_TANH = 0, 1, 2


def _out_kind(out, adt):
    """The library's code for the element type of expert outputs: 0 the activation type, 1 fp32,
    2 fp16 beside bf16 activations (three more mantissa bits than bf16 at half the bytes of fp32)."""
    if out.dtype == torch.float32:
        return 1
    return 2 if (out.dtype == torch.float16 and adt == capi.DT_BF16) else 0


def _moe_tiled_workspace(w8a16, out16, total, E, K):
    """Workspace bytes of the tiled (prefill) grouped GEMM when that route takes the launch, else None:
    16-bit activations and output, whole 128-granules, at most 1024 experts averaging 96 rows or more,
    and re-tiled activations below 2 GiB (the library's own limits, asked of the library so the two
    cannot drift; past them the streaming grouped kernel runs)."""
    if not (w8a16 and out16 and K % 128 == 0 and E <= 1024 and total >= 96 * E):
        return None
    need = ctypes.c_longlong(0)
    if capi.lib().mi_moe_gemm_fp8_tiled_workspace(int(total), int(E), int(K), ctypes.byref(need)) != 0:
        return None
    return need.value


def _moe_gemm(a, a_scale, row_map, w, w_scale, expert_start, out, E, N, K, fuse, who, *, per_expert=False,
              out_map=None, row_weight=None, row_map_div=1):
    """Grouped GEMM over expert-sorted rows.  fuse: False / True (SiLU) or one of _ACT_*.
    per_expert: w_scale holds one fp32 per expert (True / 1), or two — rows [0, N/2) and [N/2, N) —
    (2), instead of 128x128 block scales.
    out_map (int32): sorted position -> row of `out`; row_weight (activation dtype): factor
    per row of `out`; the source row of a position is row_map[position] // row_map_div."""
    _chk_fp8(w, who)
    _chk(w.numel() == E * N * K, f"{who}: weight must be [num_experts, N, K]")
    fuse = int(fuse)
    per_expert = int(per_expert)
    if per_expert:
        _chk(K % 16 == 0, f"{who}: K={K} must be a multiple of 16")
        _chk(w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() >= E * per_expert,
             f"{who}: weight_scale must be contiguous fp32 [E]" + (" x 2" if per_expert == 2 else ""))
        _chk(per_expert == 1 or (N % 2 == 0 and (fuse or (N // 2) % 16 == 0)),
             f"{who}: with gate / up scales N/2 must be a multiple of 16")
    else:
        _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
        _chk(not fuse or (N // 2) % 16 == 0, f"{who}: with block scales and the fused gate * up epilogue N/2 must be a multiple of 16")
        _chk(w_scale.dtype == torch.float32 and w_scale.is_contiguous() and
             w_scale.numel() == E * ((N + 127) // 128) * (K // 128),
             f"{who}: weight_scale must be contiguous fp32 [E, ceil(N/128), K/128]")
    _chk(expert_start.dtype in (torch.int32, torch.uint32) and expert_start.numel() >= E + 1,
         f"{who}: expert_idx must be int32/uint32 [num_experts+1]")
    _chk(out.dtype in (torch.float16, torch.bfloat16, torch.float32) and out.is_contiguous(),
         f"{who}: output must be contiguous fp16/bf16/fp32")
    n_out = N // 2 if fuse else N
    total = out.numel() // n_out
    a_rows = a.numel() // K
    if a_scale is None:
        adt = capi.act_dtype(a)
        _chk(out.dtype in (a.dtype, torch.float32, torch.float16), f"{who}: output must be fp32, fp16 or share the activation dtype")
    else:
        adt = capi.act_dtype(out) if out.dtype != torch.float32 else capi.DT_BF16
    if out_map is not None:
        _chk(out_map.dtype == torch.int32 and out_map.is_contiguous(), f"{who}: the output row map must be int32")
    if row_weight is not None:
        _chk(out.dtype != torch.float32 and row_weight.dtype == out.dtype and row_weight.is_contiguous() and
             row_weight.numel() >= total, f"{who}: row weights must share the output dtype, one per output row")
    need = _moe_tiled_workspace(a_scale is None, _out_kind(out, adt) == 0, total, E, K)
    if need is not None:
        # prefill: the tiled matrix-core GEMM, workspace from the caching allocator (graph-capturable)
        buf = torch.empty(need, dtype=torch.uint8, device=out.device)
        capi.call("mi_moe_gemm_fp8_tiled_ws", out, capi.ptr(a), capi.ptr(row_map), int(row_map_div), capi.ptr(w),
                  capi.ptr(w_scale), per_expert, capi.ptr(expert_start), capi.ptr(out), capi.ptr(out_map), capi.ptr(row_weight),
                  a_rows, total, E, N, K, fuse, adt, capi.ptr(buf), need)
        return out
    capi.call("mi_moe_gemm_fp8_grouped", out, capi.ptr(a), capi.ptr(a_scale), capi.ptr(row_map), int(row_map_div),
              capi.ptr(w), capi.ptr(w_scale), per_expert, capi.ptr(expert_start), capi.ptr(out), capi.ptr(out_map),
              capi.ptr(row_weight), a_rows, total, E, N, K, fuse, adt, _out_kind(out, adt))
    return out


def _moe_mlp_tiled(x, row_map, w13, s13, w2, s2, expert_start, y, total, E, H, I):
    """gate_up, SiLU * up and down of the w8a16 prefill regime as one library call (block scales);
    False when the tiled route does not take the shape (the caller then runs the two GEMMs)."""
    for w, s, n, kk in ((w13, s13, 2 * I, H), (w2, s2, H, I)):
        _chk_fp8(w, "moe_forward_fp8_block")
        _chk(s.dtype == torch.float32 and s.is_contiguous() and s.numel() == E * ((n + 127) // 128) * (kk // 128),
             "moe_forward_fp8_block: weight scales must be contiguous fp32 [E, ceil(N/128), K/128]")
    if not (H % 128 == 0 and I % 128 == 0 and E <= 1024 and y.dtype == x.dtype):
        return False
    need = ctypes.c_longlong(0)
    if capi.lib().mi_moe_mlp_fp8_tiled_workspace(int(total), int(E), int(H), int(I), ctypes.byref(need)) != 0:
        return False
    buf = torch.empty(need.value, dtype=torch.uint8, device=y.device)
    capi.call("mi_moe_mlp_fp8_tiled_ws", y, capi.ptr(x), capi.ptr(row_map), 1, capi.ptr(w13), capi.ptr(s13),
              capi.ptr(w2), capi.ptr(s2), 0, capi.ptr(expert_start), capi.ptr(y), None, None, x.shape[0], int(total),
              int(E), int(H), int(I), 1, capi.act_dtype(x), capi.ptr(buf), need.value)
    return True


def esimd_moe_gemm_fp8_blockscale(input, weight, weight_scale, output, expert_idx, N, K, num_experts,
                                  block_n, block_k):
    who = "esimd_moe_gemm_fp8_blockscale"
    _chk(int(block_n) == 128 and int(block_k) == 128, f"{who}: only block_n == block_k == 128 is supported")
    _chk_act(input, output, who)
    N, K, E = int(N), int(K), int(num_experts)
    _chk(input.numel() % K == 0 and output.numel() == (input.numel() // K) * N, f"{who}: output must be [total_tokens, N]")
    return _moe_gemm(input, None, None, weight, weight_scale, expert_idx, output, E, N, K, False, who)


def moe_gemm_fp8_block(a, a_scale, row_map, weight, weight_scale, expert_start, output, N, K, num_experts,
                       fuse_silu_mul):
    """Grouped block-FP8 GEMM.  a_scale given: `a` is e4m3 with per-row per-128 fp32 scales
    (native fp8 MFMA); a_scale None: `a` is fp16/bf16 (w8a16).  row_map (int32, optional)
    gathers source rows; fuse_silu_mul writes silu(gate) * up ([rows, N/2]); output may be fp32."""
    who = "moe_gemm_fp8_block"
    K = int(K)
    if a_scale is not None:
        _chk(a.dtype in _FP8_TYPES and a.is_contiguous(), f"{who}: quantised activations must be contiguous e4m3/uint8")
        _chk(a_scale.dtype == torch.float32 and a_scale.is_contiguous() and a_scale.numel() == (a.numel() // K) * (K // 128),
             f"{who}: a_scale must be fp32 [rows, K/128]")
    else:
        _chk(a.dtype in (torch.float16, torch.bfloat16) and a.is_contiguous(), f"{who}: activations must be contiguous fp16/bf16")
    if row_map is not None:
        _chk(row_map.dtype == torch.int32 and row_map.is_contiguous(), f"{who}: row_map must be int32")
    return _moe_gemm(a, a_scale, row_map, weight, weight_scale, expert_start, output, int(num_experts), int(N),
                     K, bool(fuse_silu_mul), who)


ROUTED_MAX_PAIRS = 8192       # (token, route) pairs one routed gate_up launch sorts by itself
ROUTED_GEMV_MAX_PAIRS = 96    # (token, route) pairs up to which the fused decode op runs one GEMV per route (12 tokens x top 8)


def moe_gate_up_fp8_routed(xq, xs, top_ids, weight, weight_scale, expert_start, inv, sorted_pairs, output,
                           num_experts):
    """Expert sort and the gate_up grouped GEMM (quantised activations, fused silu(gate) * up) in one
    launch.  xq [T, K] e4m3 with xs [T, K/128] fp32; top_ids [T, topk] int32; weight [E, N, K] e4m3
    with block scales; output [T*topk, N/2] fp16/bf16 in expert-sorted order.  expert_start [E+1],
    inv [T*topk] and (optional) sorted_pairs [T*topk] are written as moe_sort writes them."""
    who = "moe_gate_up_fp8_routed"
    E = int(num_experts)
    _chk(top_ids.dim() == 2 and top_ids.dtype == torch.int32 and top_ids.is_contiguous(),
         f"{who}: top_ids must be contiguous int32 [T, topk]")
    T, k = top_ids.shape
    P = T * k
    _chk(0 < P <= ROUTED_MAX_PAIRS, f"{who}: {P} pairs (1..{ROUTED_MAX_PAIRS} are sorted inside the launch)")
    _chk(xq.dim() == 2 and xq.shape[0] == T and xq.dtype in _FP8_TYPES and xq.is_contiguous(),
         f"{who}: quantised activations must be contiguous e4m3/uint8 [T, K]")
    K = xq.shape[1]
    _chk(K % 128 == 0 and K >= 256, f"{who}: K={K} must be a multiple of 128, at least 256")
    _chk(xs.dtype == torch.float32 and xs.is_contiguous() and xs.numel() == T * (K // 128),
         f"{who}: activation scales must be fp32 [T, K/128]")
    _chk_fp8(weight, who)
    _chk(weight.dim() == 3 and weight.shape[0] == E and weight.shape[2] == K and weight.is_contiguous(),
         f"{who}: weight must be contiguous [E, N, K]")
    N = weight.shape[1]
    _chk(N % 2 == 0 and (N // 2) % 16 == 0, f"{who}: N/2 must be a multiple of 16")
    _chk(weight_scale.dtype == torch.float32 and weight_scale.is_contiguous() and
         weight_scale.numel() == E * ((N + 127) // 128) * (K // 128),
         f"{who}: weight_scale must be contiguous fp32 [E, ceil(N/128), K/128]")
    _chk(1 <= E <= 1024, f"{who}: num_experts must be in 1..1024")
    for t, n, nm in ((expert_start, E + 1, "expert_start"), (inv, P, "inv")) + \
            (((sorted_pairs, P, "sorted_pairs"),) if sorted_pairs is not None else ()):
        _chk(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n,
             f"{who}: {nm} must be contiguous int32 with >= {n} entries")
    _chk(output.dtype in (torch.float16, torch.bfloat16) and output.is_contiguous() and
         output.numel() == P * (N // 2), f"{who}: output must be contiguous fp16/bf16 [T*topk, N/2]")
    for t in (xs, top_ids, weight, weight_scale, expert_start, inv, output):
        _chk(t.device == xq.device, f"{who}: all tensors must be on one device")
    capi.call("mi_moe_gate_up_fp8_routed", output, capi.ptr(xq), capi.ptr(xs), capi.ptr(top_ids), T, k,
              capi.ptr(weight), capi.ptr(weight_scale), capi.ptr(expert_start), capi.ptr(inv),
              capi.ptr(sorted_pairs), capi.ptr(output), E, N, K, capi.act_dtype(output))
    return output


def moe_forward_fp8_block(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale, output, top_k,
                          act_quant):
    """Routed-experts MoE forward for 128x128 block-FP8 weights (no shared expert).

    x [T, H], logits [T, E] fp16/bf16; gate_up_weight [E, 2I, H], down_weight [E, H, I]
    e4m3 with fp32 block scales [E, 2I/128, H/128] / [E, H/128, I/128]; output [T, H].
    act_quant=True quantises the activations entering both GEMMs per token per
    128-group to e4m3 (native fp8 MFMA); False keeps them 16 bit (w8a16).
    Pipeline: top-k -> stable expert sort -> [quantise x] -> grouped gate_up GEMM
    with fused SiLU*mul -> [quantise] -> grouped down GEMM -> weighted combine.
    """
    who = "moe_forward_fp8_block"
    _chk(x.dim() == 2 and logits.dim() == 2 and x.shape[0] == logits.shape[0], f"{who}: x [T,H], logits [T,E]")
    _chk_act(x, output, who)
    _chk(logits.dtype == x.dtype and logits.is_contiguous(), f"{who}: logits must share x's dtype")
    _chk(output.data_ptr() != x.data_ptr(), f"{who}: output must not alias x")
    T, H = x.shape
    E = logits.shape[1]
    _chk(gate_up_weight.dim() == 3 and down_weight.dim() == 3, f"{who}: weights must be [E, N, K]")
    I = down_weight.shape[2]
    _chk(tuple(gate_up_weight.shape) == (E, 2 * I, H) and tuple(down_weight.shape) == (E, H, I),
         f"{who}: expected gate_up [E, 2I, H] and down [E, H, I]")
    _chk(H % 128 == 0 and I % 128 == 0, f"{who}: H and I must be multiples of 128")
    k = int(top_k)
    P = T * k
    dev = x.device
    top_w = torch.empty(T, k, dtype=x.dtype, device=dev)
    top_ids = torch.empty(T, k, dtype=torch.int32, device=dev)
    if act_quant:
        # the routing and the quantisation of x do not depend on each other: one launch
        _chk(E <= 1024 and 0 < k <= min(E, 64), f"{who}: top_k={k} of {E} experts is not supported")
        xq = torch.empty(T, H, dtype=torch.uint8, device=dev)
        xs = torch.empty(T, H // 128, dtype=torch.float32, device=dev)
        capi.call("mi_moe_topk_quant", logits, capi.ptr(logits), capi.ptr(top_w), capi.ptr(top_ids), T, E, k, 1,
                  capi.ptr(x), capi.ptr(xq), capi.ptr(xs), H, capi.act_dtype(x))
    else:
        esimd_moe_topk(logits, top_w, top_ids, T)
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    # fp32 expert outputs (the combine adds K rounded terms otherwise); in the w8a16 prefill regime the
    # tiled grouped GEMM takes over, which writes the activation type
    prefill = (not act_quant) and P >= 96 * E
    y = torch.empty(P, H, dtype=x.dtype if prefill else torch.float32, device=dev)
    routed = act_quant and 0 < P <= ROUTED_MAX_PAIRS and H >= 256
    if not routed:
        sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
        sorted_token = torch.empty(P, dtype=torch.int32, device=dev)
        moe_sort(top_ids, E, sorted_pairs, start, inv, sorted_token, None)
    if act_quant:
        inter = torch.empty(P, I, dtype=x.dtype, device=dev)
        if routed:      # the gate_up launch sorts the pairs itself
            moe_gate_up_fp8_routed(xq, xs, top_ids, gate_up_weight, gate_up_scale, start, inv, None, inter, E)
        else:
            moe_gemm_fp8_block(xq, xs, sorted_token, gate_up_weight, gate_up_scale, start, inter, 2 * I, H, E, True)
        iq = torch.empty(P, I, dtype=torch.uint8, device=dev)
        isc = torch.empty(P, I // 128, dtype=torch.float32, device=dev)
        act_quant_fp8(inter, iq, isc)
        moe_gemm_fp8_block(iq, isc, None, down_weight, down_scale, start, y, H, I, E, False)
    elif prefill and _moe_mlp_tiled(x, sorted_token, gate_up_weight, gate_up_scale, down_weight, down_scale, start, y,
                                    P, E, H, I):
        pass            # both GEMMs in one call: the intermediate stays in the second GEMM's operand order
    else:
        inter = torch.empty(P, I, dtype=x.dtype, device=dev)
        moe_gemm_fp8_block(x, None, sorted_token, gate_up_weight, gate_up_scale, start, inter, 2 * I, H, E, True)
        moe_gemm_fp8_block(inter, None, None, down_weight, down_scale, start, y, H, I, E, False)
    moe_combine(y, inv, top_w, output, k)
    return output


def moe_forward_full_fp8_block(x, logits, output, gate_up_weight, gate_up_scale, shared_gate_up_weight,
                               shared_gate_up_scale, down_weight, down_scale, shared_down_weight,
                               shared_down_scale, shared_expert_gate_weight, top_k, num_shared_experts,
                               n_routed_experts):
    """Small-batch fused MoE decode step for 128x128 block-FP8 weights, w8a16:
    softmax top-k (renormalised) -> routed experts (gate_up, SiLU*mul, down) weighted sum
    + sigmoid(x . shared_expert_gate_weight) * shared expert.  Same arguments and checks as
    the reference op (V/csrc/moe_batch/moe.sycl:1707-1853); bf16 is accepted besides fp16
    and the 12-token limit is lifted (more tokens simply run the grouped kernels)."""
    who = "moe_forward_full_fp8_block"
    _chk(x.dim() == 2 and x.shape[0] >= 1, f"{who}: x must be [T, H] with T >= 1")
    _chk_act(x, output, who)
    _chk(tuple(output.shape) == tuple(x.shape), f"{who}: output must have x's shape")
    _chk(output.data_ptr() != x.data_ptr(), f"{who} output must not alias x")
    _chk(int(num_shared_experts) == 1, f"{who} requires one shared expert")
    E, k = int(n_routed_experts), int(top_k)
    _chk(E > 0 and 0 < k <= E, f"{who} requires 0 < top_k <= n_routed_experts")
    T, H = x.shape
    _chk(logits.dim() == 2 and tuple(logits.shape) == (T, E) and logits.dtype == x.dtype, f"{who}: logits must be [T, E] in x's dtype")
    for name, w in (("gate_up_weight", gate_up_weight), ("down_weight", down_weight),
                    ("shared_gate_up_weight", shared_gate_up_weight), ("shared_down_weight", shared_down_weight)):
        _chk(w.dtype in (torch.float8_e4m3fn, torch.uint8), f"{who} requires e4m3 weights ({name} is {w.dtype})")
    for name, t in (("gate_up_scale", gate_up_scale), ("down_scale", down_scale),
                    ("shared_gate_up_scale", shared_gate_up_scale), ("shared_down_scale", shared_down_scale)):
        _chk(t.dtype == torch.float32, f"{who}: {name} must be fp32")
    _chk(gate_up_weight.dim() == 3 and gate_up_weight.shape[0] == E and gate_up_weight.shape[2] == H and
         gate_up_weight.shape[1] % 2 == 0, f"{who}: gate_up_weight must be [E, 2I, H]")
    I = gate_up_weight.shape[1] // 2
    _chk(H % 128 == 0 and I % 128 == 0, f"{who}: hidden and intermediate sizes must be multiples of 128")
    _chk(tuple(down_weight.shape) == (E, H, I), f"{who}: down_weight must be [E, H, I]")
    _chk(tuple(shared_gate_up_weight.shape) == (2 * I, H) and tuple(shared_down_weight.shape) == (H, I),
         f"{who}: shared weights must be [2I, H] and [H, I]")
    _chk(tuple(gate_up_scale.shape) == (E, 2 * I // 128, H // 128) and tuple(down_scale.shape) == (E, H // 128, I // 128),
         f"{who}: routed scales must be [E, 2I/128, H/128] and [E, H/128, I/128]")
    _chk(tuple(shared_gate_up_scale.shape) == (2 * I // 128, H // 128) and
         tuple(shared_down_scale.shape) == (H // 128, I // 128), f"{who}: shared scales must be [2I/128, H/128] and [H/128, I/128]")
    _chk(tuple(shared_expert_gate_weight.shape) == (1, H) and shared_expert_gate_weight.dtype == x.dtype,
         f"{who}: shared_expert_gate_weight must be [1, H] in x's dtype")
    for name, t in (("logits", logits), ("output", output), ("gate_up_weight", gate_up_weight),
                    ("gate_up_scale", gate_up_scale), ("shared_gate_up_weight", shared_gate_up_weight),
                    ("shared_gate_up_scale", shared_gate_up_scale), ("down_weight", down_weight),
                    ("down_scale", down_scale), ("shared_down_weight", shared_down_weight),
                    ("shared_down_scale", shared_down_scale), ("shared_expert_gate_weight", shared_expert_gate_weight)):
        _chk(t.device == x.device, f"{who}: {name} must be on the same device as x")
        _chk(t.is_contiguous(), f"{who}: {name} must be contiguous")
    dev = x.device
    P = T * k
    # routing and routed experts (w8a16 grouped GEMMs on the expert-sorted pairs)
    top_w = torch.empty(T, k, dtype=x.dtype, device=dev)
    top_ids = torch.empty(T, k, dtype=torch.int32, device=dev)
    gate = torch.empty(T, dtype=torch.float32, device=dev)
    # routing and the shared expert's gate sigmoid(x . w) in one launch
    esimd_moe_topk(logits, top_w, top_ids, T, gate=(x, shared_expert_gate_weight, gate))
    if P <= ROUTED_GEMV_MAX_PAIRS:
        # Decode: one GEMV per (token, route), all routes in one launch per projection (no sort, no
        # grouping: with a handful of rows a grouped launch has work for a few workgroups only and
        # streams each expert's weights at a fraction of the device's rate).  The shared expert's rows
        # follow the routed ones in the same launches and buffers: four launches in all.
        adt = capi.act_dtype(x)
        gu = torch.empty(P + T, 2 * I, dtype=x.dtype, device=dev)
        capi.call("mi_moe_gemv_fp8_block_routed", x, capi.ptr(x), k, 0, capi.ptr(gate_up_weight), capi.ptr(gate_up_scale),
                  capi.ptr(gu), 2 * I, capi.ptr(top_ids), None, P, E, capi.ptr(shared_gate_up_weight),
                  capi.ptr(shared_gate_up_scale), T, 0, 2 * I, H, adt)
        # down projections: SiLU(gate) * up is applied while a row is staged; the routing weight
        # multiplies each route's row before it is rounded, so the sum over routes is plain
        y = torch.empty(P + T, H, dtype=x.dtype, device=dev)
        capi.call("mi_moe_gemv_fp8_block_routed", gu, capi.ptr(gu), 1, 1, capi.ptr(down_weight), capi.ptr(down_scale),
                  capi.ptr(y), H, capi.ptr(top_ids), capi.ptr(top_w), P, E, capi.ptr(shared_down_weight),
                  capi.ptr(shared_down_scale), T, P, H, I, adt)
        capi.call("mi_moe_combine_shared", y, capi.ptr(y), None, None, capi.ptr(output), capi.ptr(y[P:]),
                  capi.ptr(gate), H, k, T, 0, adt, 0)
        return output
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    sorted_token = torch.empty(P, dtype=torch.int32, device=dev)
    moe_sort(top_ids, E, sorted_pairs, start, inv, sorted_token, None)
    inter = torch.empty(P, I, dtype=x.dtype, device=dev)
    y = torch.empty(P, H, dtype=torch.float32, device=dev)
    moe_gemm_fp8_block(x, None, sorted_token, gate_up_weight, gate_up_scale, start, inter, 2 * I, H, E, True)
    moe_gemm_fp8_block(inter, None, None, down_weight, down_scale, start, y, H, I, E, False)
    # shared expert: dense block-scaled GEMMs on all tokens
    sh_gu = torch.empty(T, 2 * I, dtype=x.dtype, device=dev)
    esimd_gemm_fp8_blockscale(x, shared_gate_up_weight, shared_gate_up_scale, sh_gu, 128, 128)
    sh_inter = torch.empty(T, I, dtype=x.dtype, device=dev)
    esimd_moe_silu_mul(sh_gu, sh_inter, 2 * I, I, T)
    sh_out = torch.empty(T, H, dtype=x.dtype, device=dev)
    esimd_gemm_fp8_blockscale(sh_inter, shared_down_weight, shared_down_scale, sh_out, 128, 128)
    capi.call("mi_moe_combine_shared", y, capi.ptr(y), capi.ptr(inv), capi.ptr(top_w), capi.ptr(output),
              capi.ptr(sh_out), capi.ptr(gate), H, k, T, 0, capi.act_dtype(output), 1)
    return output


def moe_combine(y, inv, top_w, output, top_k):
    """output[t] = sum_j top_w[t, j] * y[inv[t * top_k + j]]; y fp32 or the activation dtype."""
    who = "moe_combine"
    T, H = output.shape
    _chk(output.dtype in (torch.float16, torch.bfloat16) and output.is_contiguous(), f"{who}: output must be contiguous fp16/bf16 [T, H]")
    _chk(y.dtype in (output.dtype, torch.float32, torch.float16) and y.is_contiguous() and y.shape[-1] == H,
         f"{who}: y must be [T*k, H] fp32, fp16 or the activation dtype")
    _chk(inv.dtype == torch.int32 and inv.numel() >= T * int(top_k), f"{who}: inv must be int32 [T*k]")
    _chk(top_w.dtype == output.dtype and top_w.is_contiguous(), f"{who}: top_w must share the output dtype")
    _chk(H % 8 == 0, f"{who}: H must be a multiple of 8")
    capi.call("mi_moe_combine", y, capi.ptr(y), capi.ptr(inv), capi.ptr(top_w), capi.ptr(output), H, int(top_k), T, 0,
              capi.act_dtype(output), _out_kind(y, capi.act_dtype(output)))
    return output


def moe_prefill_gather_forward_fp8(selected_experts, num_experts):
    """-> [expert_offsets [E], expert_tokens [T*k] (sorted position -> pair index),
    pair_to_perm [T*k], rows_for_experts [E]], with the stable in-expert order."""
    _chk(selected_experts.dim() == 2 and selected_experts.dtype == torch.int32, "moe_prefill_gather_forward_fp8: selected_experts must be int32 [T, k]")
    sel = selected_experts.contiguous()
    T, k = sel.shape
    E = int(num_experts)
    dev = sel.device
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    tokens = torch.empty(T * k, dtype=torch.int32, device=dev)
    perm = torch.empty(T * k, dtype=torch.int32, device=dev)
    moe_sort(sel, E, tokens, start, perm, None, None)
    return [start[:E], tokens, perm, start[1:] - start[:E]]

def moe_prefill_gather_forward_v2(selected_experts, num_experts):
    """moe_int4_prefill_ops::moe_prefill_gather_forward_v2: the same grouping under the name the FP8
    grouped path of the patched vLLM calls (V/csrc/moe_prefill/moe_prefill_int4.sycl:458-486,
    vllm/patches/vllm_for_multi_arc.patch:8228-8230)."""
    return moe_prefill_gather_forward_fp8(selected_experts, num_experts)


def moe_topk_softmax(router_logits, top_k, num_experts):
    """-> [weights [T, top_k] (renormalised, logits dtype), ids [T, top_k] int32]
    (V/csrc/moe_prefill/moe_prefill_int4.sycl:869-920)."""
    _chk(router_logits.dim() == 2 and router_logits.shape[1] == int(num_experts),
         "moe_topk_softmax: router_logits.size(1) must equal num_experts")
    w, ids = moe_topk(router_logits, int(top_k), True)
    return [w, ids]


# --------------------------------------------------------------------------
# decode fusions: RMS norm (+ residual add / + SiLU gate) in front of a GEMV
# (V/csrc/xpu/torch_extension.cc:103-140).  Two launches here: the norm kernel,
# then the GEMV entry point on its 16-bit output.
# --------------------------------------------------------------------------
def _rmsnorm(x, residual, gate, weight, out, rows, L, eps, who, residual_scale=1.0):
    _chk(x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(), f"{who}: activations must be contiguous fp16/bf16")
    for name, t in (("residual", residual), ("gate", gate), ("norm_weight", weight), ("normed output", out)):
        if t is not None:
            _chk(t.dtype == x.dtype and t.is_contiguous() and t.device == x.device, f"{who}: {name} must match the input's dtype/device and be contiguous")
    _chk(x.numel() == rows * L and out.numel() >= rows * L, f"{who}: size mismatch")
    _chk(weight.numel() >= 1 and L % weight.numel() == 0, f"{who}: norm_weight length must divide the row length")
    capi.call("mi_rmsnorm", x, capi.ptr(x), capi.ptr(residual), capi.ptr(gate), capi.ptr(weight), capi.ptr(out),
              rows, L, weight.numel(), float(eps), capi.act_dtype(x), float(residual_scale))
    return out


def esimd_fused_add_rms_norm(hidden_states, residual, weight, eps):
    """residual = hidden_states + residual (in place); hidden_states = rmsnorm(residual) * weight (in place)
    (V/csrc/xpu/torch_extension.cc:141-143; one row in the reference, any number here)."""
    K = hidden_states.shape[-1]
    return _rmsnorm(hidden_states, residual, None, weight, hidden_states, hidden_states.numel() // K, K, eps,
                    "esimd_fused_add_rms_norm")


def esimd_fused_add_rms_norm_batched(hidden_states, residual, weight, eps):
    """The same for any number of rows (torch_extension.cc:154-156)."""
    K = hidden_states.shape[-1]
    return _rmsnorm(hidden_states, residual, None, weight, hidden_states, hidden_states.numel() // K, K, eps,
                    "esimd_fused_add_rms_norm_batched")


def esimd_fused_scaled_add_rms_norm(hidden_states, residual, weight, eps, scalar):
    """residual = (hidden_states + residual) * scalar (in place); hidden_states = rmsnorm(residual) * weight
    (torch_extension.cc:145-148)."""
    K = hidden_states.shape[-1]
    return _rmsnorm(hidden_states, residual, None, weight, hidden_states, hidden_states.numel() // K, K, eps,
                    "esimd_fused_scaled_add_rms_norm", residual_scale=float(scalar))


def esimd_rms_norm_gated(x, z, weight, output, eps):
    """output = rmsnorm(x) * weight * silu(z) per row of V = len(weight) elements
    (torch_extension.cc:150-152)."""
    V = weight.numel()
    _chk(x.numel() % V == 0 and z.numel() == x.numel(), "esimd_rms_norm_gated: x and z must be [rows, V]")
    return _rmsnorm(x, None, z, weight, output, x.numel() // V, V, eps, "esimd_rms_norm_gated")


def esimd_rms_norm(input, output, weight, eps):
    """output = input * rsqrt(mean(input^2) + eps) * weight, per row (esimd_kernel.sycl:488-502)."""
    K = input.shape[-1]
    return _rmsnorm(input, None, None, weight, output, input.numel() // K, K, eps, "esimd_rms_norm")


_NORM_FP8_PERT, _NORM_FP8_BLOCK, _NORM_INT4 = 0, 1, 2


def _norm_gemv(x, residual, gate, norm_weight, normed_out, norm_len, eps, fmt, ws, ss, outs, who, residual_scale=1.0):
    """One launch: RMS norm (+ residual add / SiLU gate) of the single activation row, fused
    into the decode GEMV over `ws`.  More than one row takes the norm kernel + GEMV route."""
    _chk(x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(), f"{who}: activations must be contiguous fp16/bf16")
    for name, t in (("residual", residual), ("gate", gate), ("norm_weight", norm_weight), ("normed output", normed_out)):
        if t is not None:
            _chk(t.dtype == x.dtype and t.is_contiguous() and t.device == x.device,
                 f"{who}: {name} must match the input's dtype/device and be contiguous")
    if fmt == _NORM_INT4:
        K = ws[0].shape[1] * (2 if ws[0].dtype == torch.uint8 else 8)
    else:
        K = ws[0].shape[1]
    _chk(x.numel() % K == 0, f"{who}: input numel {x.numel()} is not a multiple of K={K}")
    rows = x.numel() // K
    norm_len = int(norm_len)
    _chk(norm_weight.numel() == norm_len and K % norm_len == 0, f"{who}: norm_weight must have {norm_len} entries dividing K={K}")
    for t in (residual, gate):
        if t is not None:
            _chk(t.numel() == x.numel(), f"{who}: residual / gate must have the input's size")
    if normed_out is not None:
        _chk(normed_out.numel() >= x.numel(), f"{who}: normed output is too small")
    if rows != 1:
        normed = normed_out if normed_out is not None else torch.empty_like(x)
        _rmsnorm(x, residual, gate, norm_weight, normed, x.numel() // norm_len, norm_len, eps, who, residual_scale)
        xin = normed.view(rows, K)
        if fmt == _NORM_INT4:
            return _int4_multi(xin, ws, ss, [None] * len(ws), outs, who)
        if fmt == _NORM_FP8_PERT:
            return _fp8_pert_multi(xin, ws, ss, outs, who)
        return esimd_gemm_fp8_blockscale(xin, ws[0], ss[0], outs[0], 128, 128)
    Ns = []
    for w, sc, o in zip(ws, ss, outs):
        _chk(w.dim() == 2 and w.is_contiguous(), f"{who}: weights must be contiguous 2-D tensors")
        _chk_act(x, o, who)
        if fmt == _NORM_INT4:
            _chk(w.dtype in (torch.uint8, torch.int32), f"{who}: int4 weight must be uint8 [N, K/2] or int32 [N, K/8]")
            _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
            _chk(sc.dtype == torch.float16 and sc.is_contiguous() and sc.numel() == w.shape[0] * (K // 128),
                 f"{who}: gemv_scale must be contiguous fp16 [N, K/128]")
        else:
            _chk_fp8(w, who)
            _chk(w.shape[1] == K, f"{who}: all weights must be [N, K={K}]")
            if fmt == _NORM_FP8_PERT:
                _chk(sc.dtype == torch.float32 and sc.numel() >= 1, f"{who}: gemv_scale must be an fp32 scalar tensor")
            else:
                _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
                _chk(sc.dtype == torch.float32 and sc.is_contiguous() and sc.numel() == -(-w.shape[0] // 128) * (K // 128),
                     f"{who}: gemv_scale must be contiguous fp32 [ceil(N/128), K/128]")
        _chk(o.numel() == w.shape[0], f"{who}: output has {o.numel()} elements, expected N={w.shape[0]}")
        Ns.append(w.shape[0])
    capi.call("mi_norm_gemv_scaled", x, capi.ptr(x), capi.ptr(residual), capi.ptr(gate), capi.ptr(norm_weight),
              capi.ptr(normed_out), norm_len, float(eps), float(residual_scale), fmt, len(ws), capi.ptr_array(ws), capi.ptr_array(ss),
              capi.ptr_array(outs), capi.int_array(Ns), K, capi.act_dtype(x))
    return outs[0]


def esimd_resadd_norm_gemv_int4_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                     normed_out, eps):
    """residual += hidden_states (in place); normed_out = rmsnorm(residual) * norm_weight;
    output = normed_out @ dequant(int4 weight)^T  (resadd_norm_gemv_int4.h:1-30)."""
    K = hidden_states.shape[-1]
    return _norm_gemv(hidden_states, residual, None, norm_weight, normed_out, K, eps, _NORM_INT4,
                      [gemv_weight], [gemv_scale], [output], "esimd_resadd_norm_gemv_int4_pert")


def esimd_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, gemv_weight, gemv_scale, output,
                                    normed_out, eps):
    """Same with an FP8 weight and a per-tensor scale (resadd_norm_gemv_fused.h)."""
    K = hidden_states.shape[-1]
    return _norm_gemv(hidden_states, residual, None, norm_weight, normed_out, K, eps, _NORM_FP8_PERT,
                      [gemv_weight], [gemv_scale], [output], "esimd_resadd_norm_gemv_fp8_pert")


def esimd_scaled_resadd_norm_gemv_fp8_pert(hidden_states, residual, norm_weight, qkv_weight, qkv_scale, qkv_out, eps,
                                           scalar):
    """residual <- (hidden_states + residual) * scalar (in place); qkv_out = (rmsnorm(residual) * norm_weight)
    @ (qkv_scale * e4m3(qkv_weight))^T in one launch (V/csrc/xpu/esimd_kernels/scaled_resadd_norm_gemv_fp8.h)."""
    K = hidden_states.shape[-1]
    # rows beyond the fused kernel's 16384 elements go through the norm kernel and need a buffer for its output
    normed = torch.empty_like(hidden_states) if K > 16384 else None
    _norm_gemv(hidden_states, residual, None, norm_weight, normed, K, eps, _NORM_FP8_PERT, [qkv_weight], [qkv_scale],
               [qkv_out], "esimd_scaled_resadd_norm_gemv_fp8_pert", residual_scale=float(scalar))


def _norm_add_norm(src, rows_per_token, h1, w1, w2, out, eps1, eps2, who):
    _chk(src.dtype in (torch.float16, torch.bfloat16), f"{who}: activations must be fp16 or bf16")
    for name, t in (("input", src), ("h1", h1), ("w1", w1), ("w2", w2), ("out", out)):
        _chk(t.dtype == src.dtype and t.is_contiguous() and t.device == src.device,
             f"{who}: {name} must be contiguous and share dtype and device")
    K = h1.shape[-1]
    T = h1.numel() // K
    _chk(w1.numel() == K and w2.numel() == K and out.numel() == T * K and src.numel() == T * rows_per_token * K,
         f"{who}: sizes must be h1/out [T, K], w1/w2 [K], input [T * rows, K]")
    capi.call("mi_norm_add_norm", src, capi.ptr(src), int(rows_per_token), capi.ptr(h1), capi.ptr(w1), capi.ptr(w2),
              capi.ptr(out), T, K, float(eps1), float(eps2), capi.act_dtype(src))


def esimd_norm_add_norm(h2_raw, h1, w1, w2, out, eps1, eps2):
    """h1 <- rmsnorm(h2_raw, eps1) * w1 + h1 (in place); out = rmsnorm(h1, eps2) * w2
    (V/csrc/xpu/esimd_kernels/norm_add_norm.h:46-86)."""
    _norm_add_norm(h2_raw, 1, h1, w1, w2, out, eps1, eps2, "esimd_norm_add_norm")


def esimd_accum_norm_add_norm(routed_output, h1, w1, w2, out, top_k, eps1, eps2):
    """The same with h2 = the sum of each token's top_k rows of routed_output
    (V/csrc/xpu/esimd_kernels/accum_norm_add_norm.h)."""
    _chk(int(top_k) >= 1, "esimd_accum_norm_add_norm: top_k must be positive")
    _norm_add_norm(routed_output, int(top_k), h1, w1, w2, out, eps1, eps2, "esimd_accum_norm_add_norm")


def esimd_norm_gemv_norm_fp16(residual, scale_with_root, proj_w, pre_ff_w, router_logits, moe_input, eps):
    """router_logits = (rmsnorm(residual) * scale_with_root) @ proj_w^T and moe_input = rmsnorm(residual) * pre_ff_w
    (V/csrc/xpu/esimd_kernels/norm_gemv_norm_fp16.h:1-40).  Runs the three launches the reference's fusion
    replaces (norm, 16-bit GEMV, norm); the router's input is rounded to the activation dtype in between."""
    who = "esimd_norm_gemv_norm_fp16"
    _chk(residual.dtype in (torch.float16, torch.bfloat16) and residual.is_contiguous(), f"{who}: residual must be contiguous fp16")
    K = residual.shape[-1]
    _chk(scale_with_root.numel() == K and pre_ff_w.numel() == K and moe_input.numel() == residual.numel(),
         f"{who}: scale_with_root / pre_ff_w must be [K], moe_input must match residual")
    rows = residual.numel() // K
    tmp = torch.empty_like(residual)
    _rmsnorm(residual, None, None, scale_with_root, tmp, rows, K, eps, who)
    _gemv_w16(tmp.view(rows, K), proj_w, router_logits, False, who)
    _rmsnorm(residual, None, None, pre_ff_w, moe_input, rows, K, eps, who)


def esimd_resadd_norm_gemv2_fp8_pert(hidden_states, residual, norm_weight, w0, s0, o0, w1, s1, o1, eps):
    """Residual add + RMS norm feeding two per-tensor FP8 GEMVs in one launch (resadd_norm_gemv2_fused.h)."""
    K = hidden_states.shape[-1]
    return _norm_gemv(hidden_states, residual, None, norm_weight, None, K, eps, _NORM_FP8_PERT,
                      [w0, w1], [s0, s1], [o0, o1], "esimd_resadd_norm_gemv2_fp8_pert")


def _gated_norm_gemv(x, z, norm_weight, HV, V, eps, fmt, weight, scale, output, who):
    HV, V = int(HV), int(V)
    _chk(x.numel() % (HV * V) == 0 and z.numel() == x.numel(), f"{who}: x and z must hold HV*V elements per row")
    _chk(norm_weight.numel() == V, f"{who}: norm_weight must have V entries")
    return _norm_gemv(x, None, z, norm_weight, None, V, eps, fmt, [weight], [scale], [output], who)


def esimd_norm_gemv_int4_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    """Per-head RMS norm gated by silu(z), then INT4 GEMV over the HV*V vector (norm_gemv_int4.h)."""
    return _gated_norm_gemv(x, z, norm_weight, HV, V, eps, _NORM_INT4, gemv_weight, gemv_scale, output,
                            "esimd_norm_gemv_int4_pert")


def esimd_norm_gemv_fp8_pert(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    """Per-head gated RMS norm, then per-tensor FP8 GEMV (norm_gemv_fused.h)."""
    return _gated_norm_gemv(x, z, norm_weight, HV, V, eps, _NORM_FP8_PERT, gemv_weight, gemv_scale, output,
                            "esimd_norm_gemv_fp8_pert")


def esimd_norm_gemv_fp8_blockscale(x, z, norm_weight, gemv_weight, gemv_scale, output, HV, V, eps):
    """Per-head gated RMS norm, then 128x128 block-scaled FP8 GEMV (torch_extension_gemm.cc:42-45)."""
    return _gated_norm_gemv(x, z, norm_weight, HV, V, eps, _NORM_FP8_BLOCK, gemv_weight, gemv_scale, output,
                            "esimd_norm_gemv_fp8_blockscale")


# --------------------------------------------------------------------------
# sglang FP8 MoE prefill ops (per-expert scalar scales), moe_fp8_prefill_ops
# --------------------------------------------------------------------------
def _prefill_starts(expert_offsets, total):
    """[E] exclusive offsets -> [E + 1] with the total appended."""
    tail = torch.full((1,), total, dtype=torch.int32, device=expert_offsets.device)
    return torch.cat([expert_offsets.reshape(-1), tail]).contiguous()


def _permute_rows(src, map_, dst, scatter):
    rows = map_.numel()
    capi.call("mi_permute_rows", src, capi.ptr(src), capi.ptr(map_), capi.ptr(dst), rows,
              src.shape[1] * src.element_size(), 1 if scatter else 0)
    return dst


def moe_prefill_up_forward_fp8(x, gate_up_weight, gate_up_scale, expert_offsets, expert_tokens, top_k):
    """intermediate[pair] = silu(x[t] @ (s_gate w_gate)^T) * (x[t] @ (s_up w_up)^T) for pair = t*top_k + j,
    rows grouped per expert by (expert_offsets, expert_tokens) as moe_prefill_gather_forward_fp8 returns them
    (S/csrc/moe_prefill/moe_prefill_fp8.sycl:480-530).  -> [T*top_k, I] in pair order."""
    who = "moe_prefill_up_forward_fp8"
    _chk(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(), f"{who}: x must be contiguous fp16/bf16 [T, H]")
    _chk(gate_up_weight.dim() == 3, f"{who}: gate_up_weight must be [E, 2*I, H]")
    _chk_fp8(gate_up_weight, who)
    _chk(gate_up_scale.dtype == torch.float32, f"{who}: gate_up_scale must be float32")
    _chk(expert_offsets.dtype == torch.int32 and expert_tokens.dtype == torch.int32, f"{who}: offsets and tokens must be int32")
    E, two_i, H = gate_up_weight.shape
    I = two_i // 2
    _chk(x.shape[1] == H, f"{who}: x hidden dim must equal w13 last dim")
    _chk(gate_up_scale.numel() >= 2 * E, f"{who}: gate_up_scale must have >= 2*E entries ([E,2] gate/up)")
    P = expert_tokens.numel()
    k = int(top_k)
    dev = x.device
    _chk(H % 16 == 0 and two_i % 2 == 0, f"{who}: H must be a multiple of 16")
    start = _prefill_starts(expert_offsets, P)
    tokens = expert_tokens.contiguous()
    out = torch.empty(P, I, dtype=x.dtype, device=dev)
    # the gate / up scalars of an expert go to the kernel as they are; the pair index -> token division too
    return _moe_gemm(x, None, tokens, gate_up_weight, gate_up_scale.contiguous(), start, out, E, two_i, H, _ACT_SILU, who,
                     per_expert=2, out_map=tokens, row_map_div=k)


def moe_prefill_down_forward_fp8(intermediate, down_weight, down_scale, expert_offsets, expert_tokens):
    """expert_output[pair] = intermediate[pair] @ (s[e] w2[e])^T, both in pair order
    (S/csrc/moe_prefill/moe_prefill_fp8.sycl:532-582)."""
    who = "moe_prefill_down_forward_fp8"
    _chk(intermediate.dim() == 2 and intermediate.dtype in (torch.float16, torch.bfloat16) and intermediate.is_contiguous(),
         f"{who}: intermediate must be contiguous fp16/bf16 [T*k, I]")
    _chk(down_weight.dim() == 3, f"{who}: down_weight must be [E, H, I]")
    _chk_fp8(down_weight, who)
    _chk(down_scale.dtype == torch.float32, f"{who}: down_scale must be float32")
    _chk(expert_offsets.dtype == torch.int32 and expert_tokens.dtype == torch.int32, f"{who}: offsets and tokens must be int32")
    E, H, I = down_weight.shape
    _chk(intermediate.shape[1] == I, f"{who}: intermediate dim must equal w2 last dim")
    _chk(down_scale.numel() >= E, f"{who}: down_scale must have >= E entries")
    P = expert_tokens.numel()
    _chk(I % 16 == 0, f"{who}: I must be a multiple of 16")
    start = _prefill_starts(expert_offsets, P)
    tokens = expert_tokens.contiguous()
    out = torch.empty(P, H, dtype=intermediate.dtype, device=intermediate.device)
    return _moe_gemm(intermediate, None, tokens, down_weight, down_scale.contiguous(), start, out, E, H, I, _ACT_NONE, who,
                     per_expert=1, out_map=tokens)


def moe_prefill_accumulate_forward_fp8(output, routing_weights):
    """routing_output[t] = sum_j routing_weights[t, j] * output[t*k + j]
    (S/csrc/moe_prefill/moe_prefill_fp8.sycl:413-436, :584-611)."""
    who = "moe_prefill_accumulate_forward_fp8"
    _chk(output.dim() == 2 and routing_weights.dim() == 2, f"{who}: output [T*k, H], routing_weights [T, k]")
    _chk(output.dtype in (torch.float16, torch.bfloat16) and routing_weights.dtype == output.dtype, f"{who}: fp16/bf16 tensors of one dtype")
    T, k = routing_weights.shape
    H = output.shape[1]
    _chk(output.shape[0] >= T * k and H % 8 == 0, f"{who}: output too small or H not a multiple of 8")
    res = torch.empty(T, H, dtype=output.dtype, device=output.device)
    capi.call("mi_moe_combine_shared", output, capi.ptr(output.contiguous()), None, capi.ptr(routing_weights.contiguous()),
              capi.ptr(res), None, None, H, k, T, 0, capi.act_dtype(res), 0)
    return res


def moe_prefill_full_fp8(hidden_states, topk_weights, topk_ids, w13, w13_scale, w2, w2_scale, top_k, num_experts):
    """Prefill MoE with per-expert scalar scales: stable expert sort -> grouped gate_up GEMM with
    SiLU*mul -> grouped down GEMM -> weighted combine (S/csrc/moe_prefill/moe_prefill_fp8.sycl:616-649).
    The intermediate stays in expert-sorted order, so the two pair-order round trips of the
    separate ops are not made here; H and I may be any multiples of 16."""
    who = "moe_prefill_full_fp8"
    _chk(hidden_states.dtype in (torch.float16, torch.bfloat16), f"{who}: hidden_states must be fp16 (bf16 accepted)")
    _chk(topk_weights.dtype == hidden_states.dtype, f"{who}: topk_weights must be fp16 (the activation dtype)")
    _chk(topk_ids.dtype == torch.int32, f"{who}: topk_ids must be int32")
    k, E = int(top_k), int(num_experts)
    _chk(topk_ids.dim() == 2 and topk_ids.shape[1] == k, f"{who}: topk_ids must be [M, top_k]")
    _chk(w13.dim() == 3 and w2.dim() == 3 and w13.shape[0] == E and w2.shape[0] == E, f"{who}: w13 [E,2I,H], w2 [E,H,I]")
    _chk_fp8(w13, who)
    _chk_fp8(w2, who)
    x = hidden_states.contiguous()
    T, H = x.shape
    I = w2.shape[2]
    _chk(tuple(w13.shape) == (E, 2 * I, H) and tuple(w2.shape) == (E, H, I), f"{who}: w13 [E,2I,H], w2 [E,H,I]")
    _chk(w13_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32, f"{who}: scales must be float32")
    _chk(w13_scale.numel() >= 2 * E and w2_scale.numel() >= E, f"{who}: w13_scale [E,2], w2_scale [E]")
    dev = x.device
    P = T * k
    ids = topk_ids.contiguous()
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    sorted_token = torch.empty(P, dtype=torch.int32, device=dev)
    moe_sort(ids, E, sorted_pairs, start, inv, sorted_token, None)
    inter = torch.empty(P, I, dtype=x.dtype, device=dev)
    # fp32 expert outputs; with hundreds of rows per expert the tiled grouped GEMM takes over, which writes
    # the activation type (as the reference's kernels do)
    prefill = P >= 96 * E and H % 128 == 0 and I % 128 == 0
    y = torch.empty(P, H, dtype=x.dtype if prefill else torch.float32, device=dev)
    _chk(H % 16 == 0 and I % 16 == 0, f"{who}: H and I must be multiples of 16")
    _moe_gemm(x, None, sorted_token, w13, w13_scale.contiguous(), start, inter, E, 2 * I, H, _ACT_SILU, who, per_expert=2)
    _moe_gemm(inter, None, None, w2, w2_scale.contiguous(), start, y, E, H, I, _ACT_NONE, who, per_expert=1)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    moe_combine(y, inv, topk_weights.contiguous(), out, k)
    return out


# --------------------------------------------------------------------------
# per-expert-scale FP8 MoE with the tanh-GELU gate (moe_ops: the gemma-style family)
# weights in the FusedMoE layout: gate_up [E, 2I, H], down [E, H, I] e4m3, scales [E] fp32
# --------------------------------------------------------------------------
def _chk_pert_moe(x, gate_up_weight, gate_up_scale, down_weight, down_scale, who):
    _chk(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(),
         f"{who}: x must be contiguous fp16 (bf16 accepted) [T, H]")
    if gate_up_weight is not None:
        _chk(gate_up_weight.dim() == 3 and gate_up_weight.shape[1] % 2 == 0, f"{who}: gate_up_weight must be [E, 2*I, H]")
        _chk_fp8(gate_up_weight, who)
        _chk(gate_up_scale.dtype == torch.float32 and gate_up_scale.numel() >= gate_up_weight.shape[0],
             f"{who}: gate_up_scale must be float32 [E]")
    if down_weight is not None:
        _chk(down_weight.dim() == 3, f"{who}: down_weight must be [E, H, I]")
        _chk_fp8(down_weight, who)
        _chk(down_scale.dtype == torch.float32 and down_scale.numel() >= down_weight.shape[0],
             f"{who}: down_scale must be float32 [E]")


def moe_up_fp8_grouped(x, gate_up_weight, gate_up_scale, expert_offsets, expert_tokens, top_k, n_routed_experts):
    """intermediate[pair] = gelu_tanh(x[t] @ (s[e] w_gate[e])^T) * (x[t] @ (s[e] w_up[e])^T), pair = t*top_k + j,
    for the pairs grouped per expert by (expert_offsets [E] exclusive, expert_tokens [T*top_k])
    (V/csrc/moe_batch/moe_fp8_grouped.h:348-408).  -> [T*top_k, I] in pair order."""
    who = "moe_up_fp8_grouped"
    _chk_pert_moe(x, gate_up_weight, gate_up_scale, None, None, who)
    _chk(expert_offsets.dtype == torch.int32 and expert_tokens.dtype == torch.int32, f"{who}: offsets and tokens must be int32")
    E, two_i, H = gate_up_weight.shape
    _chk(E == int(n_routed_experts) and x.shape[1] == H, f"{who}: x [T, H] against gate_up_weight [E, 2*I, H]")
    k = int(top_k)
    P = x.shape[0] * k
    _chk(expert_tokens.numel() == P and expert_offsets.numel() >= E, f"{who}: expert_tokens must hold T*top_k pairs")
    tokens = expert_tokens.contiguous()
    out = torch.empty(P, two_i // 2, dtype=x.dtype, device=x.device)
    return _moe_gemm(x, None, tokens, gate_up_weight, gate_up_scale.contiguous(), _prefill_starts(expert_offsets[:E], P),
                     out, E, two_i, H, _ACT_GELU_TANH, who, per_expert=True, out_map=tokens, row_map_div=k)


def moe_down_fp8_grouped(intermediate, down_weight, down_scale, routing_weights, expert_offsets, expert_tokens,
                         top_k, n_routed_experts):
    """out[pair] = routing_weights[pair] * (intermediate[pair] @ (s[e] w2[e])^T), pair order in and out
    (V/csrc/moe_batch/moe_fp8_grouped.h:410-433)."""
    who = "moe_down_fp8_grouped"
    _chk_pert_moe(intermediate, None, None, down_weight, down_scale, who)
    _chk(expert_offsets.dtype == torch.int32 and expert_tokens.dtype == torch.int32, f"{who}: offsets and tokens must be int32")
    E, H, I = down_weight.shape
    P = intermediate.shape[0]
    _chk(E == int(n_routed_experts) and intermediate.shape[1] == I, f"{who}: intermediate [T*top_k, I] against down_weight [E, H, I]")
    _chk(routing_weights.dtype == intermediate.dtype and routing_weights.numel() == P and expert_tokens.numel() == P,
         f"{who}: routing_weights and expert_tokens must hold one entry per pair, weights in the activation dtype")
    tokens = expert_tokens.contiguous()
    out = torch.empty(P, H, dtype=intermediate.dtype, device=intermediate.device)
    return _moe_gemm(intermediate, None, tokens, down_weight, down_scale.contiguous(), _prefill_starts(expert_offsets[:E], P),
                     out, E, H, I, _ACT_NONE, who, per_expert=True, out_map=tokens,
                     row_weight=routing_weights.contiguous().reshape(-1))


def moe_forward_full_fp8_grouped(x, gate_up_weight, gate_up_scale, down_weight, down_scale, routing_weights,
                                 expert_offsets, expert_tokens, top_k, n_routed_experts):
    """Up (tanh-GELU), down and the sum over each token's top_k routes in one call
    (V/csrc/moe_batch/moe_fp8_grouped.h:471-500).  The intermediate stays in expert-sorted order and
    the down output in fp32 until the weighted sum, which rounds once."""
    who = "moe_forward_full_fp8_grouped"
    _chk_pert_moe(x, gate_up_weight, gate_up_scale, down_weight, down_scale, who)
    _chk(expert_offsets.dtype == torch.int32 and expert_tokens.dtype == torch.int32, f"{who}: offsets and tokens must be int32")
    E, two_i, H = gate_up_weight.shape
    I = two_i // 2
    _chk(tuple(down_weight.shape) == (E, H, I) and x.shape[1] == H and E == int(n_routed_experts),
         f"{who}: gate_up_weight [E, 2*I, H], down_weight [E, H, I], x [T, H]")
    k = int(top_k)
    T = x.shape[0]
    P = T * k
    _chk(routing_weights.dtype == x.dtype and routing_weights.numel() == P and expert_tokens.numel() == P,
         f"{who}: routing_weights and expert_tokens must hold one entry per pair, weights in the activation dtype")
    tokens = expert_tokens.contiguous()
    start = _prefill_starts(expert_offsets[:E], P)
    inter = torch.empty(P, I, dtype=x.dtype, device=x.device)
    _moe_gemm(x, None, tokens, gate_up_weight, gate_up_scale.contiguous(), start, inter, E, two_i, H, _ACT_GELU_TANH, who,
              per_expert=True, row_map_div=k)
    y = torch.empty(P, H, dtype=torch.float32, device=x.device)
    _moe_gemm(inter, None, None, down_weight, down_scale.contiguous(), start, y, E, H, I, _ACT_NONE, who, per_expert=True,
              out_map=tokens)
    out = torch.empty(T, H, dtype=x.dtype, device=x.device)
    capi.call("mi_moe_combine", y, capi.ptr(y), None, capi.ptr(routing_weights.contiguous()), capi.ptr(out), H, k, T, 0,
              capi.act_dtype(out), 1)
    return out


def _moe_pert_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale, top_k,
                     act, accumulate, who):
    _chk_pert_moe(x, gate_up_weight, gate_up_scale, down_weight, down_scale, who)
    _chk(topk_weights.dtype == x.dtype, f"{who}: topk_weights must be fp16 (the activation dtype) [T, top_k]")
    _chk(topk_indices.dtype == torch.int32, f"{who}: topk_indices must be int32 [T, top_k]")
    E, two_i, H = gate_up_weight.shape
    I = two_i // 2
    T = x.shape[0]
    k = int(top_k)
    P = T * k
    _chk(tuple(down_weight.shape) == (E, H, I) and x.shape[1] == H, f"{who}: gate_up_weight [E, 2*I, H], down_weight [E, H, I], x [T, H]")
    _chk(topk_weights.numel() == P and topk_indices.numel() == P, f"{who}: routing tensors must be [T, top_k]")
    dev = x.device
    ids = topk_indices.contiguous().reshape(T, k)
    top_w = topk_weights.contiguous().reshape(T, k)
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    sorted_token = torch.empty(P, dtype=torch.int32, device=dev)
    moe_sort(ids, E, sorted_pairs, start, inv, sorted_token, None)
    inter = torch.empty(P, I, dtype=x.dtype, device=dev)
    _moe_gemm(x, None, sorted_token, gate_up_weight, gate_up_scale.contiguous(), start, inter, E, two_i, H, act, who,
              per_expert=True)
    if not accumulate:
        out = torch.empty(P, H, dtype=x.dtype, device=dev)
        return _moe_gemm(inter, None, None, down_weight, down_scale.contiguous(), start, out, E, H, I, _ACT_NONE, who,
                         per_expert=True, out_map=sorted_pairs, row_weight=top_w.reshape(-1))
    y = torch.empty(P, H, dtype=torch.float32, device=dev)
    _moe_gemm(inter, None, None, down_weight, down_scale.contiguous(), start, y, E, H, I, _ACT_NONE, who, per_expert=True)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    return moe_combine(y, inv, top_w, out, k)


def moe_forward_full_gelu_tanh_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight,
                                      down_scale, top_k, n_routed_experts):
    """out[t] = sum_j w[t, j] * down_e(gelu_tanh(gate_e(x[t])) * up_e(x[t])), e = topk_indices[t, j], with the
    caller's routing (V/csrc/moe_batch/moe.sycl:2249-2293)."""
    return _moe_pert_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale,
                            top_k, _ACT_GELU_TANH, True, "moe_forward_full_gelu_tanh_routed")


def moe_forward_full_gelu_tanh_routed_decode(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale,
                                             down_weight, down_scale, top_k, n_routed_experts):
    """The one-token form of moe_forward_full_gelu_tanh_routed (V/csrc/moe_batch/moe.sycl:2096-2170)."""
    who = "moe_forward_full_gelu_tanh_routed_decode"
    _chk(x.dim() == 2 and x.shape[0] == 1, f"{who}: the decode op takes one token")
    return _moe_pert_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale,
                            top_k, _ACT_GELU_TANH, True, who)


def moe_forward_full_gelu_tanh_routed_no_accum(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale,
                                               down_weight, down_scale, top_k, n_routed_experts):
    """The routing-weighted per-route rows [T*top_k, H] without the sum over routes
    (V/csrc/moe_batch/moe.sycl:2297-2335)."""
    return _moe_pert_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale,
                            top_k, _ACT_GELU_TANH, False, "moe_forward_full_gelu_tanh_routed_no_accum")


def moe_forward_full_silu_routed_sglang(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight,
                                        down_scale, top_k, n_routed_experts):
    """SiLU form of moe_forward_full_gelu_tanh_routed on N-major weights gate_up [E, 2*I, H] / down [E, H, I],
    one fp32 scale per expert (S/csrc/moe_batch/moe.sycl:1953-2007)."""
    return _moe_pert_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale,
                            top_k, _ACT_SILU, True, "moe_forward_full_silu_routed_sglang")


def moe_forward_full_silu_routed(x, topk_weights, topk_indices, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                 top_k, n_routed_experts):
    """The same forward with the up projection K-major: gate_up [E, H, 2*I] (the caller transposes w13),
    down [E, H, I] (S/csrc/moe_batch/moe.sycl:2022-2077).  The up projection runs on the K-major
    streaming kernel (fp32 split partials), the activation kernel rounds SiLU(gate) * up once to the
    activation dtype in pair order, and the down projection is the grouped GEMM over expert-sorted
    pairs with fp32 rows summed per token."""
    who = "moe_forward_full_silu_routed"
    _chk(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(),
         f"{who}: x must be contiguous fp16 [T, H]")
    _chk(topk_weights.dtype == x.dtype, f"{who}: topk_weights must be fp16 (the activation dtype) [T, top_k]")
    _chk(topk_indices.dtype == torch.int32, f"{who}: topk_indices must be int32 [T, top_k]")
    _chk_fp8(gate_up_weight, who)
    _chk_fp8(down_weight, who)
    T, H = x.shape
    k = int(top_k)
    P = T * k
    _chk(gate_up_weight.dim() == 3 and gate_up_weight.shape[1] == H and gate_up_weight.shape[2] % 32 == 0 and
         gate_up_weight.is_contiguous(),
         f"{who}: gate_up_weight must be [E, hidden, 2*intermediate] - transpose w13 before calling")
    E = gate_up_weight.shape[0]
    I = gate_up_weight.shape[2] // 2
    _chk(tuple(down_weight.shape) == (E, H, I) and down_weight.is_contiguous(), f"{who}: down_weight must be [E, H, I]")
    _chk(gate_up_scale.dtype == torch.float32 and gate_up_scale.numel() >= E and down_scale.dtype == torch.float32 and
         down_scale.numel() >= E, f"{who}: scales must be float32 [E]")
    _chk(topk_weights.numel() == P and topk_indices.numel() == P, f"{who}: routing tensors must be [T, top_k]")
    dev = x.device
    adt = capi.act_dtype(x)
    ids = topk_indices.contiguous().reshape(T, k)
    top_w = topk_weights.contiguous().reshape(T, k)
    route_expert = ids.reshape(-1)
    s_up = _km_splits(P, H, 2 * I, dev)
    up_part = torch.empty(P, s_up, 2 * I, dtype=torch.float32, device=dev)
    capi.call("mi_moe_kmajor_up", x, capi.ptr(x), capi.ptr(gate_up_weight), capi.ptr(route_expert), capi.ptr(up_part), P, k,
              E, H, 2 * I, s_up, adt)
    inter = torch.empty(P, I, dtype=x.dtype, device=dev)
    capi.call("mi_moe_kmajor_act", x, capi.ptr(up_part), s_up, capi.ptr(gate_up_scale.contiguous()), capi.ptr(route_expert),
              capi.ptr(inter), P, E, I, 0, adt)
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    start = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    moe_sort(ids, E, sorted_pairs, start, inv, None, None)
    y = torch.empty(P, H, dtype=torch.float32, device=dev)
    _moe_gemm(inter, None, sorted_pairs, down_weight, down_scale.contiguous(), start, y, E, H, I, _ACT_NONE, who,
              per_expert=True)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    return moe_combine(y, inv, top_w, out, k)


def moe_forward_full_gelu_tanh(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale, top_k,
                               n_routed_experts):
    """Softmax top-k with renormalisation, then moe_forward_full_gelu_tanh_routed
    (V/csrc/moe_batch/moe.sycl:2044-2094)."""
    who = "moe_forward_full_gelu_tanh"
    _chk(logits.dim() == 2 and logits.shape[1] == int(n_routed_experts) and logits.dtype == x.dtype,
         f"{who}: logits must be [T, n_routed_experts] in the activation dtype")
    top_w, top_ids = moe_topk(logits, int(top_k), True)
    return _moe_pert_routed(x, top_w, top_ids, gate_up_weight, gate_up_scale, down_weight, down_scale, top_k,
                            _ACT_GELU_TANH, True, who)


def moe_forward_full_gelu_tanh_decode(x, logits, gate_up_weight, gate_up_scale, down_weight, down_scale,
                                      per_expert_scale, top_k, n_routed_experts):
    """One token: softmax top-k, routing weights multiplied by per_expert_scale[e] and rounded to the
    activation dtype (MoeFoldExpertScale, V/csrc/moe_batch/moe_decode_gemv.h:146-158), then the routed
    forward (V/csrc/moe_batch/moe.sycl:2172-2241)."""
    who = "moe_forward_full_gelu_tanh_decode"
    _chk(x.dim() == 2 and x.shape[0] == 1, f"{who}: the decode op takes one token")
    _chk(logits.dim() == 2 and logits.shape[1] == int(n_routed_experts) and logits.dtype == x.dtype,
         f"{who}: logits must be [1, n_routed_experts] in the activation dtype")
    _chk(per_expert_scale.dtype == torch.float32 and per_expert_scale.numel() >= int(n_routed_experts),
         f"{who}: per_expert_scale must be float32 [n_routed_experts]")
    top_w, top_ids = moe_topk(logits, int(top_k), True, per_expert_scale.contiguous())
    return _moe_pert_routed(x, top_w, top_ids, gate_up_weight, gate_up_scale, down_weight, down_scale, top_k,
                            _ACT_GELU_TANH, True, who)


# --------------------------------------------------------------------------
# per-tensor FP8 MoE decode on K-major routed weights (moe_ops.moe_forward_full / _v2)
# --------------------------------------------------------------------------
def _km_splits(routes, K, N, dev):
    """Workgroups over K per (route, 1024-column block): about two per compute unit in total,
    at least 32 rows each, at most 1024 rows (the kernels' staging vector)."""
    cblocks = (N + 1023) // 1024
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    want = -(-2 * cus // max(1, routes * cblocks))
    # whole batches of 32 rows (8 per wavefront): a workgroup then waits for memory once per batch
    rows = min(1024, max(32, (K // want) // 32 * 32))
    return -(-K // rows)


def moe_forward_full(x, logits, gate_up_weight, gate_up_scale, shared_gate_up_weight, shared_gate_up_scale,
                     down_weight, down_scale, shared_down_weight, shared_down_scale, shared_expert_gate_weight,
                     top_k, num_shared_experts, n_routed_experts):
    """Per-tensor FP8 MoE decode step (V/csrc/moe_batch/moe.sycl:1855-1940): softmax top-k (renormalised),
    routed experts on K-major weights gate_up [E, H, 2I] / down [E, I, H] with one fp32 scale per expert,
    SiLU(gate) * up, + sigmoid(x . shared_expert_gate_weight[s]) * shared expert s (N-major
    [S, 2I, H] / [S, H, I], scales [S]).  -> [T, H].  E4M3 only; bf16 accepted besides fp16."""
    who = "moe_forward_full"
    _chk(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(), f"{who}: x must be contiguous fp16 [T, H]")
    E, k, S = int(n_routed_experts), int(top_k), int(num_shared_experts)
    T, H = x.shape
    _chk(E > 0 and 0 < k <= E and S >= 0, f"{who}: requires 0 < top_k <= n_routed_experts")
    _chk(logits.dim() == 2 and tuple(logits.shape) == (T, E) and logits.dtype == x.dtype, f"{who}: logits must be [T, E] in x's dtype")
    _chk(gate_up_weight.dim() == 3 and gate_up_weight.shape[0] == E and gate_up_weight.shape[1] == H and
         gate_up_weight.shape[2] % 32 == 0, f"{who}: gate_up_weight must be [E, H, 2*I] with I a multiple of 16")
    I = gate_up_weight.shape[2] // 2
    _chk(tuple(down_weight.shape) == (E, I, H) and H % 16 == 0, f"{who}: down_weight must be [E, I, H], H a multiple of 16")
    _chk_fp8(gate_up_weight, who)
    _chk_fp8(down_weight, who)
    _chk(gate_up_scale.dtype == torch.float32 and gate_up_scale.numel() >= E and down_scale.dtype == torch.float32 and
         down_scale.numel() >= E, f"{who}: routed scales must be float32 [E]")
    dev = x.device
    P = T * k
    gate = gate_args = None
    if S > 0:
        _chk(shared_expert_gate_weight.dtype == x.dtype and shared_expert_gate_weight.numel() == H,
             f"{who}: shared_expert_gate_weight must be [1, H] in x's dtype")
        gate = torch.empty(T, dtype=torch.float32, device=dev)
        gate_args = (x, shared_expert_gate_weight.contiguous(), gate)
    top_w, top_ids = moe_topk(logits, k, True, gate=gate_args)     # routing + the shared expert's gate, one launch
    route_expert = top_ids.reshape(-1)
    adt = capi.act_dtype(x)
    s_up = _km_splits(P, H, 2 * I, dev)
    up_part = torch.empty(P, s_up, 2 * I, dtype=torch.float32, device=dev)
    capi.call("mi_moe_kmajor_up", x, capi.ptr(x), capi.ptr(gate_up_weight), capi.ptr(route_expert), capi.ptr(up_part), P, k,
              E, H, 2 * I, s_up, adt)
    s_dn = _km_splits(P, I, H, dev)
    dn_part = torch.empty(P, s_dn, H, dtype=torch.float32, device=dev)
    capi.call("mi_moe_kmajor_down", x, capi.ptr(up_part), s_up, capi.ptr(gate_up_scale.contiguous()), capi.ptr(down_weight),
              capi.ptr(route_expert), capi.ptr(dn_part), P, E, I, H, s_dn, 0, adt)
    shared = None
    if S > 0:
        _chk(S == 1, f"{who}: one shared expert is supported")
        _chk_fp8(shared_gate_up_weight, who)
        _chk_fp8(shared_down_weight, who)
        _chk(shared_gate_up_weight.numel() == 2 * I * H and shared_down_weight.numel() == H * I,
             f"{who}: shared weights must be [1, 2*I, H] and [1, H, I]")
        _chk(shared_gate_up_scale.dtype == torch.float32 and shared_down_scale.dtype == torch.float32,
             f"{who}: shared scales must be float32")
        sh_gu = torch.empty(T, 2 * I, dtype=x.dtype, device=dev)
        esimd_gemm_fp8_pert(x, shared_gate_up_weight.reshape(2 * I, H), shared_gate_up_scale.reshape(-1)[:1], sh_gu)
        sh_inter = torch.empty(T, I, dtype=x.dtype, device=dev)
        esimd_moe_silu_mul(sh_gu, sh_inter, 2 * I, I, T)
        shared = torch.empty(T, H, dtype=x.dtype, device=dev)
        esimd_gemm_fp8_pert(sh_inter, shared_down_weight.reshape(H, I), shared_down_scale.reshape(-1)[:1], shared)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    capi.call("mi_moe_kmajor_finalize", x, capi.ptr(dn_part), s_dn, capi.ptr(down_scale.contiguous()), capi.ptr(route_expert),
              capi.ptr(top_w), capi.ptr(shared), capi.ptr(gate), capi.ptr(out), T, k, E, H, adt)
    return out


def w4a16_prepare(qweight, scales, qzeros, group_size, zero_bias=0):
    """GPTQ / AWQ style operands -> (weight [N, K/8] int32, scale [N, K/128] fp16, zp [N, K/128] uint8),
    the resident layout of esimd_gemm_int4_pgrp_zp / esimd_gemv_int4, converted on the device.
    qweight: logical [K/8, N] int32, either contiguous or with strides (1, K/8) (then its bytes are
    used as they are); scales [K/128, N] fp16; qzeros: [K/128, N/8] int32 packed along N, or a
    one-element tensor holding the zero-point of every group (the symmetric case: 8)."""
    who = "w4a16_prepare"
    _chk(int(group_size) == 128, f"{who}: only group_size 128 is supported, got {group_size}")
    _chk(qweight.dim() == 2 and qweight.dtype == torch.int32, f"{who}: qweight must be int32 [K/8, N]")
    K8, N = qweight.shape
    K = K8 * 8
    _chk(K % 128 == 0, f"{who}: K={K} must be a multiple of 128")
    G = K // 128
    _chk(scales.dtype == torch.float16 and scales.is_contiguous() and tuple(scales.shape) == (G, N),
         f"{who}: scales must be contiguous fp16 [K/128, N]")
    scalar = qzeros.numel() == 1
    _chk(qzeros.dtype == torch.int32 and qzeros.is_contiguous(), f"{who}: qzeros must be contiguous int32")
    _chk(scalar or (N % 8 == 0 and tuple(qzeros.shape) == (G, N // 8)),
         f"{who}: qzeros must be [K/128, N/8] int32 (N a multiple of 8) or hold one value")
    dev = qweight.device
    n_major = qweight.stride() == (1, K8) or N == 1
    _chk(n_major or qweight.is_contiguous(), f"{who}: qweight must be contiguous or have strides (1, K/8)")
    w_out = qweight.t() if n_major else torch.empty(N, K8, dtype=torch.int32, device=dev)
    s_out = torch.empty(N, G, dtype=torch.float16, device=dev)
    zp_out = torch.empty(N, G, dtype=torch.uint8, device=dev)
    capi.call("mi_w4a16_kmajor_prepare", scales, None if n_major else capi.ptr(qweight), capi.ptr(scales), capi.ptr(qzeros),
              1 if scalar else 0, int(zero_bias), None if n_major else capi.ptr(w_out), capi.ptr(s_out), capi.ptr(zp_out), N, K)
    return w_out, s_out, zp_out


def _w4a16_prepare_meta(qweight, scales, qzeros, group_size, zero_bias=0):
    K8, N = qweight.shape
    G = K8 * 8 // 128
    return (qweight.new_empty(N, K8), scales.new_empty(N, G), scales.new_empty(N, G, dtype=torch.uint8))


def int4_gemm_w4a16(x, qweight, bias, scales, qzeros, group_size, g_idx):
    """The call the reference's GPTQ / AWQ / sym_int4 linears make
    (vllm/patches/vllm_for_multi_arc.patch:5492-5500): out[M, N] = x @ ((q - z) * s) + bias, output
    allocated here.  The operands are converted per call (the weight only when it is not already
    N-major in memory); a loader that calls w4a16_prepare once and esimd_gemm_int4_pgrp_zp per
    step skips that."""
    who = "int4_gemm_w4a16"
    _chk(g_idx is None, f"{who}: activation reordering (g_idx) is not supported")
    _chk(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous(),
         f"{who}: x must be contiguous fp16 / bf16 [M, K]")
    w, s, zp = w4a16_prepare(qweight, scales, qzeros, group_size)
    M, N = x.shape[0], w.shape[0]
    _chk(x.shape[1] == w.shape[1] * 8, f"{who}: x has K={x.shape[1]}, the weight K={w.shape[1] * 8}")
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    _gemm_int4(x, w.contiguous() if not w.is_contiguous() else w, s, zp, out, who)
    if bias is not None:
        _chk(bias.dtype == x.dtype and bias.is_contiguous() and bias.numel() == N, f"{who}: bias must be [N] in x's dtype")
        capi.call("mi_add_bias", out, capi.ptr(out), capi.ptr(bias), M, N, capi.act_dtype(x))
    return out


def _int4_gemm_w4a16_meta(x, qweight, bias, scales, qzeros, group_size, g_idx):
    return x.new_empty(x.shape[0], qweight.shape[1])


def register_xpu_c_alias():
    """Also registers int4_gemm_w4a16 as torch.ops._xpu_C.int4_gemm_w4a16, the name the reference's
    GPTQ / AWQ / sym_int4 linears call (vllm/patches/vllm_for_multi_arc.patch:5492).  Opt-in, because
    `_xpu_C` is another package's namespace: call it only where that package is not installed."""
    if "_xpu_C" in _DEFINED and "int4_gemm_w4a16" in _DEFINED["_xpu_C"]:
        return
    _define("_xpu_C", "int4_gemm_w4a16(Tensor x, Tensor qweight, Tensor? bias, Tensor scales, Tensor qzeros, "
                      "int group_size, Tensor? g_idx) -> Tensor", int4_gemm_w4a16, _int4_gemm_w4a16_meta)


def moe_forward_full_v2(*args):
    """The reference's variant for more than one token (V/csrc/moe_batch/moe.sycl:2337-2430): same
    arguments and result as moe_forward_full; one implementation serves both here."""
    return moe_forward_full(*args)


# --------------------------------------------------------------------------
# registration
# --------------------------------------------------------------------------
def _ret(idx):
    """Meta implementation: the op returns its pre-allocated output argument."""
    return lambda *a: a[idx]


_V = "custom_esimd_kernels_vllm"
_S = "custom_esimd_kernels_sglang"

_registered = False


def register():
    global _registered
    if _registered:
        return
    _registered = True
    for ns in (_V, _S):
        _define(ns, "esimd_gemv_fp8_pern(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output, int N, int K) -> Tensor", esimd_gemv_fp8_pern, _ret(3))
        _define(ns, "esimd_gemv_fp8_pern_fused2(Tensor input, Tensor w0, Tensor s0, Tensor o0, int N0, "
                    "Tensor w1, Tensor s1, Tensor o1, int N1, int K) -> Tensor", esimd_gemv_fp8_pern_fused2, _ret(3))
        _define(ns, "esimd_gemv_fp8_pern_fused3(Tensor input, Tensor w0, Tensor s0, Tensor o0, int N0, "
                    "Tensor w1, Tensor s1, Tensor o1, int N1, Tensor w2, Tensor s2, Tensor o2, int N2, "
                    "int K) -> Tensor", esimd_gemv_fp8_pern_fused3, _ret(3))
        _define(ns, "esimd_gemv_fp8_pert(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemv_fp8_pert, _ret(3))
        _define(ns, "esimd_gemv_fp8_pert_bmg(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemv_fp8_pert_bmg, _ret(3))
        _define(ns, "esimd_gemv_fp8_pert_fused2(Tensor input, Tensor w0, Tensor s0, Tensor o0, "
                    "Tensor w1, Tensor s1, Tensor o1) -> Tensor", esimd_gemv_fp8_pert_fused2, _ret(3))
        _define(ns, "esimd_gemv_fp8_pert_fused3(Tensor input, Tensor w0, Tensor s0, Tensor o0, "
                    "Tensor w1, Tensor s1, Tensor o1, Tensor w2, Tensor s2, Tensor o2) -> Tensor",
                esimd_gemv_fp8_pert_fused3, _ret(3))
        _define(ns, "esimd_gemv_int4(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemv_int4, _ret(3))
        _define(ns, "esimd_gemv_int4_fused2(Tensor input, Tensor w0, Tensor s0, Tensor o0, "
                    "Tensor w1, Tensor s1, Tensor o1) -> Tensor", esimd_gemv_int4_fused2, _ret(3))
    # the reference registers its GEMM fragment under the vllm namespace, and in the
    # sglang fork under `custom_esimd_kernels`
    for ns in (_V, "custom_esimd_kernels"):
        _define(ns, "esimd_gemm_int4_pgrp(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemm_int4_pgrp, _ret(3))
        _define(ns, "esimd_gemm_int4_pgrp_zp(Tensor input, Tensor weight, Tensor weight_scale, Tensor weight_zp, "
                    "Tensor(a!) output) -> Tensor(a!)", esimd_gemm_int4_pgrp_zp, _ret(4))
        _define(ns, "int4_gemm_w4a16(Tensor x, Tensor qweight, Tensor? bias, Tensor scales, Tensor qzeros, "
                    "int group_size, Tensor? g_idx) -> Tensor", int4_gemm_w4a16, _int4_gemm_w4a16_meta)
        _define(ns, "w4a16_prepare(Tensor qweight, Tensor scales, Tensor qzeros, int group_size, int zero_bias=0) "
                    "-> (Tensor, Tensor, Tensor)", w4a16_prepare, _w4a16_prepare_meta)
        _define(ns, "esimd_gemm_fp8_pert(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemm_fp8_pert, _ret(3))
        _define(ns, "esimd_gemm_fp8_blockscale(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output, int block_n, int block_k) -> Tensor", esimd_gemm_fp8_blockscale, _ret(3))
        _define(ns, "esimd_gemv_fp16(Tensor input, Tensor weight, Tensor output) -> Tensor", esimd_gemv_fp16, _ret(2))
        _define(ns, "esimd_gemv_fp16_gelu_mul(Tensor input, Tensor weight, Tensor output) -> Tensor",
                esimd_gemv_fp16_gelu_mul, _ret(2))
        _define(ns, "esimd_gemv_fp8_blockscale_fp16_fused2(Tensor input, Tensor w0, Tensor s0, Tensor(a!) o0, "
                    "Tensor w1, Tensor(b!) o1, int block_n, int block_k) -> Tensor(a!)",
                esimd_gemv_fp8_blockscale_fp16_fused2, _ret(3))
        _define(ns, "esimd_gemv_fp8_blockscale_fused2(Tensor input, Tensor w0, Tensor s0, Tensor(a!) o0, "
                    "Tensor w1, Tensor s1, Tensor(b!) o1, int block_n, int block_k) -> Tensor(a!)",
                esimd_gemv_fp8_blockscale_fused2, _ret(3))
    for ns in (_V, _S):
        _define(ns, "esimd_rms_norm(Tensor input, Tensor output, Tensor weight, float eps) -> Tensor", esimd_rms_norm, _ret(1))
        _define(ns, "esimd_fused_add_rms_norm(Tensor hidden_states, Tensor residual, Tensor weight, float eps) -> Tensor",
                esimd_fused_add_rms_norm, _ret(0))
        _define(ns, "esimd_fused_scaled_add_rms_norm(Tensor hidden_states, Tensor residual, Tensor weight, float eps, "
                    "float scalar) -> Tensor", esimd_fused_scaled_add_rms_norm, _ret(0))
        _define(ns, "esimd_rms_norm_gated(Tensor x, Tensor z, Tensor weight, Tensor output, float eps) -> Tensor",
                esimd_rms_norm_gated, _ret(3))
        _define(ns, "esimd_fused_add_rms_norm_batched(Tensor hidden_states, Tensor residual, Tensor weight, float eps) -> Tensor",
                esimd_fused_add_rms_norm_batched, _ret(0))
        _define(ns, "esimd_resadd_norm_gemv_int4_pert(Tensor hidden_states, Tensor residual, Tensor norm_weight, "
                    "Tensor gemv_weight, Tensor gemv_scale, Tensor output, Tensor normed_out, float eps) -> Tensor",
                esimd_resadd_norm_gemv_int4_pert, _ret(5))
        _define(ns, "esimd_resadd_norm_gemv_fp8_pert(Tensor hidden_states, Tensor residual, Tensor norm_weight, "
                    "Tensor gemv_weight, Tensor gemv_scale, Tensor output, Tensor normed_out, float eps) -> Tensor",
                esimd_resadd_norm_gemv_fp8_pert, _ret(5))
        _define(ns, "esimd_scaled_resadd_norm_gemv_fp8_pert(Tensor hidden_states, Tensor residual, Tensor norm_weight, "
                    "Tensor qkv_weight, Tensor qkv_scale, Tensor qkv_out, float eps, float scalar) -> ()",
                esimd_scaled_resadd_norm_gemv_fp8_pert, lambda *a: None)
        _define(ns, "esimd_norm_gemv_norm_fp16(Tensor residual, Tensor scale_with_root, Tensor proj_w, Tensor pre_ff_w, "
                    "Tensor router_logits, Tensor moe_input, float eps) -> ()", esimd_norm_gemv_norm_fp16, lambda *a: None)
        _define(ns, "esimd_norm_add_norm(Tensor h2_raw, Tensor h1, Tensor w1, Tensor w2, Tensor out, float eps1, "
                    "float eps2) -> ()", esimd_norm_add_norm, lambda *a: None)
        _define(ns, "esimd_accum_norm_add_norm(Tensor routed_output, Tensor h1, Tensor w1, Tensor w2, Tensor out, "
                    "int top_k, float eps1, float eps2) -> ()", esimd_accum_norm_add_norm, lambda *a: None)
        _define(ns, "esimd_resadd_norm_gemv2_fp8_pert(Tensor hidden_states, Tensor residual, Tensor norm_weight, "
                    "Tensor w0, Tensor s0, Tensor o0, Tensor w1, Tensor s1, Tensor o1, float eps) -> Tensor",
                esimd_resadd_norm_gemv2_fp8_pert, _ret(5))
        _define(ns, "esimd_norm_gemv_int4_pert(Tensor x, Tensor z, Tensor norm_weight, Tensor gemv_weight, "
                    "Tensor gemv_scale, Tensor output, int HV, int V, float eps) -> Tensor", esimd_norm_gemv_int4_pert, _ret(5))
        _define(ns, "esimd_norm_gemv_fp8_pert(Tensor x, Tensor z, Tensor norm_weight, Tensor gemv_weight, "
                    "Tensor gemv_scale, Tensor output, int HV, int V, float eps) -> Tensor", esimd_norm_gemv_fp8_pert, _ret(5))
    _define(_V, "esimd_norm_gemv_fp8_blockscale(Tensor x, Tensor z, Tensor norm_weight, Tensor gemv_weight, "
                "Tensor gemv_scale, Tensor(a!) output, int HV, int V, float eps) -> Tensor(a!)",
            esimd_norm_gemv_fp8_blockscale, _ret(5))
    _define(_S, "esimd_gemv_q4_k(Tensor input, Tensor weight, Tensor weight_scale, "
                "Tensor weight_min, Tensor output) -> Tensor", esimd_gemv_q4_k, _ret(4))
    # siblings without a reference counterpart
    _define(_S, "q4_k_repack(Tensor qweight, Tensor(a!) ql, Tensor(b!) weight_scale, "
                "Tensor(c!) weight_min) -> Tensor(a!)", q4_k_repack, _ret(1))
    _define(_S, "q4_k_dequant(Tensor weight, Tensor weight_scale, Tensor weight_min, "
                "Tensor(a!) output) -> Tensor(a!)", q4_k_dequant, _ret(3))
    # other GGUF formats (S/csrc/xpu/torch_extension.cc:48-106) and their weight preparation
    _define(_S, "esimd_gemv_q4_0(Tensor input, Tensor weight, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemv_q4_0, _ret(3))
    _define(_S, "esimd_gemm_q4_0(Tensor input, Tensor weight, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemm_q4_0, _ret(3))
    _define(_S, "esimd_gemv_q8_0(Tensor input, Tensor weight, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemv_q8_0, _ret(3))
    _define(_S, "esimd_gemv_q8_0_m(Tensor input, Tensor weight, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemv_q8_0_m, _ret(3))
    _define(_S, "esimd_moe_up_q4k(Tensor x, Tensor gate_ql, Tensor gate_sc, Tensor gate_mn, Tensor up_ql, Tensor up_sc, "
                "Tensor up_mn, Tensor sel, Tensor inter, int n_tokens, int hidden, int intermediate, int top_k) -> Tensor",
            esimd_moe_up_q4k, _ret(8))
    _define(_S, "esimd_moe_down_q5k(Tensor inter, Tensor ql, Tensor qh, Tensor sc, Tensor mn, Tensor sel, Tensor topk_w, "
                "Tensor out_partial, int n_tokens, int hidden, int intermediate, int top_k) -> Tensor",
            esimd_moe_down_q5k, _ret(7))
    _define(_S, "esimd_moe_down_q6k(Tensor inter, Tensor ql, Tensor qh, Tensor sc, Tensor sel, Tensor topk_w, "
                "Tensor out_partial, int n_tokens, int hidden, int intermediate, int top_k) -> Tensor",
            esimd_moe_down_q6k, _ret(6))
    _define(_S, "esimd_gemv_q5_k(Tensor input, Tensor ql, Tensor qh, Tensor weight_scale, Tensor weight_min, "
                "Tensor output) -> Tensor", esimd_gemv_q5_k, _ret(5))
    _define(_S, "esimd_gemv_q6_k(Tensor input, Tensor ql, Tensor qh, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemv_q6_k, _ret(4))
    _define(_S, "esimd_gemv_q6_k_m(Tensor input, Tensor ql, Tensor qh, Tensor weight_scale, Tensor output) -> Tensor",
            esimd_gemv_q6_k_m, _ret(4))
    _define(_S, "q4_0_repack(Tensor qweight, Tensor(a!) weight, Tensor(b!) weight_scale) -> Tensor(a!)", q4_0_repack, _ret(1))
    _define(_S, "q8_0_repack(Tensor qweight, Tensor(a!) weight, Tensor(b!) weight_scale) -> Tensor(a!)", q8_0_repack, _ret(1))
    _define(_S, "q5_k_repack(Tensor qweight, Tensor(a!) ql, Tensor(b!) qh, Tensor(c!) weight_scale, "
                "Tensor(d!) weight_min) -> Tensor(a!)", q5_k_repack, _ret(1))
    _define(_S, "q6_k_repack(Tensor qweight, Tensor(a!) ql, Tensor(b!) qh, Tensor(c!) weight_scale) -> Tensor(a!)",
            q6_k_repack, _ret(1))
    _define(_S, "q5_k_repack_plain(Tensor qweight, Tensor(a!) ql, Tensor(b!) qh, Tensor(c!) weight_scale, "
                "Tensor(d!) weight_min) -> Tensor(a!)", q5_k_repack_plain, _ret(1))
    _define(_S, "q6_k_repack_plain(Tensor qweight, Tensor(a!) ql, Tensor(b!) qh, Tensor(c!) weight_scale) -> Tensor(a!)",
            q6_k_repack_plain, _ret(1))
    _define(_S, "q4_0_dequant(Tensor weight, Tensor weight_scale, Tensor(a!) output) -> Tensor(a!)", q4_0_dequant, _ret(2))
    _define(_S, "q8_0_dequant(Tensor weight, Tensor weight_scale, Tensor(a!) output) -> Tensor(a!)", q8_0_dequant, _ret(2))
    _define(_S, "q5_k_dequant(Tensor ql, Tensor qh, Tensor weight_scale, Tensor weight_min, Tensor(a!) output) -> Tensor(a!)",
            q5_k_dequant, _ret(4))
    _define(_S, "q6_k_dequant(Tensor ql, Tensor qh, Tensor weight_scale, Tensor(a!) output) -> Tensor(a!)",
            q6_k_dequant, _ret(3))
    _define(_V, "q4_0_quantize(Tensor input, Tensor(a!) out_qweight, Tensor(b!) out_scale) -> ()", q4_0_quantize,
            lambda *a: None)
    _define(_V, "int4_dequant(Tensor weight, Tensor weight_scale, Tensor? weight_zp, "
                "Tensor(a!) output) -> Tensor(a!)", int4_dequant, _ret(3))
    _define(_V, "fp8_dequant(Tensor weight, Tensor weight_scale, Tensor(a!) output, str mode) -> Tensor(a!)",
            fp8_dequant, _ret(2))
    _define(_V, "e4m3_decode(Tensor codes, Tensor(a!) output) -> Tensor(a!)", e4m3_decode, _ret(1))

    # ---- MoE (reference fragment torch_extension_moe.cc + moe_ops + sglang prefill ops)
    for ns in (_V, _S):
        _define(ns, "esimd_moe_topk(Tensor router_logits, Tensor top_values, Tensor top_indices, int T) -> Tensor",
                esimd_moe_topk, _ret(1))
        _define(ns, "esimd_moe_scatter(Tensor hidden_states, Tensor router_top_value, Tensor sorted_token_ids, "
                    "Tensor scattered_hidden, Tensor scattered_weights, int K, int topk, int total_expanded) -> Tensor",
                esimd_moe_scatter, _ret(3))
        _define(ns, "esimd_moe_scatter_fused(Tensor hidden_states, Tensor top_values, Tensor top_indices, "
                    "Tensor scattered_hidden, Tensor scattered_weights, Tensor topk_ids, Tensor expert_start, "
                    "Tensor max_tokens_out, int K, int topk, int T, int num_experts) -> Tensor",
                esimd_moe_scatter_fused, _ret(3))
        _define(ns, "esimd_moe_silu_mul(Tensor input, Tensor output, int N_gate_up, int N_half, int total_rows) -> Tensor",
                esimd_moe_silu_mul, _ret(1))
        _define(ns, "esimd_moe_gelu_tanh_mul(Tensor input, Tensor output, int N_gate_up, int N_half, int total_rows) -> Tensor",
                esimd_moe_gelu_tanh_mul, _ret(1))
        _define(ns, "esimd_moe_gather(Tensor moe_output, Tensor topk_ids, Tensor scattered_weights, "
                    "Tensor final_hidden, int K, int topk, int T) -> Tensor", esimd_moe_gather, _ret(3))
    _define(_V, "esimd_moe_gemm_fp8_blockscale(Tensor input, Tensor weight, Tensor weight_scale, Tensor(a!) output, "
                "Tensor expert_idx, int N, int K, int num_experts, int block_n, int block_k) -> Tensor(a!)",
            esimd_moe_gemm_fp8_blockscale, _ret(3))
    _define("moe_ops", "moe_topk(Tensor logits, int top_k, bool norm) -> (Tensor, Tensor)", moe_topk,
            lambda logits, top_k, norm: (logits.new_empty(logits.shape[0], top_k),
                                         logits.new_empty(logits.shape[0], top_k, dtype=torch.int32)))
    _define("moe_ops", "moe_forward_full_fp8_block(Tensor x, Tensor logits, Tensor(a!) output, Tensor gate_up_weight, "
                       "Tensor gate_up_scale, Tensor shared_gate_up_weight, Tensor shared_gate_up_scale, "
                       "Tensor down_weight, Tensor down_scale, Tensor shared_down_weight, Tensor shared_down_scale, "
                       "Tensor shared_expert_gate_weight, int top_k, int num_shared_experts, "
                       "int n_routed_experts) -> Tensor(a!)", moe_forward_full_fp8_block, _ret(2))
    _define("moe_int4_prefill_ops", "moe_prefill_gather_forward_v2(Tensor selected_experts, int num_experts) -> Tensor[]",
            moe_prefill_gather_forward_v2,
            lambda sel, e: [sel.new_empty(e), sel.new_empty(sel.numel()), sel.new_empty(sel.numel()), sel.new_empty(e)])
    _define("moe_int4_prefill_ops", "moe_topk_softmax(Tensor router_logits, int top_k, int num_experts) -> Tensor[]",
            moe_topk_softmax,
            lambda l, k, e: [l.new_empty(l.shape[0], k), l.new_empty(l.shape[0], k, dtype=torch.int32)])
    _define("esimd_topk_v2", "topk_v2(Tensor router_logits, Tensor top_values, Tensor top_indices, int T, "
            "int num_experts, int topk) -> Tensor", topk_v2, _ret(1))
    _define("moe_ops", "moe_router_forward(Tensor x, Tensor weight, Tensor scale) -> Tensor", moe_router_forward,
            lambda x, w, s: x.new_empty(x.shape[0], w.shape[0]))
    _define("moe_ops", "moe_accumulate(Tensor partials, int top_k, int num_shared_experts) -> Tensor", moe_accumulate,
            lambda p, k, n: p.new_empty(p.shape[0] // (k + n), p.shape[1]))
    _pert = ("Tensor gate_up_weight, Tensor gate_up_scale, Tensor down_weight, Tensor down_scale, "
             "int top_k, int n_routed_experts) -> Tensor")
    _define("moe_ops", "moe_forward_full_gelu_tanh(Tensor x, Tensor logits, " + _pert, moe_forward_full_gelu_tanh,
            lambda x, *a: torch.empty_like(x))
    for name, fn in (("moe_forward_full_gelu_tanh_routed", moe_forward_full_gelu_tanh_routed),
                     ("moe_forward_full_gelu_tanh_routed_decode", moe_forward_full_gelu_tanh_routed_decode)):
        _define("moe_ops", name + "(Tensor x, Tensor topk_weights, Tensor topk_indices, " + _pert, fn,
                lambda x, *a: torch.empty_like(x))
    for name, fn in (("moe_forward_full_silu_routed", moe_forward_full_silu_routed),
                     ("moe_forward_full_silu_routed_sglang", moe_forward_full_silu_routed_sglang)):
        _define("moe_ops", name + "(Tensor x, Tensor topk_weights, Tensor topk_indices, " + _pert, fn,
                lambda x, *a: torch.empty_like(x))
    _define("moe_ops", "moe_forward_full_gelu_tanh_routed_no_accum(Tensor x, Tensor topk_weights, Tensor topk_indices, "
            + _pert, moe_forward_full_gelu_tanh_routed_no_accum,
            lambda x, tw, *a: x.new_empty(tw.numel(), x.shape[1]))
    _define("moe_ops", "moe_forward_full_gelu_tanh_decode(Tensor x, Tensor logits, Tensor gate_up_weight, "
            "Tensor gate_up_scale, Tensor down_weight, Tensor down_scale, Tensor per_expert_scale, int top_k, "
            "int n_routed_experts) -> Tensor", moe_forward_full_gelu_tanh_decode, lambda x, *a: torch.empty_like(x))
    _full = ("(Tensor x, Tensor logits, Tensor gate_up_weight, Tensor gate_up_scale, Tensor shared_gate_up_weight, "
             "Tensor shared_gate_up_scale, Tensor down_weight, Tensor down_scale, Tensor shared_down_weight, "
             "Tensor shared_down_scale, Tensor shared_expert_gate_weight, int top_k, int num_shared_experts, "
             "int n_routed_experts) -> Tensor")
    _define("moe_ops", "moe_forward_full" + _full, moe_forward_full, lambda x, *a: torch.empty_like(x))
    _define("moe_ops", "moe_forward_full_v2" + _full, moe_forward_full_v2, lambda x, *a: torch.empty_like(x))
    _define("moe_ops", "moe_up_fp8_grouped(Tensor x, Tensor gate_up_weight, Tensor gate_up_scale, Tensor expert_offsets, "
            "Tensor expert_tokens, int top_k, int n_routed_experts) -> Tensor", moe_up_fp8_grouped,
            lambda x, w, s, eo, et, k, e: x.new_empty(et.numel(), w.shape[1] // 2))
    _define("moe_ops", "moe_down_fp8_grouped(Tensor intermediate, Tensor down_weight, Tensor down_scale, "
            "Tensor routing_weights, Tensor expert_offsets, Tensor expert_tokens, int top_k, int n_routed_experts) -> Tensor",
            moe_down_fp8_grouped, lambda i, w, *a: i.new_empty(i.shape[0], w.shape[1]))
    _define("moe_ops", "moe_forward_full_fp8_grouped(Tensor x, Tensor gate_up_weight, Tensor gate_up_scale, "
            "Tensor down_weight, Tensor down_scale, Tensor routing_weights, Tensor expert_offsets, Tensor expert_tokens, "
            "int top_k, int n_routed_experts) -> Tensor", moe_forward_full_fp8_grouped, lambda x, *a: torch.empty_like(x))
    _define("moe_fp8_prefill_ops", "moe_prefill_gather_forward_fp8(Tensor selected_experts, int num_experts) -> Tensor[]",
            moe_prefill_gather_forward_fp8,
            lambda sel, e: [sel.new_empty(e), sel.new_empty(sel.numel()), sel.new_empty(sel.numel()), sel.new_empty(e)])
    _define("moe_fp8_prefill_ops", "moe_prefill_full_fp8(Tensor hidden_states, Tensor topk_weights, Tensor topk_ids, "
            "Tensor w13, Tensor w13_scale, Tensor w2, Tensor w2_scale, int top_k, int num_experts) -> Tensor",
            moe_prefill_full_fp8, lambda h, *a: torch.empty_like(h))
    _define("moe_fp8_prefill_ops", "moe_prefill_up_forward_fp8(Tensor x, Tensor gate_up_weight, Tensor gate_up_scale, "
            "Tensor expert_offsets, Tensor expert_tokens, int top_k) -> Tensor", moe_prefill_up_forward_fp8,
            lambda x, w, s, eo, et, k: x.new_empty(et.numel(), w.shape[1] // 2))
    _define("moe_fp8_prefill_ops", "moe_prefill_down_forward_fp8(Tensor intermediate, Tensor down_weight, "
            "Tensor down_scale, Tensor expert_offsets, Tensor expert_tokens) -> Tensor", moe_prefill_down_forward_fp8,
            lambda i, w, s, eo, et: i.new_empty(et.numel(), w.shape[1]))
    _define("moe_fp8_prefill_ops", "moe_prefill_accumulate_forward_fp8(Tensor output, Tensor routing_weights) -> Tensor",
            moe_prefill_accumulate_forward_fp8, lambda o, w: o.new_empty(w.shape[0], o.shape[1]))
    # siblings without a reference counterpart
    _define(_V, "moe_sort(Tensor top_ids, int num_experts, Tensor(a!) sorted_pairs, Tensor(b!) expert_start, "
                "Tensor(c!) inv, Tensor(d!)? sorted_token, Tensor(e!)? max_count) -> Tensor(a!)", moe_sort, _ret(2))
    _define(_V, "act_quant_fp8(Tensor x, Tensor(a!) q, Tensor(b!) scale) -> Tensor(a!)", act_quant_fp8, _ret(1))
    _define(_V, "moe_gemm_fp8_block(Tensor a, Tensor? a_scale, Tensor? row_map, Tensor weight, Tensor weight_scale, "
                "Tensor expert_start, Tensor(a!) output, int N, int K, int num_experts, bool fuse_silu_mul) -> Tensor(a!)",
            moe_gemm_fp8_block, _ret(6))
    _define(_V, "moe_gate_up_fp8_routed(Tensor xq, Tensor xs, Tensor top_ids, Tensor weight, Tensor weight_scale, "
                "Tensor(b!) expert_start, Tensor(c!) inv, Tensor(d!)? sorted_pairs, Tensor(a!) output, "
                "int num_experts) -> Tensor(a!)", moe_gate_up_fp8_routed, _ret(8))
    _define(_V, "moe_combine(Tensor y, Tensor inv, Tensor top_w, Tensor(a!) output, int top_k) -> Tensor(a!)",
            moe_combine, _ret(3))
    _define(_V, "moe_forward_fp8_block(Tensor x, Tensor logits, Tensor gate_up_weight, Tensor gate_up_scale, "
                "Tensor down_weight, Tensor down_scale, Tensor(a!) output, int top_k, bool act_quant) -> Tensor(a!)",
            moe_forward_fp8_block, _ret(6))


register()
