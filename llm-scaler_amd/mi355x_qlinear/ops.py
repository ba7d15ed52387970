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

import torch

from . import capi

_FP8_TYPES = (torch.float8_e4m3fn, torch.uint8)

_libs = {}


def _library(ns: str) -> torch.library.Library:
    if ns not in _libs:
        _libs[ns] = torch.library.Library(ns, "FRAGMENT")
    return _libs[ns]


def _define(ns: str, schema: str, impl, meta=None):
    lib = _library(ns)
    lib.define(schema)
    name = schema.split("(", 1)[0]
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
        _define(ns, "esimd_gemm_fp8_pert(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output) -> Tensor", esimd_gemm_fp8_pert, _ret(3))
        _define(ns, "esimd_gemm_fp8_blockscale(Tensor input, Tensor weight, Tensor weight_scale, "
                    "Tensor output, int block_n, int block_k) -> Tensor", esimd_gemm_fp8_blockscale, _ret(3))
        _define(ns, "esimd_gemv_fp8_blockscale_fused2(Tensor input, Tensor w0, Tensor s0, Tensor(a!) o0, "
                    "Tensor w1, Tensor s1, Tensor(b!) o1, int block_n, int block_k) -> Tensor(a!)",
                esimd_gemv_fp8_blockscale_fused2, _ret(3))
    _define(_S, "esimd_gemv_q4_k(Tensor input, Tensor weight, Tensor weight_scale, "
                "Tensor weight_min, Tensor output) -> Tensor", esimd_gemv_q4_k, _ret(4))
    # siblings without a reference counterpart
    _define(_S, "q4_k_repack(Tensor qweight, Tensor(a!) ql, Tensor(b!) weight_scale, "
                "Tensor(c!) weight_min) -> Tensor(a!)", q4_k_repack, _ret(1))
    _define(_S, "q4_k_dequant(Tensor weight, Tensor weight_scale, Tensor weight_min, "
                "Tensor(a!) output) -> Tensor(a!)", q4_k_dequant, _ret(3))
    _define(_V, "int4_dequant(Tensor weight, Tensor weight_scale, Tensor? weight_zp, "
                "Tensor(a!) output) -> Tensor(a!)", int4_dequant, _ret(3))
    _define(_V, "fp8_dequant(Tensor weight, Tensor weight_scale, Tensor(a!) output, str mode) -> Tensor(a!)",
            fp8_dequant, _ret(2))
    _define(_V, "e4m3_decode(Tensor codes, Tensor(a!) output) -> Tensor(a!)", e4m3_decode, _ret(1))


register()
