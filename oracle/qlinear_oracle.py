"""CPU oracle for the quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the arithmetic that the reference's own tests
and torch fallback paths define for the quantized-linear ops.  It exists to
check the HIP kernels; nothing in the product package imports it.  Only the
test-suite, the smoke check and the CPU-baseline leg of the benchmark may use it.

Every function cites the reference text it follows (paths relative to the
reference checkout; V/ = vllm/custom-esimd-kernels-vllm, S/ =
sglang/custom-esimd-kernels, SP = sglang/patches/sglang_for_multi_arc.patch,
VP = vllm/patches/vllm_for_multi_arc.patch).

Pinning status (see tests/test_oracle_*.py):
  * E4M3 decode: closed form below vs torch.float8_e4m3fn for all 256 codes, and
    the reference's all-codes known-answer construction.
  * int4 pack/unpack/dequant: brute force over all nibbles x scales, the
    reference's known-answer case (7,-7,3,-3 -> scale -0.875), uint8<->int32
    view identity.
  * Q4_K: all 64x64 (sc6, mn6) encodings of the 12-byte field, an independent
    straight-from-super-block dequant, a hand-built super-block fixture.
  * top-k / permutation: brute force on tiny inputs, invariants, a hand-checked
    4-token / 8-expert fixture.
  * per-token-per-128 activation quantisation (cfg3) and the asymmetric int4
    zero-point layout have NO counterpart in the reference: parity unpinned in
    the reference, pinned here only by their closed forms.
  * w4a16_kmajor_* (the operand layout of the third-party int4_gemm_w4a16 the
    reference calls for GPTQ / AWQ weights, VP:5492-5500): PARITY UNPINNED in the
    reference -- that op's source is not in the reference tree and no reference
    test exercises it.  Restated from the published GPTQ packing (eight nibbles
    per int32, lowest nibble first, along K for weights and along N for
    zero-points) and pinned by the reference's statement that its [K/8, N]
    tensor with strides (1, K/8) holds the same bytes as the ESIMD [N, K/2]
    weight (VP:5516-5523), hand-placed nibbles and a round trip.
"""
from __future__ import annotations

import numpy as np
import torch

FP8_MAX = 448.0          # float8_e4m3fn max finite magnitude
INT4_GROUP = 128         # V/csrc/xpu/esimd_kernels/int4_GEMV.h:69
FP8_BLOCK = 128          # V/csrc/xpu/esimd_kernel_gemm.sycl:104-126
Q4K_SB = 256             # SP:2521
Q4K_BYTES = 144          # SP:2522


# ----------------------------------------------------------------------------
# E4M3 (OCP float8_e4m3fn)
# ----------------------------------------------------------------------------
def e4m3_decode_table() -> np.ndarray:
    """All 256 E4M3 codes -> float32, closed form.

    Follows V/csrc/xpu/esimd_kernels/fp8_GEMM_blockscale.h:37-49 for the finite
    codes (sign, 4-bit exponent bias 7, 3-bit mantissa, subnormals m * 2^-9 kept,
    not flushed) and torch for the two NaN codes 0x7F / 0xFF.
    """
    out = np.empty(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 0x7
        if e == 0xF and m == 0x7:
            out[c] = np.nan
        elif e == 0:
            out[c] = s * m * 2.0 ** -9
        else:
            out[c] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


_E4M3_TABLE = e4m3_decode_table()


def e4m3_decode(codes: torch.Tensor) -> torch.Tensor:
    """uint8 / float8_e4m3fn tensor -> float32 (exact)."""
    if codes.dtype == torch.float8_e4m3fn:
        codes = codes.view(torch.uint8)
    assert codes.dtype == torch.uint8
    return torch.from_numpy(_E4M3_TABLE[codes.cpu().numpy()])


def e4m3_quantize(x_f32: torch.Tensor) -> torch.Tensor:
    """float32 -> E4M3 codes (uint8), round-to-nearest-even.

    The reference quantises with torch's cast, `(w / scale).to(float8_e4m3fn)`
    (V/tests/test_fp8_blockscale_gemm.py:24-27); this is that library routine.
    """
    return x_f32.to(torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)


# ----------------------------------------------------------------------------
# INT4, group 128, offset-binary nibbles  (cfg0, cfg2)
# ----------------------------------------------------------------------------
def int4_pack(q_signed: torch.Tensor) -> torch.Tensor:
    """signed int4 values [N, K] in [-8, 7] -> packed uint8 [N, K/2].

    Stored nibble = value + 8; low nibble = even k, high nibble = odd k
    (V/csrc/xpu/esimd_kernels/int4_GEMV.h:14-22, V/tests/test_gemv_int4.py:163-168).
    """
    u = (q_signed.to(torch.int32) + 8)
    assert int(u.min()) >= 0 and int(u.max()) <= 15
    return ((u[:, 0::2] & 0xF) | ((u[:, 1::2] & 0xF) << 4)).to(torch.uint8)


def int4_unpack_u4(packed: torch.Tensor) -> torch.Tensor:
    """packed uint8 [N, K/2] (or its int32 [N, K/8] view) -> stored nibbles [N, K] int32.

    The int32 view is the same bytes, little endian: nibble z of word i is
    element 8 i + z (V/tests/test_moe_int4_kernel.py:42-85, VP:5516).
    """
    if packed.dtype == torch.int32:
        packed = packed.contiguous().view(torch.uint8)
    assert packed.dtype == torch.uint8
    lo = (packed & 0xF).to(torch.int32)
    hi = ((packed >> 4) & 0xF).to(torch.int32)
    return torch.stack([lo, hi], dim=-1).reshape(packed.shape[0], -1)


def _round_to(x_f32: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return x_f32.to(dtype)


def int4_dequant(packed: torch.Tensor, scale: torch.Tensor, out_dtype=torch.float16,
                 zp: torch.Tensor | None = None, group: int = INT4_GROUP) -> torch.Tensor:
    """Dequantised weight [N, K] in `out_dtype`: rne(f32(u4 - z) * f32(scale)).

    Symmetric form (z == 8 implicit): V/tests/test_gemv_int4.py:172-212.
    Asymmetric form takes `zp` [N, K/group] uint8 with values 0..15; the reference
    has no ESIMD op with a zero-point operand, so that layout is this build's own.
    """
    u = int4_unpack_u4(packed).to(torch.float32)
    N, K = u.shape
    if zp is None:
        z = torch.full((N, K // group), 8.0)
    else:
        z = zp.to(torch.float32)
    z = z.repeat_interleave(group, dim=-1)
    s = scale.to(torch.float32).repeat_interleave(group, dim=-1)
    return _round_to((u - z) * s, out_dtype)


def w4a16_kmajor_pack(u4: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor):
    """Stored nibbles u4 [N, K] (0..15), scale [N, K/128] fp16, zp [N, K/128] (0..15) -> the operands
    of int4_gemm_w4a16 (VP:5492-5500): qweight [K/8, N] int32 with nibble z of word (i, n) = element
    k = 8 i + z of column n; scales [K/128, N] fp16; qzeros [K/128, N/8] int32 with nibble c of word
    (g, j) = zero-point of column n = 8 j + c in group g.  Parity unpinned in the reference (see the
    module header)."""
    N, K = u4.shape
    a = u4.to(torch.int64).numpy().reshape(N, K // 8, 8)
    words = np.zeros((N, K // 8), dtype=np.int64)
    for z in range(8):
        words |= a[:, :, z] << (4 * z)
    qweight = torch.from_numpy(words.astype(np.uint32).view(np.int32).T.copy())
    zz = zp.to(torch.int64).numpy().T.reshape(K // INT4_GROUP, N // 8, 8)
    zw = np.zeros((K // INT4_GROUP, N // 8), dtype=np.int64)
    for c in range(8):
        zw |= zz[:, :, c] << (4 * c)
    qzeros = torch.from_numpy(zw.astype(np.uint32).view(np.int32).copy())
    return qweight, scale.t().contiguous(), qzeros


def w4a16_kmajor_unpack(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor, zero_bias: int = 0):
    """Inverse of w4a16_kmajor_pack, element by element: (u4 [N, K] int32, scale [N, G] fp16,
    zp [N, G] uint8).  A one-element qzeros is the zero-point of every group (the symmetric case)."""
    K8, N = qweight.shape
    G = scales.shape[0]
    w = qweight.numpy().astype(np.int64) & 0xFFFFFFFF
    u4 = np.zeros((N, K8 * 8), dtype=np.int32)
    for i in range(K8):
        for z in range(8):
            u4[:, 8 * i + z] = (w[i, :] >> (4 * z)) & 0xF
    if qzeros.numel() == 1:
        zp = np.full((N, G), int(qzeros.reshape(-1)[0]), dtype=np.uint8)
    else:
        q = qzeros.numpy().astype(np.int64) & 0xFFFFFFFF
        zp = np.zeros((N, G), dtype=np.uint8)
        for n in range(N):
            zp[n, :] = ((q[:, n // 8] >> (4 * (n % 8))) & 0xF) + zero_bias
    return torch.from_numpy(u4), scales.t().contiguous(), torch.from_numpy(zp)


def w4a16_kmajor_dequant(qweight, scales, qzeros, out_dtype=torch.float16, zero_bias: int = 0) -> torch.Tensor:
    """Dense [N, K] weight of those operands: rne(f32(q - z) * f32(s)), the asymmetric form of int4_dequant."""
    u4, s, zp = w4a16_kmajor_unpack(qweight, scales, qzeros, zero_bias)
    z = zp.to(torch.float32).repeat_interleave(INT4_GROUP, dim=-1)
    sf = s.to(torch.float32).repeat_interleave(INT4_GROUP, dim=-1)
    return _round_to((u4.to(torch.float32) - z) * sf, out_dtype)


# ----------------------------------------------------------------------------
# FP8 weight-only dequant (cfg1, cfg3)
# ----------------------------------------------------------------------------
def fp8_dequant_per_channel(w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """[N, K] E4M3 + [N] scale -> float32 [N, K];  out[n] = s[n] * sum(x * w)
    (V/csrc/xpu/esimd_kernels/fp8_GEMV_v2.h:46-92; exact decode, no subnormal flush)."""
    return e4m3_decode(w8) * scale.to(torch.float32).reshape(-1, 1)


def fp8_dequant_per_tensor(w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """[N, K] E4M3 + scalar fp32 scale (V/csrc/xpu/esimd_kernels/fp8_GEMV_v2.h:291-337)."""
    return e4m3_decode(w8) * scale.to(torch.float32).reshape(())


def fp8_dequant_block(w8: torch.Tensor, scale: torch.Tensor, bn=FP8_BLOCK, bk=FP8_BLOCK, out_dtype=None) -> torch.Tensor:
    """[..., N, K] E4M3 + [..., ceil(N/bn), ceil(K/bk)] fp32 -> float32.

    V/tests/test_fp8_blockscale_gemm.py:31-36, V/tests/test_fp8_blockscale_moe_prefill.py:47-50.
    out_dtype (fp16 / bf16): the fp32 product rounded once to that type and returned as float32 —
    the dequantized weight of a prefill path that materialises 16-bit weights, as the reference's
    caller does for M >= 16 (`B.to(fp16) * Bs.to(fp16)`, vllm/patches/vllm_for_multi_arc.patch:2680-2682;
    here the scale stays fp32 and only the product is rounded).
    """
    n, k = w8.shape[-2:]
    wf = e4m3_decode(w8.reshape(-1, k)).reshape(w8.shape)
    full = scale.to(torch.float32).repeat_interleave(bn, -2).repeat_interleave(bk, -1)
    out = wf * full[..., :n, :k]
    return out if out_dtype is None else out.to(out_dtype).to(torch.float32)


def fp8_quantize_per_channel(w: torch.Tensor):
    """bf16/f32 [N, K] -> (codes uint8 [N, K], scale fp32 [N]); s = absmax / 448
    (V/tests/test_fp8_device_lost.py:31-36)."""
    w = w.to(torch.float32)
    s = (w.abs().amax(dim=1).clamp(min=1e-12) / FP8_MAX).to(torch.float32)
    return e4m3_quantize(w / s[:, None]), s


def fp8_quantize_block(w: torch.Tensor, bn=FP8_BLOCK, bk=FP8_BLOCK):
    """[..., N, K] -> (codes uint8, scale fp32 [..., Nb, Kb]), per 128x128 block
    s = absmax.clamp(1e-12) / 448  (V/tests/test_fp8_blockscale_gemm.py:13-28).
    N and K must be multiples of the block here (the configs are)."""
    w = w.to(torch.float32)
    lead = w.shape[:-2]
    n, k = w.shape[-2:]
    assert n % bn == 0 and k % bk == 0
    blk = w.reshape(*lead, n // bn, bn, k // bk, bk)
    amax = blk.abs().amax(dim=(-3, -1)).clamp(min=1e-12)        # [..., Nb, Kb]
    s = (amax / FP8_MAX).to(torch.float32)
    q = blk / s[..., :, None, :, None]
    return e4m3_quantize(q.reshape(w.shape)), s


def act_quant_per_token_group(x: torch.Tensor, group: int = 128):
    """Dynamic activation quantisation, per token per 128-wide K group (cfg3).

    s = max|x_g| / 448 in fp32 (clamped at 1e-12), q = (x_g / s) -> E4M3 RNE.
    Not present in the reference's ESIMD path (it is w8a16,
    V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:5-7): parity unpinned in
    the reference; the closed form mirrors V/tests/test_fp8_blockscale_gemm.py:22-25.
    Returns (codes uint8 [M, K], scale fp32 [M, K/group]).
    """
    xf = x.to(torch.float32)
    M, K = xf.shape
    g = xf.reshape(M, K // group, group)
    s = (g.abs().amax(dim=-1).clamp(min=1e-12) / FP8_MAX).to(torch.float32)
    q = e4m3_quantize((g / s[..., None]).reshape(M, K))
    return q, s


def act_dequant_per_token_group(q: torch.Tensor, s: torch.Tensor, group: int = 128) -> torch.Tensor:
    M, K = q.shape
    return (e4m3_decode(q).reshape(M, K // group, group) * s[..., None]).reshape(M, K)


# ----------------------------------------------------------------------------
# GEMV / GEMM result
# ----------------------------------------------------------------------------
def matmul_ref(x: torch.Tensor, w_deq: torch.Tensor) -> torch.Tensor:
    """x.float() @ w_deq.float().T, fp32 accumulate
    (V/tests/test_gemv_int4.py:232-233, V/tests/test_fp8_blockscale_gemm.py:46)."""
    return x.to(torch.float32) @ w_deq.to(torch.float32).t()


# ----------------------------------------------------------------------------
# GGUF Q4_K  (cfg4)
# ----------------------------------------------------------------------------
def q4k_pack_scales(sc6: np.ndarray, mn6: np.ndarray) -> np.ndarray:
    """8 six-bit scales + 8 six-bit mins -> the 12-byte field (inverse of
    get_scale_min_k4, SP:2549-2555)."""
    sc6 = sc6.astype(np.uint8)
    mn6 = mn6.astype(np.uint8)
    out = np.zeros(sc6.shape[:-1] + (12,), dtype=np.uint8)
    for j in range(4):
        out[..., j] = (sc6[..., j] & 63) | ((sc6[..., j + 4] >> 4) << 6)
        out[..., j + 4] = (mn6[..., j] & 63) | ((mn6[..., j + 4] >> 4) << 6)
        out[..., j + 8] = (sc6[..., j + 4] & 0xF) | ((mn6[..., j + 4] & 0xF) << 4)
    return out


def q4k_unpack_scales(sc12: np.ndarray):
    """get_scale_min_k4 for j = 0..7 (SP:2549-2555)."""
    s = sc12.astype(np.int32)
    sc6 = np.empty(s.shape[:-1] + (8,), dtype=np.int32)
    mn6 = np.empty_like(sc6)
    for j in range(8):
        if j < 4:
            sc6[..., j] = s[..., j] & 63
            mn6[..., j] = s[..., j + 4] & 63
        else:
            sc6[..., j] = (s[..., j + 4] & 0xF) | ((s[..., j - 4] >> 6) << 4)
            mn6[..., j] = (s[..., j + 4] >> 4) | ((s[..., j] >> 6) << 4)
    return sc6, mn6


def q4k_build_raw(q: np.ndarray, sc6: np.ndarray, mn6: np.ndarray,
                  d: np.ndarray, dmin: np.ndarray) -> np.ndarray:
    """Assemble raw GGUF super-blocks [N, nsb*144] uint8.

    q [N, nsb, 256] values 0..15 in ELEMENT order; sc6/mn6 [N, nsb, 8]; d/dmin
    [N, nsb] float16.  Layout {fp16 d, fp16 dmin, u8 scales[12], u8 qs[128]}
    (S/csrc/xpu/esimd_kernels/q4_k_GEMV.h:3-7, SP:2521-2535); element 64 il + p
    (p < 32) is the low nibble of qs[32 il + p], element 64 il + 32 + p the high
    nibble (SP:2559-2566).
    """
    N, nsb, _ = q.shape
    raw = np.zeros((N, nsb, Q4K_BYTES), dtype=np.uint8)
    raw[:, :, 0:2] = d.astype(np.float16).reshape(N, nsb, 1).view(np.uint8)
    raw[:, :, 2:4] = dmin.astype(np.float16).reshape(N, nsb, 1).view(np.uint8)
    raw[:, :, 4:16] = q4k_pack_scales(sc6, mn6)
    qq = q.astype(np.uint8).reshape(N, nsb, 4, 2, 32)          # il, half, p
    raw[:, :, 16:144] = (qq[:, :, :, 0, :] | (qq[:, :, :, 1, :] << 4)).reshape(N, nsb, 128)
    return raw.reshape(N, nsb * Q4K_BYTES)


def q4k_repack(raw: np.ndarray):
    """Raw super-blocks -> (ql [N, K/2] u8 interleaved nibbles, scale, min [N, K/32] fp16).

    SP:2527-2573: scale = fp16(f32(d) * sc6), min = fp16(f32(dmin) * mn6); byte j
    of ql holds element 2j in the low nibble and 2j+1 in the high nibble.
    """
    N = raw.shape[0]
    nsb = raw.shape[1] // Q4K_BYTES
    buf = raw.reshape(N, nsb, Q4K_BYTES)
    dm = np.ascontiguousarray(buf[:, :, 0:4]).view(np.float16).reshape(N, nsb, 2)
    dall = dm[:, :, 0].astype(np.float32)
    dmin = dm[:, :, 1].astype(np.float32)
    sc6, mn6 = q4k_unpack_scales(buf[:, :, 4:16])
    scale = (dall[:, :, None] * sc6.astype(np.float32)).astype(np.float16)
    minv = (dmin[:, :, None] * mn6.astype(np.float32)).astype(np.float16)
    qs = buf[:, :, 16:144].reshape(N, nsb, 4, 32)
    nib = np.empty((N, nsb, 4, 2, 32), dtype=np.uint8)
    nib[:, :, :, 0, :] = qs & 0xF
    nib[:, :, :, 1, :] = qs >> 4
    nib = nib.reshape(N, nsb * Q4K_SB)
    ql = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    K = nsb * Q4K_SB
    return (np.ascontiguousarray(ql), np.ascontiguousarray(scale.reshape(N, K // 32)),
            np.ascontiguousarray(minv.reshape(N, K // 32)))


def q4k_dequant(ql: np.ndarray, scale: np.ndarray, minv: np.ndarray) -> np.ndarray:
    """Repacked rep -> dense fp16 [N, K]: fp16(fp16(nib * scale) - min), two
    roundings, as the torch eager fp16 ops at SP:2576-2587 compute it."""
    N, half = ql.shape
    K = half * 2
    nib = np.empty((N, K), dtype=np.float16)
    nib[:, 0::2] = (ql & 0xF).astype(np.float16)
    nib[:, 1::2] = (ql >> 4).astype(np.float16)
    nb = scale.shape[1]
    prod = (nib.reshape(N, nb, 32) * scale.astype(np.float16)[:, :, None]).astype(np.float16)
    w = (prod - minv.astype(np.float16)[:, :, None]).astype(np.float16)
    return w.reshape(N, K)


def q4k_dequant_from_raw(raw: np.ndarray) -> np.ndarray:
    """Independent route: walk each super-block byte by byte (no repack) and apply
    the same fp16 roundings.  Used to cross-check repack + dequant."""
    N = raw.shape[0]
    nsb = raw.shape[1] // Q4K_BYTES
    out = np.empty((N, nsb * Q4K_SB), dtype=np.float16)
    for n in range(N):
        for b in range(nsb):
            blk = raw[n, b * Q4K_BYTES:(b + 1) * Q4K_BYTES]
            d = np.frombuffer(blk[0:2].tobytes(), dtype=np.float16)[0]
            dmin = np.frombuffer(blk[2:4].tobytes(), dtype=np.float16)[0]
            sc = blk[4:16].astype(np.int32)
            qs = blk[16:144]
            for j in range(8):
                if j < 4:
                    s6, m6 = sc[j] & 63, sc[j + 4] & 63
                else:
                    s6 = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)
                    m6 = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)
                s16 = np.float16(np.float32(d) * np.float32(s6))
                m16 = np.float16(np.float32(dmin) * np.float32(m6))
                il, hi = j // 2, j % 2
                for p in range(32):
                    byte = int(qs[32 * il + p])
                    nibv = (byte >> 4) if hi else (byte & 0xF)
                    prod = np.float16(np.float16(nibv) * s16)
                    out[n, b * 256 + 32 * j + p] = np.float16(prod - m16)
    return out


# ----------------------------------------------------------------------------
# MoE routing, permutation, forward (cfg3)
# ----------------------------------------------------------------------------
def moe_topk(logits: torch.Tensor, top_k: int, out_dtype=None):
    """softmax -> top-k -> renormalise.

    fp32 softmax, K rounds of argmax with the LOWEST index winning ties, weights
    renormalised over the selected K and stored in the activation dtype, ids
    int32 in descending-probability order
    (V/csrc/xpu/esimd_kernels/moe_ops.h:77-104, :126-197).  Softmax is strictly
    monotone, so the selection is made on the logits themselves: (logit desc,
    index asc) — this keeps the ids independent of the exp implementation.
    """
    lf = logits.to(torch.float32)
    T, E = lf.shape
    # stable descending sort: among equal logits the lower index stays first
    order = torch.sort(lf, dim=-1, descending=True, stable=True).indices[:, :top_k]
    probs = torch.softmax(lf, dim=-1)
    tv = torch.gather(probs, 1, order)
    tv = tv / tv.sum(dim=-1, keepdim=True)
    return tv.to(out_dtype or logits.dtype), order.to(torch.int32)


def moe_sort(top_ids: torch.Tensor, num_experts: int):
    """Stable counting sort of the flattened (token, route) pairs by expert.

    Returns sorted_pairs [T*k] int32 (sorted position -> pair index t*k + j),
    expert_start [E+1] int32 (exclusive prefix of counts) and inv [T*k] int32
    (pair index -> sorted position).  build_sorted_token_ids / build_topk_ids,
    V/csrc/xpu/esimd_kernels/moe_ops.h:238-271;
    V/python/custom_esimd_kernels_vllm/ops.py:1318-1330 (argsort stable=True).
    """
    flat = top_ids.reshape(-1).to(torch.int64)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=num_experts)
    start = torch.zeros(num_experts + 1, dtype=torch.int64)
    start[1:] = counts.cumsum(0)
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel())
    return order.to(torch.int32), start.to(torch.int32), inv.to(torch.int32)


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up on [rows, 2I] -> [rows, I], fp32 math
    (V/csrc/xpu/esimd_kernels/moe_ops.h:576-621; gate is the first half)."""
    g, u = gate_up.to(torch.float32).chunk(2, dim=-1)
    return g * torch.sigmoid(g) * u


def gelu_tanh_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """[rows, 2I] -> [rows, I] fp32: GELU_tanh(gate) * up, gate = first half
    (V/csrc/xpu/esimd_kernels/moe_ops.h:696-723; the textbook tanh form, which
    torch.nn.functional.gelu(approximate="tanh") implements)."""
    half = gate_up.shape[-1] // 2
    g, u = gate_up[..., :half].float(), gate_up[..., half:].float()
    return torch.nn.functional.gelu(g, approximate="tanh") * u


def moe_forward(x, top_w, top_ids, w13_q, w13_s, w2_q, w2_s, *, act_quant: bool,
                act_dtype=torch.bfloat16):
    """Routed-experts MoE forward (no shared expert), per-token / per-route loop.

    V/tests/test_moe_forward_full_fp8_block.py:49-80 without the shared-expert
    terms.  With act_quant the activations entering both GEMMs are quantised per
    token per 128-group to E4M3 and dequantised again (cfg3); the intermediate is
    rounded to `act_dtype` first, as a kernel that stores it would.
    """
    T, H = x.shape
    k = top_ids.shape[1]
    dw13 = fp8_dequant_block(w13_q, w13_s)
    dw2 = fp8_dequant_block(w2_q, w2_s)
    if act_quant:
        xq, xs = act_quant_per_token_group(x)
        x32 = act_dequant_per_token_group(xq, xs)
    else:
        x32 = x.to(torch.float32)
    out = torch.zeros(T, H, dtype=torch.float32)
    for t in range(T):
        for j in range(k):
            e = int(top_ids[t, j])
            gu = x32[t] @ dw13[e].t()
            inter = silu_mul(gu[None, :])
            if act_quant:
                inter = inter.to(act_dtype)
                iq, isc = act_quant_per_token_group(inter)
                inter = act_dequant_per_token_group(iq, isc)
            else:
                inter = inter.to(act_dtype).to(torch.float32)
            out[t] += top_w[t, j].to(torch.float32) * (inter[0] @ dw2[e].t())
    return out


def moe_forward_grouped(x, top_w, top_ids, w13_q, w13_s, w2_q, w2_s, num_experts, *,
                        act_quant: bool, act_dtype=torch.bfloat16, inter_q=None, return_parts=False,
                        weight_dtype=None):
    """Same result as moe_forward, computed expert by expert on the sorted rows
    (V/tests/test_fp8_blockscale_moe_prefill.py:113-118).  Fast enough for cfg3.

    inter_q = (codes uint8 [T*k, I], scale fp32 [T*k, I/128]) in SORTED row order
    replaces this function's own quantisation of the intermediate: re-quantising
    is discontinuous (a 1-ulp change of a group's largest element moves the whole
    group's grid), so a check of the down GEMM and of the combine has to start
    from the very codes the kernel under test produced.
    return_parts -> (out, inter [T*k, I] in act_dtype, y [T*k, H] fp32), sorted order.
    weight_dtype: round the block-scaled weights to this type first (see fp8_dequant_block).
    """
    T, H = x.shape
    k = top_ids.shape[1]
    order, start, _ = moe_sort(top_ids, num_experts)
    tok = (order // k).long()
    if act_quant:
        xq, xs = act_quant_per_token_group(x)
        x32 = act_dequant_per_token_group(xq, xs)
    else:
        x32 = x.to(torch.float32)
    out = torch.zeros(T, H, dtype=torch.float32)
    wflat = top_w.reshape(-1).to(torch.float32)
    I = w2_q.shape[-1]
    inter_all = torch.zeros(T * k, I, dtype=act_dtype)
    y_all = torch.zeros(T * k, H, dtype=torch.float32)
    for e in range(num_experts):
        lo, hi = int(start[e]), int(start[e + 1])
        if hi == lo:
            continue
        rows = tok[lo:hi]
        dw13 = fp8_dequant_block(w13_q[e], w13_s[e], out_dtype=weight_dtype)
        dw2 = fp8_dequant_block(w2_q[e], w2_s[e], out_dtype=weight_dtype)
        inter = silu_mul(x32[rows] @ dw13.t()).to(act_dtype)
        inter_all[lo:hi] = inter
        if inter_q is not None:
            inter32 = act_dequant_per_token_group(inter_q[0][lo:hi], inter_q[1][lo:hi])
        elif act_quant:
            iq, isc = act_quant_per_token_group(inter)
            inter32 = act_dequant_per_token_group(iq, isc)
        else:
            inter32 = inter.to(torch.float32)
        y = inter32 @ dw2.t()
        y_all[lo:hi] = y
        out.index_add_(0, rows, y * wflat[order[lo:hi].long()][:, None])
    if return_parts:
        return out, inter_all, y_all
    return out


# ----------------------------------------------------------------------------
# Seeded synthetic inputs for the five benchmark configs
# ----------------------------------------------------------------------------
def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def make_int4_case(M, K, N, *, seed=1234, act_dtype=torch.float16, asym=False):
    """cfg0 / cfg2 inputs: signed int4 uniform [-8,7] stored +8, fp16 group scales
    U[0.005,0.02], optional uint4 zero-points U[0,15], activations ~N(0,1)."""
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(act_dtype)
    q = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    packed = int4_pack(q)
    scale = (torch.rand(N, K // INT4_GROUP, generator=g) * 0.015 + 0.005).to(torch.float16)
    zp = None
    if asym:
        zp = torch.randint(0, 16, (N, K // INT4_GROUP), generator=g, dtype=torch.int32).to(torch.uint8)
    return x, packed, scale, zp


def make_fp8_pern_case(M, K, N, *, seed=1235, act_dtype=torch.bfloat16):
    """cfg1 inputs: N(0,0.02) bf16 weights quantised per output channel, fp32 scales."""
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(act_dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    w8, s = fp8_quantize_per_channel(w)
    return x, w8, s


def make_fp8_block_case(M, K, N, *, seed=1237, act_dtype=torch.bfloat16, std=0.02):
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(act_dtype)
    w = torch.randn(N, K, generator=g) * std
    w8, s = fp8_quantize_block(w)
    return x, w8, s


def make_moe_case(T, E, top_k, H, I, *, seed=1237, act_dtype=torch.bfloat16):
    """cfg3 inputs."""
    g = _gen(seed)
    x = torch.randn(T, H, generator=g).to(act_dtype)
    logits = torch.randn(T, E, generator=g).to(act_dtype)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    w13_q, w13_s = fp8_quantize_block(w13)
    del w13
    w2_q, w2_s = fp8_quantize_block(w2)
    del w2
    return x, logits, w13_q, w13_s, w2_q, w2_s


def make_q4k_case(M, K, N, *, seed=1238):
    """cfg4 inputs: raw super-blocks with q U{0..15}, sc6/mn6 U{0..63},
    d ~ U(0.001,0.01), dmin ~ U(0,0.005); activations fp16 ~N(0,1)."""
    rng = np.random.default_rng(seed)
    nsb = K // Q4K_SB
    q = rng.integers(0, 16, size=(N, nsb, 256), dtype=np.uint8)
    sc6 = rng.integers(0, 64, size=(N, nsb, 8), dtype=np.uint8)
    mn6 = rng.integers(0, 64, size=(N, nsb, 8), dtype=np.uint8)
    d = rng.uniform(0.001, 0.01, size=(N, nsb)).astype(np.float16)
    dmin = rng.uniform(0.0, 0.005, size=(N, nsb)).astype(np.float16)
    raw = q4k_build_raw(q, sc6, mn6, d, dmin)
    x = torch.randn(M, K, generator=_gen(seed)).to(torch.float16)
    return x, raw


# ----------------------------------------------------------------------------
# Error metric used by every GEMV / GEMM parity test
# ----------------------------------------------------------------------------
def max_rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max |out - ref| / max(|ref|, floor) with floor = mean |ref|.

    The north-star bound is "max relative error <= 1e-2 against the
    fp32-accumulated reference"; outputs of a dot product can sit arbitrarily
    close to zero, so the denominator is floored at the tensor's mean magnitude
    (the reference floors at 1e-3 absolute, V/tests/test_fp8_blockscale_gemm.py:55).
    """
    o = out.to(torch.float32)
    r = ref.to(torch.float32)
    floor = r.abs().mean().clamp(min=1e-12)
    return float(((o - r).abs() / r.abs().clamp(min=float(floor))).max())


def max_rel_err_abs_floor(out: torch.Tensor, ref: torch.Tensor, floor: float = 1e-3) -> float:
    """max |out - ref| / max(|ref|, floor): the reference's own element-wise form
    (`ref.abs().clamp(min=1e-3)`, V/tests/test_fp8_blockscale_gemm.py:55).  Stricter than
    max_rel_err on the outputs that sit near zero: there the error of a K-long dot product
    (rounding of the 16-bit output, summation order, weights kept unrounded by a kernel) is
    judged against 1e-3 instead of against the tensor's typical magnitude."""
    o = out.to(torch.float32)
    r = ref.to(torch.float32)
    return float(((o - r).abs() / r.abs().clamp(min=floor)).max())


def moe_forward_full(x, logits, w13, s13, shared_w13, shared_s13, w2, s2, shared_w2, shared_s2, shared_gate, top_k):
    """Small-batch fused MoE decode step with one shared expert, fp32 throughout.
    Follows the per-token loop of V/tests/test_moe_forward_full_fp8_block.py:49-80:
    softmax -> top-k (lowest index wins ties) -> renormalise -> routed experts ->
    + sigmoid(x . gate) * shared expert.  Weights are uint8 E4M3 codes with 128x128
    block scales."""
    top_w, top_ids = moe_topk(logits, top_k, out_dtype=torch.float32)
    x32 = x.float()
    out = torch.zeros_like(x32)
    dw13 = fp8_dequant_block(w13, s13)
    dw2 = fp8_dequant_block(w2, s2)
    for t in range(x.shape[0]):
        for j in range(top_k):
            e = int(top_ids[t, j])
            gate, up = (x32[t] @ dw13[e].t()).chunk(2, dim=-1)
            inter = torch.nn.functional.silu(gate) * up
            out[t] += top_w[t, j].float() * (inter @ dw2[e].t())
    g = torch.sigmoid(x32 @ shared_gate.float().t())
    gate, up = (x32 @ fp8_dequant_block(shared_w13, shared_s13).t()).chunk(2, dim=-1)
    sh = torch.nn.functional.silu(gate) * up
    out += g * (sh @ fp8_dequant_block(shared_w2, shared_s2).t())
    return out


def moe_forward_full_kmajor(x, logits, w13, s13, shared_w13, shared_s13, w2, s2, shared_w2, shared_s2, shared_gate,
                            top_k):
    """Per-tensor FP8 MoE decode step on K-major routed weights, fp32 throughout: what the kernels of
    V/csrc/moe_batch/moe.sycl compute for moe_forward_full (:1855-1940) — routed up :371-456
    (gate_up [E, H, 2I]: element [e, k, n]; scale gate_up_scale[e]; SiLU(gate) * up), routed down :815-868
    (down [E, I, H]: element [e, i, h]; times routing weight and down_scale[e]), shared up :647-692
    (shared_gate_up [2I, H], N-major), finalize :1386-1421 (sigmoid(x . gate) * shared down [H, I]).
    Weights are uint8 E4M3 codes; shared_w13 / shared_w2 may be None (no shared expert)."""
    top_w, top_ids = moe_topk(logits, top_k, out_dtype=torch.float32)
    x32 = x.float()
    T, H = x.shape
    E, _, two_i = w13.shape
    I = two_i // 2
    d13 = e4m3_decode(w13.reshape(-1, two_i)).reshape(E, H, two_i)
    d2 = e4m3_decode(w2.reshape(-1, H)).reshape(E, I, H)
    out = torch.zeros_like(x32)
    for t in range(T):
        for j in range(top_k):
            e = int(top_ids[t, j])
            gu = (x32[t] @ d13[e]) * s13[e]
            inter = torch.nn.functional.silu(gu[:I]) * gu[I:]
            out[t] += top_w[t, j].float() * s2[e] * (inter @ d2[e])
    if shared_w13 is not None:
        gu = (x32 @ e4m3_decode(shared_w13.reshape(two_i, H)).t()) * shared_s13.reshape(-1)[0]
        sh = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
        y = (sh @ e4m3_decode(shared_w2.reshape(H, I)).t()) * shared_s2.reshape(-1)[0]
        out += torch.sigmoid(x32 @ shared_gate.float().reshape(H, 1)) * y
    return out


def moe_prefill_scalar(x, topk_weights, topk_ids, w13, w13_scale, w2, w2_scale, return_parts=False, act="silu"):
    """FP8 MoE prefill with per-expert scalar scales, fp32 throughout
    (S/csrc/moe_prefill/moe_prefill_fp8.sycl:616-649; gate/up scales separate, :196-199):
      gate = s13[e,0] * (x @ w13[e,:I]^T), up = s13[e,1] * (x @ w13[e,I:]^T),
      inter = silu(gate) * up, y = s2[e] * (inter @ w2[e]^T), out[t] = sum_j w[t,j] * y[t,j].
    w13_scale of shape [E] is one scale for both halves, and act="gelu_tanh" the tanh form of
    GELU on the gate: the per-route loop of V/tests/test_moe_full_gelu_tanh.py:14-29 and
    V/tests/test_moe_fp8_grouped.py:6-15 (kept in fp32 here).
    return_parts also gives the [T*k, I] intermediate and the [T*k, H] expert output in pair order."""
    if w13_scale.dim() == 1:
        w13_scale = torch.stack([w13_scale, w13_scale], 1)
    fn = torch.nn.functional.silu if act == "silu" else (lambda g: torch.nn.functional.gelu(g, approximate="tanh"))
    T, H = x.shape
    k = topk_ids.shape[1]
    E, two_i, _ = w13.shape
    I = two_i // 2
    d13 = e4m3_decode(w13.reshape(-1, H)).reshape(E, two_i, H)
    d2 = e4m3_decode(w2.reshape(-1, I)).reshape(E, H, I)
    x32 = x.float()
    inter = torch.zeros(T * k, I)
    y = torch.zeros(T * k, H)
    for t in range(T):
        for j in range(k):
            e = int(topk_ids[t, j])
            gate = (x32[t] @ d13[e, :I].t()) * w13_scale[e, 0]
            up = (x32[t] @ d13[e, I:].t()) * w13_scale[e, 1]
            inter[t * k + j] = fn(gate) * up
            y[t * k + j] = (inter[t * k + j] @ d2[e].t()) * w2_scale[e]
    out = (topk_weights.float().reshape(T, k, 1) * y.reshape(T, k, H)).sum(1)
    return (out, inter, y) if return_parts else out


def rmsnorm(x, weight, eps, residual=None, gate=None, heads=None):
    """RMS norm as the reference's fused decode ops define it, fp32:
    a = x (+ residual);  normed = a * rsqrt(mean(a^2) + eps) * weight (* silu(gate)),
    per row, or per head of len(weight) elements when `heads` is given
    (V/tests/test_resadd_norm_gemv_int4.py:41-58, V/tests/test_norm_gemv_int4.py:36-68).
    Returns (normed fp32, updated residual rounded to x's dtype or None)."""
    a = x.float()
    new_res = None
    if residual is not None:
        a = a + residual.float()
        new_res = a.to(x.dtype)
    shape = a.shape
    if heads is not None:
        a = a.reshape(-1, weight.numel())
    var = a.pow(2).mean(dim=-1, keepdim=True)
    normed = a * torch.rsqrt(var + eps) * weight.float()
    normed = normed.reshape(shape)
    if gate is not None:
        z = gate.float()
        normed = normed * (z * torch.sigmoid(z))
    return normed, new_res
