"""CPU oracle for the weight-preparation side of the quantized-linear path:
GGUF Q4_0 / Q8_0 / Q5_K / Q6_K repack + dequant, and the on-device Q4_0
(group-128) quantizer.  TEST INFRASTRUCTURE ONLY: nothing in the product
package imports it.

Citations: SP = sglang/patches/sglang_for_multi_arc.patch, V/ =
vllm/custom-esimd-kernels-vllm, S/ = sglang/custom-esimd-kernels.

Every format has two routes here.  `*_repack` + `*_dequant` restate the
reference's torch code (vectorised numpy); `*_dequant_from_raw` walks the raw
GGML blocks element by element from the published GGML block definitions
(block_q4_0 / block_q8_0 / block_q5_K / block_q6_K and their
dequantize_row_* loops) with the reference's fp16 roundings, without going
through the repacked representation.  The two are written from different
sources and in different index orders, so a slip in the nibble order, the
high-bit placement, the 6-bit scale unpacking or the tile pre-shuffle shows up
as a mismatch (tests/test_oracle_gguf.py), together with hand-built blocks
whose values are set one element at a time.

Pinning status:
  * Q4_0, Q8_0, Q5_K, Q6_K repack / dequant: the two routes above, hand-built
    single-block fixtures, all 64x64 (sc6, mn6) encodings for Q5_K (shared with
    Q4_K), every 2-bit / 1-bit high field position of a 512-tile.
  * Q5_K / Q6_K element-order ("plain") high bits of the MoE down stacks
    (q5k_repack_plain, q6k_repack_plain + the *_dequant_plain element decodes): against the
    raw-block walk, against the tile-shuffled route, and hand-built single-element blocks
    that fix byte and bit position.
  * q4_0_quantize: GGML's published quantize_row_q4_0 rule restated; pinned by
    the reference's known-answer block (7, -7, 3, -3 -> scale -0.875,
    V/tests/test_gemv_int4.py:360-414), by the error envelope the reference's
    own test asserts (V/tests/test_q4_0_quant_xpu.py:88-118) and by brute force
    on tiny blocks.  The CPU library the reference compares against
    (ggml_quantize_tensor, an external .so) is not in the reference tree.
"""
from __future__ import annotations

import numpy as np

from .qlinear_oracle import q4k_unpack_scales

Q4_0_BYTES = 18      # {fp16 d; u8 qs[16]} per 32 elements            SP:2170
Q8_0_BYTES = 34      # {fp16 d; i8 qs[32]} per 32 elements            SP:3028
Q5K_BYTES = 176      # d, dmin, scales[12], qh[32], qs[128] per 256   SP:2638
Q6K_BYTES = 210      # ql[128], qh[64], scales[16] i8, d per 256      SP:2639
KQ_SB = 256
KQ_TILE = 512        # K tile of the high-bit pre-shuffle              SP:2642


def _f16(a):
    return np.asarray(a).astype(np.float16)


def pack_nibble_interleaved(u: np.ndarray) -> np.ndarray:
    """[N, K] values (low 4 bits used) -> [N, K/2] u8, byte j = elem 2j | elem 2j+1 << 4
    (SP:2652-2656)."""
    return ((u[:, 0::2] & 0xF) | ((u[:, 1::2] & 0xF) << 4)).astype(np.uint8)


def unpack_nibble_interleaved(ql: np.ndarray) -> np.ndarray:
    N, half = ql.shape
    v = np.empty((N, half * 2), dtype=np.int32)
    v[:, 0::2] = ql & 0xF
    v[:, 1::2] = ql >> 4
    return v


# ---------------------------------------------------------------------------
# Q4_0
# ---------------------------------------------------------------------------
def q4_0_build_raw(q: np.ndarray, d: np.ndarray) -> np.ndarray:
    """q [N, K] in 0..15 (element order), d [N, K/32] fp16 -> raw blocks [N, K/32*18].
    GGML block_q4_0: byte j of qs = elem j (low nibble) | elem j+16 (high nibble)."""
    N, K = q.shape
    nb = K // 32
    raw = np.zeros((N, nb, Q4_0_BYTES), dtype=np.uint8)
    raw[:, :, 0:2] = _f16(d).reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    qb = q.reshape(N, nb, 32).astype(np.uint8)
    raw[:, :, 2:18] = qb[:, :, 0:16] | (qb[:, :, 16:32] << 4)
    return raw.reshape(N, nb * Q4_0_BYTES)


def q4_0_repack(raw: np.ndarray):
    """SP:2173-2193: split-half GGML nibbles -> interleaved [N, K/2] u8 + scale [N, K/32] fp16."""
    N = raw.shape[0]
    nb = raw.shape[1] // Q4_0_BYTES
    buf = raw.reshape(N, nb, Q4_0_BYTES)
    scale = np.ascontiguousarray(buf[:, :, 0:2]).view(np.float16).reshape(N, nb)
    qs = buf[:, :, 2:18]
    nib = np.concatenate([qs & 0xF, qs >> 4], axis=2)          # [N, nb, 32], element order
    packed = (nib[:, :, 0::2] | (nib[:, :, 1::2] << 4)).astype(np.uint8).reshape(N, nb * 16)
    return np.ascontiguousarray(packed), np.ascontiguousarray(scale)


def q4_0_dequant(packed: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """SP:2196-2213 with out_dtype fp16: fp16(nib - 8) * fp16 scale, one rounding."""
    N = packed.shape[0]
    nb = scale.shape[1]
    v = (unpack_nibble_interleaved(packed) - 8).astype(np.float16)
    w = (v.reshape(N, nb, 32) * _f16(scale)[:, :, None]).astype(np.float16)
    return w.reshape(N, nb * 32)


def q4_0_dequant_from_raw(raw: np.ndarray) -> np.ndarray:
    """GGML dequantize_row_q4_0 order: y[j] = (qs[j] & 0xF) - 8, y[j+16] = (qs[j] >> 4) - 8, times d."""
    N = raw.shape[0]
    nb = raw.shape[1] // Q4_0_BYTES
    out = np.empty((N, nb * 32), dtype=np.float16)
    for n in range(N):
        for b in range(nb):
            blk = raw[n, b * Q4_0_BYTES:(b + 1) * Q4_0_BYTES]
            d = np.frombuffer(blk[0:2].tobytes(), dtype=np.float16)[0]
            for j in range(16):
                byte = int(blk[2 + j])
                out[n, b * 32 + j] = np.float16(np.float16((byte & 0xF) - 8) * d)
                out[n, b * 32 + j + 16] = np.float16(np.float16((byte >> 4) - 8) * d)
    return out


# ---------------------------------------------------------------------------
# Q8_0
# ---------------------------------------------------------------------------
def q8_0_build_raw(q: np.ndarray, d: np.ndarray) -> np.ndarray:
    """q [N, K] int8, d [N, K/32] fp16 -> raw [N, K/32*34]."""
    N, K = q.shape
    nb = K // 32
    raw = np.zeros((N, nb, Q8_0_BYTES), dtype=np.uint8)
    raw[:, :, 0:2] = _f16(d).reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    raw[:, :, 2:34] = q.astype(np.int8).reshape(N, nb, 32).view(np.uint8)
    return raw.reshape(N, nb * Q8_0_BYTES)


def q8_0_repack(raw: np.ndarray):
    """SP:3031-3044: -> (qs [N, K] int8, scale [N, K/32] fp16)."""
    N = raw.shape[0]
    nb = raw.shape[1] // Q8_0_BYTES
    buf = raw.reshape(N, nb, Q8_0_BYTES)
    scale = np.ascontiguousarray(buf[:, :, 0:2]).view(np.float16).reshape(N, nb)
    qs = np.ascontiguousarray(buf[:, :, 2:34]).view(np.int8).reshape(N, nb * 32)
    return qs, np.ascontiguousarray(scale)


def q8_0_dequant(qs: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """SP:3047-3054 with out_dtype fp16: fp16(qs) * scale, one rounding."""
    N, K = qs.shape
    nb = scale.shape[1]
    w = (qs.astype(np.float16).reshape(N, nb, 32) * _f16(scale)[:, :, None]).astype(np.float16)
    return w.reshape(N, K)


def q8_0_dequant_from_raw(raw: np.ndarray) -> np.ndarray:
    N = raw.shape[0]
    nb = raw.shape[1] // Q8_0_BYTES
    out = np.empty((N, nb * 32), dtype=np.float16)
    for n in range(N):
        for b in range(nb):
            blk = raw[n, b * Q8_0_BYTES:(b + 1) * Q8_0_BYTES]
            d = np.frombuffer(blk[0:2].tobytes(), dtype=np.float16)[0]
            q = np.frombuffer(blk[2:34].tobytes(), dtype=np.int8)
            for j in range(32):
                out[n, b * 32 + j] = np.float16(np.float16(int(q[j])) * d)
    return out


# ---------------------------------------------------------------------------
# high-bit pre-shuffles (SP:2659-2686)
# ---------------------------------------------------------------------------
def preshuffle_qh1(high: np.ndarray) -> np.ndarray:
    """[N, K] 0/1 -> [N, K/8] u8; per 512-tile, bit b of byte t = element b*64 + t."""
    N, K = high.shape
    h = high.astype(np.int32).reshape(N, K // KQ_TILE, 8, KQ_TILE // 8)
    byte = np.zeros((N, K // KQ_TILE, KQ_TILE // 8), dtype=np.int32)
    for b in range(8):
        byte |= (h[:, :, b, :] & 1) << b
    return byte.astype(np.uint8).reshape(N, K // 8)


def preshuffle_qh2(high: np.ndarray) -> np.ndarray:
    """[N, K] 0..3 -> [N, K/4] u8; per 512-tile, 2-bit field p of byte t = element p*128 + t."""
    N, K = high.shape
    h = high.astype(np.int32).reshape(N, K // KQ_TILE, 4, KQ_TILE // 4)
    byte = np.zeros((N, K // KQ_TILE, KQ_TILE // 4), dtype=np.int32)
    for p in range(4):
        byte |= (h[:, :, p, :] & 3) << (2 * p)
    return byte.astype(np.uint8).reshape(N, K // 4)


def unshuffle_qh1(qh: np.ndarray, K: int) -> np.ndarray:
    N = qh.shape[0]
    q = qh.astype(np.int32).reshape(N, K // KQ_TILE, KQ_TILE // 8)
    high = np.zeros((N, K // KQ_TILE, 8, KQ_TILE // 8), dtype=np.int32)
    for b in range(8):
        high[:, :, b, :] = (q >> b) & 1
    return high.reshape(N, K)


def unshuffle_qh2(qh: np.ndarray, K: int) -> np.ndarray:
    N = qh.shape[0]
    q = qh.astype(np.int32).reshape(N, K // KQ_TILE, KQ_TILE // 4)
    high = np.zeros((N, K // KQ_TILE, 4, KQ_TILE // 4), dtype=np.int32)
    for p in range(4):
        high[:, :, p, :] = (q >> (2 * p)) & 3
    return high.reshape(N, K)


# ---------------------------------------------------------------------------
# Q5_K
# ---------------------------------------------------------------------------
def q5k_build_raw(v5: np.ndarray, sc12: np.ndarray, d: np.ndarray, dmin: np.ndarray) -> np.ndarray:
    """v5 [N, K] in 0..31 (element order), sc12 [N, nsb, 12] u8, d/dmin [N, nsb] fp16.
    GGML block_q5_K: for group pair il (64 elements), qs[32 il + p] holds elem 64il+p
    (low nibble) and 64il+32+p (high nibble); bit 2il of qh[p] is the 5th bit of
    elem 64il+p, bit 2il+1 that of elem 64il+32+p."""
    N, K = v5.shape
    nsb = K // KQ_SB
    raw = np.zeros((N, nsb, Q5K_BYTES), dtype=np.uint8)
    raw[:, :, 0:2] = _f16(d).reshape(N, nsb, 1).view(np.uint8).reshape(N, nsb, 2)
    raw[:, :, 2:4] = _f16(dmin).reshape(N, nsb, 1).view(np.uint8).reshape(N, nsb, 2)
    raw[:, :, 4:16] = sc12
    v = v5.reshape(N, nsb, 4, 2, 32).astype(np.int32)
    qs = (v[:, :, :, 0, :] & 0xF) | ((v[:, :, :, 1, :] & 0xF) << 4)          # [N, nsb, 4, 32]
    raw[:, :, 48:176] = qs.reshape(N, nsb, 128).astype(np.uint8)
    qh = np.zeros((N, nsb, 32), dtype=np.int32)
    for il in range(4):
        qh |= ((v[:, :, il, 0, :] >> 4) & 1) << (2 * il)
        qh |= ((v[:, :, il, 1, :] >> 4) & 1) << (2 * il + 1)
    raw[:, :, 16:48] = qh.astype(np.uint8)
    return raw.reshape(N, nsb * Q5K_BYTES)


def q5k_elem(raw: np.ndarray):
    """SP:2689-2722: raw -> (v5 [N, K] int32, scale, min [N, K/32] fp16)."""
    N = raw.shape[0]
    nsb = raw.shape[1] // Q5K_BYTES
    buf = raw.reshape(N, nsb, Q5K_BYTES)
    dm = np.ascontiguousarray(buf[:, :, 0:4]).view(np.float16).reshape(N, nsb, 2)
    dall = dm[:, :, 0].astype(np.float32)
    dmin = dm[:, :, 1].astype(np.float32)
    sc6, mn6 = q4k_unpack_scales(buf[:, :, 4:16])
    qh = buf[:, :, 16:48].astype(np.int32)
    qs = buf[:, :, 48:176].astype(np.int32).reshape(N, nsb, 4, 32)
    scale = (dall[:, :, None] * sc6.astype(np.float32)).astype(np.float16)
    minv = (dmin[:, :, None] * mn6.astype(np.float32)).astype(np.float16)
    v = np.empty((N, nsb, 4, 2, 32), dtype=np.int32)
    for il in range(4):
        v[:, :, il, 0, :] = (qs[:, :, il, :] & 0xF) + ((qh >> (2 * il)) & 1) * 16
        v[:, :, il, 1, :] = (qs[:, :, il, :] >> 4) + ((qh >> (2 * il + 1)) & 1) * 16
    K = nsb * KQ_SB
    return v.reshape(N, K), scale.reshape(N, K // 32), minv.reshape(N, K // 32)


def q5k_repack(raw: np.ndarray):
    """SP:2725-2740 (no col_perm): -> (ql [N,K/2], qh [N,K/8] pre-shuffled, scale, min)."""
    v5, scale, minv = q5k_elem(raw)
    return (pack_nibble_interleaved(v5), preshuffle_qh1((v5 >> 4) & 1),
            np.ascontiguousarray(scale), np.ascontiguousarray(minv))


def q5k_dequant(ql, qh, scale, minv) -> np.ndarray:
    """SP:2952-2970 with out_dtype fp16: fp16(fp16(v5 * scale) - min), two roundings."""
    N = ql.shape[0]
    K = ql.shape[1] * 2
    v = unpack_nibble_interleaved(ql) + (unshuffle_qh1(qh, K) << 4)
    nb = scale.shape[1]
    prod = (v.astype(np.float16).reshape(N, nb, 32) * _f16(scale)[:, :, None]).astype(np.float16)
    return (prod - _f16(minv)[:, :, None]).astype(np.float16).reshape(N, K)


def q5k_repack_plain(raw: np.ndarray):
    """SP:2736-2750 (`_xpu_repack_q5_k_plain`), the representation the MoE down kernels read
    (S/csrc/xpu/esimd_kernels/moe_kquant_GEMV.h:109-116): ql [N, K/2] interleaved nibbles,
    qh [N, K/8] in ELEMENT order (byte j bit b = element 8j + b), scale / min [N, K/32] fp16.
    Any K that is a multiple of 256 (the super-block)."""
    v5, scale, minv = q5k_elem(raw)
    N, K = v5.shape
    hbit = ((v5 >> 4) & 1).reshape(N, K // 8, 8)
    weights = (1 << np.arange(8, dtype=np.int32))
    qh = (hbit * weights).sum(axis=2).astype(np.uint8)
    return (pack_nibble_interleaved(v5), np.ascontiguousarray(qh),
            np.ascontiguousarray(scale), np.ascontiguousarray(minv))


def q5k_dequant_plain(ql, qh, scale, minv) -> np.ndarray:
    """Element decode of the MoE down kernel, moe_kquant_GEMV.h:136-151: per 32-element block the
    fifth bit of element e is bit e of the little-endian 4-byte qh word; v5 = nibble + 16 bit;
    w = v5 * scale - min, here with the two fp16 roundings of the dense dequant (SP:2952-2970)
    so that both representations of one tensor give the same fp16 weights."""
    N = ql.shape[0]
    K = ql.shape[1] * 2
    words = np.ascontiguousarray(qh).view("<u4").reshape(N, K // 32)
    out = np.empty((N, K), dtype=np.float16)
    for blk in range(K // 32):
        w32 = words[:, blk].astype(np.int64)
        for e in range(32):
            byte = ql[:, blk * 16 + e // 2].astype(np.int32)
            nib = (byte >> 4) if (e & 1) else (byte & 0xF)
            v = nib + (((w32 >> e) & 1) << 4).astype(np.int32)
            prod = (v.astype(np.float16) * _f16(scale[:, blk])).astype(np.float16)
            out[:, blk * 32 + e] = (prod - _f16(minv[:, blk])).astype(np.float16)
    return out


def _scale_min_k4(j: int, sc) -> tuple:
    if j < 4:
        return int(sc[j]) & 63, int(sc[j + 4]) & 63
    return ((int(sc[j + 4]) & 0xF) | ((int(sc[j - 4]) >> 6) << 4),
            (int(sc[j + 4]) >> 4) | ((int(sc[j]) >> 6) << 4))


def q5k_dequant_from_raw(raw: np.ndarray) -> np.ndarray:
    """GGML dequantize_row_q5_K order (u1/u2 masks walking qh), fp16 roundings of the reference."""
    N = raw.shape[0]
    nsb = raw.shape[1] // Q5K_BYTES
    out = np.empty((N, nsb * KQ_SB), dtype=np.float16)
    for n in range(N):
        for b in range(nsb):
            blk = raw[n, b * Q5K_BYTES:(b + 1) * Q5K_BYTES]
            d = np.float32(np.frombuffer(blk[0:2].tobytes(), dtype=np.float16)[0])
            dmin = np.float32(np.frombuffer(blk[2:4].tobytes(), dtype=np.float16)[0])
            sc = blk[4:16]
            qh = blk[16:48]
            ql = blk[48:176]
            u1, u2, is_ = 1, 2, 0
            for j in range(0, 256, 64):
                s1, m1 = _scale_min_k4(is_, sc)
                s2, m2 = _scale_min_k4(is_ + 1, sc)
                d1, mm1 = np.float16(d * np.float32(s1)), np.float16(dmin * np.float32(m1))
                d2, mm2 = np.float16(d * np.float32(s2)), np.float16(dmin * np.float32(m2))
                base = j // 2
                for l in range(32):
                    lo = (int(ql[base + l]) & 0xF) + (16 if int(qh[l]) & u1 else 0)
                    hi = (int(ql[base + l]) >> 4) + (16 if int(qh[l]) & u2 else 0)
                    out[n, b * 256 + j + l] = np.float16(np.float16(np.float16(lo) * d1) - mm1)
                    out[n, b * 256 + j + 32 + l] = np.float16(np.float16(np.float16(hi) * d2) - mm2)
                is_ += 2
                u1 <<= 2
                u2 <<= 2
    return out


# ---------------------------------------------------------------------------
# Q6_K
# ---------------------------------------------------------------------------
def q6k_build_raw(v6: np.ndarray, sc: np.ndarray, d: np.ndarray) -> np.ndarray:
    """v6 [N, K] in 0..63 (element order), sc [N, nsb, 16] int8, d [N, nsb] fp16.
    GGML block_q6_K: per 128-element half ip, ql[64ip + l] = elem l (low) | elem l+64 (high),
    ql[64ip + 32 + l] = elem l+32 | elem l+96; qh[32ip + l] holds the top 2 bits of elems
    l, l+32, l+64, l+96 in fields 0..3."""
    N, K = v6.shape
    nsb = K // KQ_SB
    raw = np.zeros((N, nsb, Q6K_BYTES), dtype=np.uint8)
    v = v6.reshape(N, nsb, 2, 4, 32).astype(np.int32)          # [.., ip, quarter, l]
    ql = np.zeros((N, nsb, 2, 64), dtype=np.int32)
    ql[:, :, :, 0:32] = (v[:, :, :, 0, :] & 0xF) | ((v[:, :, :, 2, :] & 0xF) << 4)
    ql[:, :, :, 32:64] = (v[:, :, :, 1, :] & 0xF) | ((v[:, :, :, 3, :] & 0xF) << 4)
    qh = np.zeros((N, nsb, 2, 32), dtype=np.int32)
    for qtr in range(4):
        qh |= ((v[:, :, :, qtr, :] >> 4) & 3) << (2 * qtr)
    raw[:, :, 0:128] = ql.reshape(N, nsb, 128).astype(np.uint8)
    raw[:, :, 128:192] = qh.reshape(N, nsb, 64).astype(np.uint8)
    raw[:, :, 192:208] = sc.astype(np.int8).view(np.uint8)
    raw[:, :, 208:210] = _f16(d).reshape(N, nsb, 1).view(np.uint8).reshape(N, nsb, 2)
    return raw.reshape(N, nsb * Q6K_BYTES)


def q6k_elem(raw: np.ndarray):
    """SP:2973-2993: raw -> (v6 [N, K] int32, scale [N, K/16] fp16 = fp16(f32(d) * sc))."""
    N = raw.shape[0]
    nsb = raw.shape[1] // Q6K_BYTES
    buf = raw.reshape(N, nsb, Q6K_BYTES)
    ql = buf[:, :, 0:128].astype(np.int32)
    qh = buf[:, :, 128:192].astype(np.int32)
    sc = np.ascontiguousarray(buf[:, :, 192:208]).view(np.int8).astype(np.float32)
    d = np.ascontiguousarray(buf[:, :, 208:210]).view(np.float16).reshape(N, nsb).astype(np.float32)
    u6 = np.empty((N, nsb, KQ_SB), dtype=np.int32)
    for ip in range(2):
        q0 = ql[:, :, 64 * ip:64 * ip + 32]
        q32 = ql[:, :, 64 * ip + 32:64 * ip + 64]
        h = qh[:, :, 32 * ip:32 * ip + 32]
        u6[:, :, 128 * ip + 0:128 * ip + 32] = (q0 & 0xF) | (((h >> 0) & 3) << 4)
        u6[:, :, 128 * ip + 32:128 * ip + 64] = (q32 & 0xF) | (((h >> 2) & 3) << 4)
        u6[:, :, 128 * ip + 64:128 * ip + 96] = (q0 >> 4) | (((h >> 4) & 3) << 4)
        u6[:, :, 128 * ip + 96:128 * ip + 128] = (q32 >> 4) | (((h >> 6) & 3) << 4)
    scale16 = (d[:, :, None] * sc).astype(np.float16)
    K = nsb * KQ_SB
    return u6.reshape(N, K), scale16.reshape(N, K // 16)


def q6k_repack(raw: np.ndarray):
    """SP:2996-3008 (no col_perm): -> (ql [N,K/2], qh [N,K/4] pre-shuffled, scale [N,K/16])."""
    u6, scale = q6k_elem(raw)
    return pack_nibble_interleaved(u6), preshuffle_qh2((u6 >> 4) & 3), np.ascontiguousarray(scale)


def q6k_dequant(ql, qh, scale) -> np.ndarray:
    """SP:3011-3026 with out_dtype fp16: (fp16(v6) - 32) * scale, one rounding."""
    N = ql.shape[0]
    K = ql.shape[1] * 2
    v = unpack_nibble_interleaved(ql) + (unshuffle_qh2(qh, K) << 4)
    nb = scale.shape[1]
    w = ((v.astype(np.float16).reshape(N, nb, 16) - np.float16(32)) * _f16(scale)[:, :, None]).astype(np.float16)
    return w.reshape(N, K)


def q6k_repack_plain(raw: np.ndarray):
    """SP:2753-2765 (`_xpu_repack_q6_k_plain`), read by moe_kquant_GEMV.h:159-166: ql [N, K/2]
    interleaved nibbles, qh [N, K/4] in ELEMENT order (byte j 2-bit field p = element 4j + p),
    scale [N, K/16] fp16."""
    u6, scale = q6k_elem(raw)
    N, K = u6.shape
    h2 = ((u6 >> 4) & 3).reshape(N, K // 4, 4)
    shifts = 2 * np.arange(4, dtype=np.int32)
    qh = (h2 << shifts).sum(axis=2).astype(np.uint8)
    return pack_nibble_interleaved(u6), np.ascontiguousarray(qh), np.ascontiguousarray(scale)


def q6k_dequant_plain(ql, qh, scale) -> np.ndarray:
    """Element decode of moe_kquant_GEMV.h:185-203: per 32-element block two little-endian words,
    element e of the first 16 = bits [2e, 2e+1] of w0, of the second 16 of w1; v6 = nibble + 16 h;
    w = (v6 - 32) * scale[k / 16], one fp16 rounding as in the dense dequant (SP:3011-3026)."""
    N = ql.shape[0]
    K = ql.shape[1] * 2
    words = np.ascontiguousarray(qh).view("<u4").reshape(N, K // 16)
    out = np.empty((N, K), dtype=np.float16)
    for blk in range(K // 32):
        for half in range(2):
            w32 = words[:, 2 * blk + half].astype(np.int64)
            s16 = _f16(scale[:, 2 * blk + half])
            for e in range(16):
                k = blk * 32 + half * 16 + e
                byte = ql[:, k // 2].astype(np.int32)
                nib = (byte >> 4) if (k & 1) else (byte & 0xF)
                v = nib + (((w32 >> (2 * e)) & 3) << 4).astype(np.int32)
                out[:, k] = ((v.astype(np.float16) - np.float16(32)) * s16).astype(np.float16)
    return out


def q6k_dequant_from_raw(raw: np.ndarray) -> np.ndarray:
    """GGML dequantize_row_q6_K order (q1..q4 per l, is = l / 16), fp16 roundings of the reference."""
    N = raw.shape[0]
    nsb = raw.shape[1] // Q6K_BYTES
    out = np.empty((N, nsb * KQ_SB), dtype=np.float16)
    for n in range(N):
        for b in range(nsb):
            blk = raw[n, b * Q6K_BYTES:(b + 1) * Q6K_BYTES]
            ql = blk[0:128]
            qh = blk[128:192]
            sc = np.frombuffer(blk[192:208].tobytes(), dtype=np.int8)
            d = np.float32(np.frombuffer(blk[208:210].tobytes(), dtype=np.float16)[0])
            for ip in range(2):
                for l in range(32):
                    is_ = l // 16
                    h = int(qh[32 * ip + l])
                    q1 = ((int(ql[64 * ip + l]) & 0xF) | (((h >> 0) & 3) << 4)) - 32
                    q2 = ((int(ql[64 * ip + l + 32]) & 0xF) | (((h >> 2) & 3) << 4)) - 32
                    q3 = ((int(ql[64 * ip + l]) >> 4) | (((h >> 4) & 3) << 4)) - 32
                    q4 = ((int(ql[64 * ip + l + 32]) >> 4) | (((h >> 6) & 3) << 4)) - 32
                    for off, q, si in ((0, q1, 0), (32, q2, 2), (64, q3, 4), (96, q4, 6)):
                        s16 = np.float16(d * np.float32(int(sc[8 * ip + is_ + si])))
                        out[n, b * 256 + 128 * ip + l + off] = np.float16(np.float16(q) * s16)
    return out


# ---------------------------------------------------------------------------
# on-device Q4_0 (group 128) quantizer
# ---------------------------------------------------------------------------
def q4_0_quantize(x: np.ndarray, block: int = 128):
    """V/csrc/xpu/q4_0_quant.sycl:1-13,58-96 (GGML quantize_row_q4_0 with 128-wide blocks).

    x [M, K] (fp16/bf16 values given as float32).  Per block: max = the element of
    largest magnitude, sign kept, first one on ties (GGML's strict `amax < |v|`
    scan); d = max / -8 (fp32), stored as fp16; id = 1/d in fp32 (0 when d == 0),
    NOT recomputed from the rounded fp16 d; q = min(15, int(x * id + 8.5)) with the
    product and the sum each rounded to fp32 and the conversion truncating.
    Returns (qweight [M, K/8] int32, nibble i of word w = element 8w + i;
    scale [M, K/block] fp16).  Dequant on the consumer side: (q - 8) * scale.
    """
    x = np.asarray(x, dtype=np.float32)
    M, K = x.shape
    nb = K // block
    xb = x.reshape(M, nb, block)
    idx = np.argmax(np.abs(xb), axis=2)                        # first maximum
    mx = np.take_along_axis(xb, idx[:, :, None], axis=2)[:, :, 0]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    t = (xb * inv[:, :, None]).astype(np.float32)
    t = (t + np.float32(8.5)).astype(np.float32)
    q = np.minimum(np.trunc(t).astype(np.int32), 15)
    q = np.maximum(q, 0).astype(np.uint32).reshape(M, K // 8, 8)
    word = np.zeros((M, K // 8), dtype=np.uint32)
    for i in range(8):
        word |= q[:, :, i] << np.uint32(4 * i)
    return word.view(np.int32), d.astype(np.float16)
