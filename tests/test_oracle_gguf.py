"""Pins the weight-preparation oracle (GGUF Q4_0 / Q8_0 / Q5_K / Q6_K, Q4_0 quantizer).

Each format is checked three ways that do not share code: the vectorised
restatement of the reference's repack + dequant, an element-by-element walk of
the raw GGML blocks, and a raw-block builder that places every element from its
GGML block definition.  A wrong nibble order, high-bit position, tile shuffle or
scale index breaks at least one of the round trips below.
"""
import numpy as np
import pytest

from oracle import gguf_oracle as G
from oracle import qlinear_oracle as O


def _rng(seed):
    return np.random.default_rng(seed)


def _f16u(rng, shape, lo, hi):
    return rng.uniform(lo, hi, size=shape).astype(np.float16)


# ------------------------------------------------------------------ Q4_0 ----
def test_q4_0_hand_built_block():
    # one block, element e has nibble (e * 5 + 3) % 16, d = 0.5: GGML byte j = elem j | elem j+16 << 4
    q = np.array([[(e * 5 + 3) % 16 for e in range(32)]], dtype=np.uint8)
    raw = G.q4_0_build_raw(q, np.array([[0.5]], dtype=np.float16))
    assert raw.shape == (1, 18)
    assert raw[0, 2] == (q[0, 0] | (q[0, 16] << 4)) and raw[0, 17] == (q[0, 15] | (q[0, 31] << 4))
    packed, scale = G.q4_0_repack(raw)
    assert packed.shape == (1, 16) and scale[0, 0] == np.float16(0.5)
    # interleaved: byte j = elem 2j | elem 2j+1 << 4
    for j in range(16):
        assert packed[0, j] == (q[0, 2 * j] | (q[0, 2 * j + 1] << 4))
    w = G.q4_0_dequant(packed, scale)
    assert np.array_equal(w[0], ((q[0].astype(np.float32) - 8) * 0.5).astype(np.float16))


def test_q4_0_routes_agree():
    rng = _rng(1)
    N, K = 5, 256
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    d = _f16u(rng, (N, K // 32), -0.02, 0.02)
    raw = G.q4_0_build_raw(q, d)
    packed, scale = G.q4_0_repack(raw)
    assert np.array_equal(G.unpack_nibble_interleaved(packed), q.astype(np.int32))
    assert np.array_equal(G.q4_0_dequant(packed, scale).view(np.uint16), G.q4_0_dequant_from_raw(raw).view(np.uint16))


# ------------------------------------------------------------------ Q8_0 ----
def test_q8_0_routes_agree_and_signs():
    rng = _rng(2)
    N, K = 4, 128
    q = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    q[0, :4] = [-128, 127, -1, 0]
    d = _f16u(rng, (N, K // 32), -0.01, 0.01)
    d[0, 0] = np.float16(0.25)
    raw = G.q8_0_build_raw(q, d)
    qs, scale = G.q8_0_repack(raw)
    assert qs.dtype == np.int8 and np.array_equal(qs, q) and np.array_equal(scale, d)
    w = G.q8_0_dequant(qs, scale)
    assert list(w[0, :4]) == [np.float16(-32.0), np.float16(31.75), np.float16(-0.25), np.float16(0.0)]
    assert np.array_equal(w.view(np.uint16), G.q8_0_dequant_from_raw(raw).view(np.uint16))


# ------------------------------------------------------- tile pre-shuffles ----
def test_preshuffle_positions():
    K = 1024
    for e in (0, 63, 64, 200, 511, 512, 700, 1023):
        h = np.zeros((1, K), dtype=np.int32)
        h[0, e] = 1
        qh = G.preshuffle_qh1(h)
        tile, r = divmod(e, 512)
        b, t = divmod(r, 64)
        assert qh[0, tile * 64 + t] == (1 << b) and qh.sum() == (1 << b)
        assert np.array_equal(G.unshuffle_qh1(qh, K), h)
        h2 = np.zeros((1, K), dtype=np.int32)
        h2[0, e] = 3
        q2 = G.preshuffle_qh2(h2)
        p, t2 = divmod(r, 128)
        assert q2[0, tile * 128 + t2] == (3 << (2 * p)) and q2.astype(np.int64).sum() == (3 << (2 * p))
        assert np.array_equal(G.unshuffle_qh2(q2, K), h2)


# ------------------------------------------------------------------ Q5_K ----
def _q5k_case(rng, N, K):
    nsb = K // 256
    v5 = rng.integers(0, 32, size=(N, K))
    sc6 = rng.integers(0, 64, size=(N, nsb, 8))
    mn6 = rng.integers(0, 64, size=(N, nsb, 8))
    sc12 = O.q4k_pack_scales(sc6, mn6)
    d = _f16u(rng, (N, nsb), 0.001, 0.01)
    dmin = _f16u(rng, (N, nsb), 0.0, 0.005)
    return v5, sc6, mn6, G.q5k_build_raw(v5, sc12, d, dmin), d, dmin


def test_q5k_round_trip_and_routes():
    rng = _rng(3)
    N, K = 3, 1024
    v5, sc6, mn6, raw, d, dmin = _q5k_case(rng, N, K)
    assert raw.shape == (N, K // 256 * 176)
    u5, scale, minv = G.q5k_elem(raw)
    assert np.array_equal(u5, v5)
    exp_scale = (d.astype(np.float32)[:, :, None] * sc6.astype(np.float32)).astype(np.float16).reshape(N, K // 32)
    exp_min = (dmin.astype(np.float32)[:, :, None] * mn6.astype(np.float32)).astype(np.float16).reshape(N, K // 32)
    assert np.array_equal(scale, exp_scale) and np.array_equal(minv, exp_min)
    ql, qh, s, m = G.q5k_repack(raw)
    assert ql.shape == (N, K // 2) and qh.shape == (N, K // 8)
    w = G.q5k_dequant(ql, qh, s, m)
    assert np.array_equal(w.view(np.uint16), G.q5k_dequant_from_raw(raw).view(np.uint16))


def test_q5k_single_high_bit():
    # exactly one element with its 5th bit set: lands in bit 2*il (+1) of qh[p] of the raw block
    N, K = 1, 512
    for e in (0, 31, 32, 100, 255, 256 + 77, 511):
        v5 = np.zeros((N, K), dtype=np.int64)
        v5[0, e] = 16
        sc12 = np.zeros((N, K // 256, 12), dtype=np.uint8)
        raw = G.q5k_build_raw(v5, sc12, np.ones((N, 2), np.float16), np.ones((N, 2), np.float16))
        sb, r = divmod(e, 256)
        il, r2 = divmod(r, 64)
        half, p = divmod(r2, 32)
        blk = raw[0, sb * 176:(sb + 1) * 176]
        assert blk[16 + p] == (1 << (2 * il + half)) and blk[16:48].sum() == blk[16 + p]
        assert blk[48:176].sum() == 0
        u5, _, _ = G.q5k_elem(raw)
        assert np.array_equal(u5, v5)


# ------------------------------------------------------------------ Q6_K ----
def test_q6k_round_trip_and_routes():
    rng = _rng(4)
    N, K = 3, 1024
    nsb = K // 256
    v6 = rng.integers(0, 64, size=(N, K))
    sc = rng.integers(-128, 128, size=(N, nsb, 16)).astype(np.int8)
    d = _f16u(rng, (N, nsb), 0.0005, 0.005)
    raw = G.q6k_build_raw(v6, sc, d)
    assert raw.shape == (N, nsb * 210)
    u6, scale = G.q6k_elem(raw)
    assert np.array_equal(u6, v6)
    exp = (d.astype(np.float32)[:, :, None] * sc.astype(np.float32)).astype(np.float16).reshape(N, K // 16)
    assert np.array_equal(scale, exp)
    ql, qh, s = G.q6k_repack(raw)
    assert ql.shape == (N, K // 2) and qh.shape == (N, K // 4) and s.shape == (N, K // 16)
    w = G.q6k_dequant(ql, qh, s)
    assert np.array_equal(w.view(np.uint16), G.q6k_dequant_from_raw(raw).view(np.uint16))


def test_q6k_single_element():
    # one element = 0b110101 (53): nibble 5 in ql, 3 in its 2-bit qh field
    N, K = 1, 512                      # the pre-shuffle works on whole 512-tiles
    for e in (0, 40, 70, 127, 128 + 33, 255, 256 + 100, 511):
        v6 = np.zeros((N, K), dtype=np.int64)
        v6[0, e] = 53
        raw = G.q6k_build_raw(v6, np.ones((N, 2, 16), np.int8), np.ones((N, 2), np.float16))
        sb, r0 = divmod(e, 256)
        ip, r = divmod(r0, 128)
        qtr, l = divmod(r, 32)
        blk = raw[0, sb * 210:(sb + 1) * 210]
        assert blk[128 + 32 * ip + l] == (3 << (2 * qtr)) and blk[128:192].sum() == blk[128 + 32 * ip + l]
        qlb = 64 * ip + (32 if qtr in (1, 3) else 0) + l
        assert blk[qlb] == (5 << 4 if qtr >= 2 else 5) and blk[0:128].sum() == blk[qlb]
        assert raw[0, (1 - sb) * 210:(1 - sb) * 210 + 192].sum() == 0
        w = G.q6k_dequant(*G.q6k_repack(raw))
        exp = np.full((N, K), -32.0, dtype=np.float16)
        exp[0, e] = 21.0
        assert np.array_equal(w, exp)


# ---------------------------------- element-order high bits (MoE down stacks) ----
@pytest.mark.parametrize("K", [768, 1024, 256])
def test_plain_high_bits_routes_agree(K):
    # the element-order representation, decoded the way the MoE down kernels index it, equals
    # the raw-block walk and the tile-shuffled route; K = 768 and 256 are not whole 512-tiles
    rng = _rng(5 + K)
    N = 3
    v5, _, _, raw5, _, _ = _q5k_case(rng, N, K)
    ql, qh, s, m = G.q5k_repack_plain(raw5)
    assert ql.shape == (N, K // 2) and qh.shape == (N, K // 8) and s.shape == m.shape == (N, K // 32)
    w = G.q5k_dequant_plain(ql, qh, s, m)
    assert np.array_equal(w.view(np.uint16), G.q5k_dequant_from_raw(raw5).view(np.uint16))
    nsb = K // 256
    v6 = rng.integers(0, 64, size=(N, K))
    raw6 = G.q6k_build_raw(v6, rng.integers(-128, 128, size=(N, nsb, 16)).astype(np.int8), _f16u(rng, (N, nsb), 0.0005, 0.005))
    ql6, qh6, s6 = G.q6k_repack_plain(raw6)
    assert ql6.shape == (N, K // 2) and qh6.shape == (N, K // 4) and s6.shape == (N, K // 16)
    w6 = G.q6k_dequant_plain(ql6, qh6, s6)
    assert np.array_equal(w6.view(np.uint16), G.q6k_dequant_from_raw(raw6).view(np.uint16))
    if K % 512 == 0:
        # same nibbles, scales and decoded weights as the tile-shuffled representation
        t5 = G.q5k_repack(raw5)
        assert np.array_equal(t5[0], ql) and np.array_equal(t5[2], s) and np.array_equal(t5[3], m)
        assert np.array_equal(G.q5k_dequant(*t5).view(np.uint16), w.view(np.uint16))
        t6 = G.q6k_repack(raw6)
        assert np.array_equal(t6[0], ql6) and np.array_equal(t6[2], s6)
        assert np.array_equal(G.q6k_dequant(*t6).view(np.uint16), w6.view(np.uint16))


def test_plain_high_bits_positions():
    # one element with high bits set: Q5_K byte e // 8 bit e % 8; Q6_K byte e // 4 field e % 4
    N, K = 1, 768
    for e in (0, 7, 8, 33, 255, 256 + 77, 511, 512 + 130, 767):
        v5 = np.zeros((N, K), dtype=np.int64)
        v5[0, e] = 16
        raw = G.q5k_build_raw(v5, np.zeros((N, 3, 12), np.uint8), np.ones((N, 3), np.float16), np.ones((N, 3), np.float16))
        ql, qh, _, _ = G.q5k_repack_plain(raw)
        assert qh[0, e // 8] == (1 << (e % 8)) and qh.astype(np.int64).sum() == (1 << (e % 8)) and ql.sum() == 0
        v6 = np.zeros((N, K), dtype=np.int64)
        v6[0, e] = 0b100000 | 0b0101          # high field 2, nibble 5
        raw = G.q6k_build_raw(v6, np.ones((N, 3, 16), np.int8), np.ones((N, 3), np.float16))
        ql, qh, _ = G.q6k_repack_plain(raw)
        assert qh[0, e // 4] == (2 << (2 * (e % 4))) and qh.astype(np.int64).sum() == (2 << (2 * (e % 4)))
        assert ql[0, e // 2] == (5 << 4 if e & 1 else 5) and ql.astype(np.int64).sum() == ql[0, e // 2]
        w = G.q6k_dequant_plain(ql, qh, np.ones((N, K // 16), np.float16))
        exp = np.full((N, K), -32.0, dtype=np.float16)
        exp[0, e] = 37.0 - 32.0
        assert np.array_equal(w, exp)


# ------------------------------------------------------- Q4_0 quantizer ----
def test_q4_0_quantize_known_answer():
    # V/tests/test_gemv_int4.py:360-414: 7, -7, 3, -3 in an otherwise zero block -> scale -0.875
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, :4] = [7.0, -7.0, 3.0, -3.0]
    qw, sc = G.q4_0_quantize(x)
    assert sc[0, 0] == np.float16(-0.875)
    nib = [(int(qw.view(np.uint32)[0, 0]) >> (4 * i)) & 0xF for i in range(8)]
    assert nib[:4] == [0, 15, 5, 11] and nib[4:] == [8, 8, 8, 8]
    deq = [(n - 8) * -0.875 for n in nib[:4]]
    assert deq[0] == 7.0 and abs(deq[1] + 7.0) <= 0.875 and abs(deq[2] - 3.0) <= 0.4375 + 1e-6
    # as bytes: low nibble = even element (the layout esimd_gemv_int4 reads)
    b = qw.view(np.uint8)
    assert b[0, 0] == (0 | (15 << 4)) and b[0, 1] == (5 | (11 << 4))


def test_q4_0_quantize_tie_takes_first_and_zero_block():
    x = np.zeros((1, 256), dtype=np.float32)
    x[0, 5] = -2.0
    x[0, 9] = 2.0                      # same magnitude later: the first one (negative) wins
    qw, sc = G.q4_0_quantize(x)
    assert sc[0, 0] == np.float16(0.25) and sc[0, 1] == np.float16(0.0)
    w = qw.view(np.uint32)
    assert (int(w[0, 0]) >> 20) & 0xF == 0            # -2 / 0.25 = -8 -> 0
    assert (int(w[0, 1]) >> 4) & 0xF == 15            # +8 -> 16 -> clamped to 15
    assert np.all(w[0, 16:] == 0x88888888)            # all-zero block: d = 0, id = 0, q = 8


def test_q4_0_quantize_error_envelope():
    # V/tests/test_q4_0_quant_xpu.py:88-118: |dequant - x| <= |d| except the clamped extreme
    rng = _rng(7)
    x = (rng.standard_normal((16, 512)) * 0.5).astype(np.float16).astype(np.float32)
    qw, sc = G.q4_0_quantize(x)
    q = np.stack([(qw.view(np.uint32) >> np.uint32(4 * i)) & 0xF for i in range(8)], axis=2).reshape(16, 512)
    deq = (q.astype(np.float32) - 8) * np.repeat(sc.astype(np.float32), 128, axis=1)
    err = np.abs(deq - x)
    dabs = np.repeat(np.abs(sc.astype(np.float32)), 128, axis=1)
    assert np.all(err <= dabs + 1e-4)
    assert np.mean(err <= 0.5 * dabs + 1e-3) > 0.98   # round-to-nearest everywhere but the clamp
    # brute force against a scalar restatement of GGML's loop on a few blocks
    for r in range(2):
        for b in range(4):
            blk = x[r, b * 128:(b + 1) * 128]
            amax, mx = 0.0, 0.0
            for v in blk:
                if amax < abs(v):
                    amax, mx = abs(v), v
            d = np.float32(mx) / np.float32(-8)
            inv = np.float32(1) / d if d != 0 else np.float32(0)
            for i, v in enumerate(blk):
                qq = min(15, int(np.float32(np.float32(v * inv) + np.float32(8.5))))
                assert qq == q[r, b * 128 + i]
            assert np.float16(d) == sc[r, b]
