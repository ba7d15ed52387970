"""Pins the CPU oracle before anything is checked against it.

Each check is chosen so that a plausible slip (nibble order, offset, group
index, sign, a dropped rounding, a transposed operand) fails it; none of them
re-types the oracle's own formula.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import qlinear_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ---------------------------------------------------------------- E4M3
def test_e4m3_table_matches_torch_library_routine():
    codes = torch.arange(256, dtype=torch.uint8)
    lib = codes.view(torch.float8_e4m3fn).float()
    mine = torch.from_numpy(O.e4m3_decode_table())
    finite = torch.isfinite(lib)
    assert int(finite.sum()) == 254
    assert torch.equal(mine[finite], lib[finite])
    assert torch.isnan(mine[0x7F]) and torch.isnan(mine[0xFF])
    # signed zero is kept
    assert mine[0x80].item() == 0.0 and np.signbit(mine[0x80].item())


def test_e4m3_known_answers():
    t = O.e4m3_decode_table()
    known = {0x00: 0.0, 0x01: 2.0 ** -9, 0x07: 7 * 2.0 ** -9, 0x08: 2.0 ** -6,
             0x38: 1.0, 0x3C: 1.5, 0x40: 2.0, 0x7E: 448.0, 0xB8: -1.0, 0xFE: -448.0}
    for c, v in known.items():
        assert t[c] == np.float32(v), hex(c)


def test_e4m3_reference_all_codes_construction():
    # V/tests/test_fp8_blockscale_moe_prefill.py:54-90: weight row c is code c
    # repeated 128 times, x = ones, unit scale -> out[c] = decode(c) * 128.
    raw = torch.arange(256, dtype=torch.uint8).view(256, 1).expand(256, 128).contiguous()
    scale = torch.ones(2, 1)
    w = O.fp8_dequant_block(raw, scale)
    out = O.matmul_ref(torch.ones(1, 128, dtype=torch.float16), w)[0]
    reference = raw[:, 0].view(torch.float8_e4m3fn).float() * 128
    finite = torch.isfinite(reference)
    assert torch.equal(out[finite], reference[finite])
    assert out[0x80].item() == 0.0


def test_e4m3_quantize_roundtrip_and_rne():
    t = torch.from_numpy(O.e4m3_decode_table())
    finite = torch.isfinite(t)
    codes = torch.arange(256, dtype=torch.uint8)[finite]
    back = O.e4m3_quantize(t[finite])
    # -0.0 and +0.0 keep their own codes; every finite value maps to itself
    assert torch.equal(back, codes)
    # midpoint between 1.0 (0x38, even mantissa) and 1.125 (0x39) rounds to even
    assert int(O.e4m3_quantize(torch.tensor([1.0625]))[0]) == 0x38
    assert int(O.e4m3_quantize(torch.tensor([1.1875]))[0]) == 0x3A


# ---------------------------------------------------------------- INT4
def test_int4_known_answer_nibble_order_and_offset():
    # V/tests/test_gemv_int4.py:360-414: values 7,-7,3,-3 at k=0..3, scale -0.875:
    # stored nibbles are value/scale + 8.
    scale = -0.875
    vals = [7.0, -7.0, 3.0, -3.0]
    q = [int(round(v / scale)) for v in vals]            # -8, 8->clamped? no: 7/-0.875=-8, -7/-0.875=8
    q = [max(-8, min(7, v)) for v in q]
    row = torch.zeros(1, 128, dtype=torch.int32)
    row[0, :4] = torch.tensor(q)
    packed = O.int4_pack(row)
    # byte 0 = (q0+8) | (q1+8) << 4, byte 1 = (q2+8) | (q3+8) << 4
    assert int(packed[0, 0]) == ((q[0] + 8) | ((q[1] + 8) << 4))
    assert int(packed[0, 1]) == ((q[2] + 8) | ((q[3] + 8) << 4))
    deq = O.int4_dequant(packed, torch.tensor([[scale]], dtype=torch.float16))
    assert deq[0, 0].item() == 7.0            # (-8) * -0.875
    assert deq[0, 1].item() == -6.125         # clamp(8 -> 7) * -0.875
    assert deq[0, 4].item() == 0.0            # stored nibble 8 is zero


def test_int4_bruteforce_all_nibbles():
    scales = torch.tensor([0.005, 0.0123, 0.02, -0.875, 1.0, 6.1e-5], dtype=torch.float16)
    for s in scales:
        for u in range(16):
            row = torch.full((1, 128), 8, dtype=torch.int32)
            row[0, 37] = u                          # odd k -> high nibble of byte 18
            packed = ((row[:, 0::2] & 0xF) | ((row[:, 1::2] & 0xF) << 4)).to(torch.uint8)
            assert int(packed[0, 18]) >> 4 == u
            for dt in (torch.float16, torch.bfloat16):
                deq = O.int4_dequant(packed, s.reshape(1, 1), out_dtype=dt)
                exact = torch.tensor(float(u - 8) * float(s), dtype=torch.float64)
                assert deq[0, 37].item() == exact.to(torch.float32).to(dt).item()
                assert deq[0, 36].item() == 0.0


def test_int4_group_index_and_zero_point():
    N, K = 3, 384
    g = torch.Generator().manual_seed(0)
    q = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    packed = O.int4_pack(q)
    scale = torch.tensor([[1, 2, 4]] * N, dtype=torch.float16)
    deq = O.int4_dequant(packed, scale).float()
    assert torch.equal(deq[:, :128], q[:, :128].float())
    assert torch.equal(deq[:, 128:256], 2 * q[:, 128:256].float())
    assert torch.equal(deq[:, 256:], 4 * q[:, 256:].float())
    zp = torch.tensor([[0, 8, 15]] * N, dtype=torch.uint8)
    deqz = O.int4_dequant(packed, scale, zp=zp).float()
    u = q.float() + 8
    assert torch.equal(deqz[:, :128], u[:, :128])
    assert torch.equal(deqz[:, 128:256], 2 * (u[:, 128:256] - 8))
    assert torch.equal(deqz[:, 256:], 4 * (u[:, 256:] - 15))


def test_int4_int32_view_identity():
    g = torch.Generator().manual_seed(1)
    q = torch.randint(-8, 8, (4, 256), generator=g, dtype=torch.int32)
    packed = O.int4_pack(q)
    as_i32 = packed.view(torch.int32)
    assert as_i32.shape == (4, 32)
    # nibble z of word i is element 8 i + z
    w = as_i32.to(torch.int64) & 0xFFFFFFFF
    for z in range(8):
        assert torch.equal(((w >> (4 * z)) & 0xF).to(torch.int32), q[:, z::8] + 8)
    assert torch.equal(O.int4_unpack_u4(as_i32), O.int4_unpack_u4(packed))


# ---------------------------------------------------------------- FP8 scale broadcast
def test_block_scale_broadcast_is_per_128_block():
    N, K = 256, 384
    w8 = torch.full((N, K), 0x38, dtype=torch.uint8)                 # 1.0 everywhere
    s = torch.arange(1, 7, dtype=torch.float32).reshape(2, 3)
    d = O.fp8_dequant_block(w8, s)
    for nb in range(2):
        for kb in range(3):
            blk = d[nb * 128:(nb + 1) * 128, kb * 128:(kb + 1) * 128]
            assert torch.all(blk == s[nb, kb])
    # a transposed scale would fail here: [0,2] != [2,0] has no meaning for a 2x3 grid
    assert d[0, 383].item() == 3.0 and d[255, 0].item() == 4.0


def test_per_channel_scale_is_per_row():
    w8 = torch.full((4, 256), 0x38, dtype=torch.uint8)
    s = torch.tensor([1.0, 2.0, 3.0, 4.0])
    d = O.fp8_dequant_per_channel(w8, s)
    assert torch.equal(d[:, 0], s) and torch.equal(d[:, 255], s)


def test_fp8_block_quantizer_matches_reference_loop():
    # V/tests/test_fp8_blockscale_gemm.py:13-28 written as the explicit block loop
    g = torch.Generator().manual_seed(3)
    w = torch.randn(256, 256, generator=g) * 0.3
    q, s = O.fp8_quantize_block(w)
    for i in range(2):
        for j in range(2):
            blk = w[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128]
            sc = (blk.abs().max().clamp(min=1e-12) / 448.0).to(torch.float32)
            assert s[i, j].item() == sc.item()
            ref = (blk / sc).to(torch.float8_e4m3fn).view(torch.uint8)
            assert torch.equal(q[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128], ref)


def test_act_quant_closed_form():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 256, generator=g).to(torch.bfloat16)
    q, s = O.act_quant_per_token_group(x)
    assert q.shape == (5, 256) and s.shape == (5, 2)
    for m in range(5):
        for gidx in range(2):
            seg = x[m, gidx * 128:(gidx + 1) * 128].float()
            sc = seg.abs().max() / 448.0
            assert s[m, gidx].item() == sc.item()
            # the largest element lands exactly on +-448
            assert O.e4m3_decode(q[m, gidx * 128:(gidx + 1) * 128]).abs().max().item() == 448.0
    back = O.act_dequant_per_token_group(q, s)
    assert ((back - x.float()).abs() <= 0.0625 * x.float().abs() + 2.0 ** -9 * s.max()).all()


# ---------------------------------------------------------------- Q4_K
def test_q4k_scale_field_all_encodings():
    # every (sc6, mn6) pair in each of the 8 slots survives pack -> get_scale_min_k4
    sc = np.arange(64, dtype=np.uint8)
    a, b = np.meshgrid(sc, sc, indexing="ij")
    for j in range(8):
        sc6 = np.zeros((64 * 64, 8), dtype=np.uint8)
        mn6 = np.zeros_like(sc6)
        sc6[:, j] = a.ravel()
        mn6[:, j] = b.ravel()
        # fill the other slots with a pattern so cross-talk between slots shows
        for o in range(8):
            if o != j:
                sc6[:, o] = (17 * o + 5) % 64
                mn6[:, o] = (29 * o + 11) % 64
        f = O.q4k_pack_scales(sc6, mn6)
        s2, m2 = O.q4k_unpack_scales(f)
        assert np.array_equal(s2, sc6) and np.array_equal(m2, mn6)


def test_q4k_scale_field_ggml_layout_known_bytes():
    # ggml get_scale_min_k4: j<4 -> q[j]&63, q[j+4]&63; j>=4 -> (q[j+4]&0xF)|((q[j-4]>>6)<<4), (q[j+4]>>4)|((q[j]>>6)<<4)
    f = np.array([[0xC1, 0x02, 0x03, 0x04, 0x85, 0x06, 0x07, 0x08, 0x2A, 0, 0, 0]], dtype=np.uint8)
    sc6, mn6 = O.q4k_unpack_scales(f)
    assert sc6[0, 0] == 1 and mn6[0, 0] == 5
    assert sc6[0, 4] == (0xA | (3 << 4)) and mn6[0, 4] == (0x2 | (2 << 4))


def test_q4k_hand_built_superblock():
    # d = 1, dmin = 0.5, sc6[j] = j + 1, mn6[j] = 2 j, element e of sub-block j has nibble (e + j) % 16
    q = np.zeros((1, 1, 256), dtype=np.uint8)
    for j in range(8):
        for p in range(32):
            q[0, 0, 32 * j + p] = (p + j) % 16
    sc6 = np.arange(1, 9, dtype=np.uint8).reshape(1, 1, 8)
    mn6 = (2 * np.arange(8, dtype=np.uint8)).reshape(1, 1, 8)
    raw = O.q4k_build_raw(q, sc6, mn6, np.array([[1.0]], np.float16), np.array([[0.5]], np.float16))
    assert raw.shape == (1, 144)
    # raw byte 16 + 32*il + p holds element 64 il + p (low) and 64 il + 32 + p (high)
    assert raw[0, 16 + 32 * 1 + 3] == (q[0, 0, 64 + 3] | (q[0, 0, 96 + 3] << 4))
    ql, sc, mn = O.q4k_repack(raw)
    assert ql.shape == (1, 128) and sc.shape == (1, 8) and mn.shape == (1, 8)
    assert np.array_equal(sc[0], np.arange(1, 9, dtype=np.float16))
    assert np.array_equal(mn[0], np.arange(8, dtype=np.float16))
    # ql byte j: element 2j low, 2j+1 high
    assert ql[0, 5] == (q[0, 0, 10] | (q[0, 0, 11] << 4))
    w = O.q4k_dequant(ql, sc, mn)
    for j in range(8):
        for p in range(32):
            assert w[0, 32 * j + p] == np.float16((j + 1) * ((p + j) % 16) - j)


def test_q4k_repack_dequant_equals_direct_walk():
    x, raw = O.make_q4k_case(1, 512, 6, seed=7)
    ql, sc, mn = O.q4k_repack(raw)
    assert np.array_equal(O.q4k_dequant(ql, sc, mn), O.q4k_dequant_from_raw(raw))


def test_q4k_two_roundings_not_fused():
    # a case where fma(nib, s, -m) and round(round(nib*s) - m) differ
    s = np.float16(0.0123)
    m = np.float16(0.0777)
    found = False
    for nib in range(16):
        two = np.float16(np.float16(np.float16(nib) * s) - m)
        one = np.float16(np.float64(nib) * np.float64(s) - np.float64(m))
        ql = np.array([[nib] + [0] * 15], dtype=np.uint8)
        w = O.q4k_dequant(ql, np.array([[s]], np.float16), np.array([[m]], np.float16))
        assert w[0, 0] == two
        found |= (two != one)
    assert found
    # and torch's eager fp16 ops give the same two-rounding value
    nibt = torch.arange(16, dtype=torch.float16)
    tw = nibt * torch.tensor(float(s), dtype=torch.float16) - torch.tensor(float(m), dtype=torch.float16)
    for nib in range(16):
        assert tw[nib].item() == float(np.float16(np.float16(np.float16(nib) * s) - m))


# ---------------------------------------------------------------- MoE routing
def test_topk_bruteforce_small():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(6, 8, generator=g).to(torch.float16)
    logits[2, 3] = logits[2, 5]                     # a tie: index 3 must come first
    logits[4, :] = 0.25                             # all equal: ids 0,1,2
    w, ids = O.moe_topk(logits, 3)
    for t in range(6):
        row = logits[t].float().tolist()
        order = sorted(range(8), key=lambda i: (-row[i], i))[:3]
        assert ids[t].tolist() == order
        p = np.exp(np.array(row, dtype=np.float64) - max(row))
        p /= p.sum()
        sel = p[order] / p[order].sum()
        assert np.allclose(w[t].float().numpy(), sel, atol=1e-3)
        assert len(set(ids[t].tolist())) == 3
    assert abs(float(w.float().sum(-1).mean()) - 1.0) < 2e-3
    assert ids[4].tolist() == [0, 1, 2]


def test_sort_fixture_and_invariants():
    with open(os.path.join(GOLD, "routing_4tok_8exp.json")) as f:
        fx = json.load(f)
    ids = torch.tensor(fx["top_ids"], dtype=torch.int32)
    order, start, inv = O.moe_sort(ids, fx["num_experts"])
    assert order.tolist() == fx["sorted_pairs"]
    assert start.tolist() == fx["expert_start"]
    assert inv.tolist() == fx["inv"]
    # invariants: permutation, grouped by expert, stable inside an expert
    flat = ids.reshape(-1)
    assert sorted(order.tolist()) == list(range(flat.numel()))
    e_sorted = flat[order.long()]
    assert torch.all(e_sorted[1:] >= e_sorted[:-1])
    for e in range(fx["num_experts"]):
        seg = order[start[e]:start[e + 1]]
        assert torch.all(seg[1:] > seg[:-1])
    assert torch.equal(inv[order.long()], torch.arange(flat.numel(), dtype=torch.int32))


def test_sort_matches_reference_counting_sort():
    # build_sorted_token_ids, V/csrc/xpu/esimd_kernels/moe_ops.h:238-260, as plain loops
    g = torch.Generator().manual_seed(6)
    T, k, E = 37, 4, 16
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    count = [0] * E
    for t in range(T):
        for j in range(k):
            count[int(ids[t, j])] += 1
    start = [0]
    for e in range(E):
        start.append(start[-1] + count[e])
    pos = start[:-1].copy()
    sorted_ids = [0] * (T * k)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            sorted_ids[pos[e]] = t * k + j
            pos[e] += 1
    order, st, inv = O.moe_sort(ids, E)
    assert order.tolist() == sorted_ids and st.tolist() == start


def test_moe_grouped_equals_per_token_loop():
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(5, 8, 2, 256, 128, seed=11)
    tw, ids = O.moe_topk(logits, 2)
    for aq in (False, True):
        a = O.moe_forward(x, tw, ids, w13q, w13s, w2q, w2s, act_quant=aq)
        b = O.moe_forward_grouped(x, tw, ids, w13q, w13s, w2q, w2s, 8, act_quant=aq)
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)


def test_silu_mul_gate_is_first_half():
    gu = torch.tensor([[0.0, 100.0, 3.0, 5.0]])
    out = O.silu_mul(gu)
    assert out[0, 0].item() == 0.0 and abs(out[0, 1].item() - 500.0) < 1e-3


def test_matmul_ref_orientation():
    x = torch.tensor([[1.0, 2.0, 3.0]])
    w = torch.tensor([[1.0, 0.0, 0.0], [0.0, 0.0, 1.0]])
    assert O.matmul_ref(x, w).tolist() == [[1.0, 3.0]]


def test_moe_forward_full_oracle_against_dense_formulation():
    """The per-token loop of moe_forward_full must equal a dense restatement: every expert's
    output computed for every token, masked by the routing matrix (no loop shared with the
    oracle), plus the gated shared expert.  A transposed weight, a missing renormalisation or
    a gate applied to the wrong term fails this."""
    g = torch.Generator().manual_seed(5)
    T, E, H, I, k = 5, 8, 128, 128, 3
    x = (torch.randn(T, H, generator=g) * 0.2).half()
    logits = (torch.randn(T, E, generator=g) * 0.4).half()
    w13, s13 = O.fp8_quantize_block(torch.randn(E, 2 * I, H, generator=g) * 0.15)
    w2, s2 = O.fp8_quantize_block(torch.randn(E, H, I, generator=g) * 0.15)
    sw13, ss13 = O.fp8_quantize_block(torch.randn(2 * I, H, generator=g) * 0.15)
    sw2, ss2 = O.fp8_quantize_block(torch.randn(H, I, generator=g) * 0.15)
    gate = (torch.randn(1, H, generator=g) * 0.1).half()
    got = O.moe_forward_full(x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate, k)
    # dense restatement with library routines
    probs = torch.softmax(logits.float(), -1)
    tw, ti = torch.topk(probs, k, dim=-1)                     # no ties in this random case
    tw = tw / tw.sum(-1, keepdim=True)
    route = torch.zeros(T, E).scatter_(1, ti, tw)             # [T, E] routing weights
    d13 = w13.view(torch.float8_e4m3fn).float() * s13.repeat_interleave(128, -2).repeat_interleave(128, -1)
    d2 = w2.view(torch.float8_e4m3fn).float() * s2.repeat_interleave(128, -2).repeat_interleave(128, -1)
    gu = torch.einsum("th,enh->ten", x.float(), d13)          # [T, E, 2I]
    inter = torch.nn.functional.silu(gu[..., :I]) * gu[..., I:]
    ye = torch.einsum("tei,ehi->teh", inter, d2)              # [T, E, H]
    want = (route.unsqueeze(-1) * ye).sum(1)
    ds13 = sw13.view(torch.float8_e4m3fn).float() * ss13.repeat_interleave(128, -2).repeat_interleave(128, -1)
    ds2 = sw2.view(torch.float8_e4m3fn).float() * ss2.repeat_interleave(128, -2).repeat_interleave(128, -1)
    sgu = x.float() @ ds13.t()
    sh = (torch.nn.functional.silu(sgu[:, :I]) * sgu[:, I:]) @ ds2.t()
    want = want + torch.sigmoid(x.float() @ gate.float().t()) * sh
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_moe_prefill_scalar_is_the_block_scaled_forward_with_constant_blocks():
    """Per-expert scalar scales are the special case of 128x128 block scales in which every block of
    the gate half, of the up half and of the down weight carries one value: the scalar-scale oracle
    must agree with the (independently pinned) block-scale dequantisation + dense routing algebra."""
    g = torch.Generator().manual_seed(11)
    T, E, H, I, k = 6, 4, 128, 128, 2
    x = (torch.randn(T, H, generator=g) * 0.3).half()
    tw, ti = O.moe_topk(torch.randn(T, E, generator=g).half(), k)
    w13 = torch.randint(0, 120, (E, 2 * I, H), generator=g, dtype=torch.int32).to(torch.uint8)
    w2 = torch.randint(0, 120, (E, H, I), generator=g, dtype=torch.int32).to(torch.uint8)
    s13 = torch.rand(E, 2, generator=g) * 1e-3 + 1e-4
    s2 = torch.rand(E, generator=g) * 1e-3 + 1e-4
    got, inter, y = O.moe_prefill_scalar(x, tw, ti, w13, s13, w2, s2, return_parts=True)
    b13 = s13.view(E, 2, 1).expand(E, 2, H // 128).reshape(E, 2 * I // 128, H // 128)
    b2 = s2.view(E, 1, 1).expand(E, H // 128, I // 128)
    d13, d2 = O.fp8_dequant_block(w13, b13), O.fp8_dequant_block(w2, b2)
    route = torch.zeros(T, E).scatter_(1, ti.long(), tw.float())
    gu = torch.einsum("th,enh->ten", x.float(), d13)
    it = torch.nn.functional.silu(gu[..., :I]) * gu[..., I:]
    want = (route.unsqueeze(-1) * torch.einsum("tei,ehi->teh", it, d2)).sum(1)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-7)
    assert inter.shape == (T * k, I) and y.shape == (T * k, H)
    # pair order: row t*k + j belongs to token t
    e = int(ti[3, 1])
    assert torch.allclose(inter[3 * k + 1], it[3, e], rtol=1e-4, atol=1e-7)


def test_rmsnorm_oracle_against_library_and_hand_values():
    """rms_norm of the library for the plain case; hand values for the residual and gated forms."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 64, generator=g).half()
    w = torch.rand(64, generator=g).half()
    got, none = O.rmsnorm(x, w, 1e-6)
    assert none is None
    want = torch.nn.functional.rms_norm(x.float(), (64,), w.float(), 1e-6)
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-7)
    # residual: a = x + r = [3, 4] -> rms = sqrt(12.5); gate z = 0 -> silu(0) = 0 kills the output
    xs, rs = torch.tensor([[1.0, 1.0]]).half(), torch.tensor([[2.0, 3.0]]).half()
    ws = torch.tensor([1.0, 2.0]).half()
    n, nr = O.rmsnorm(xs, ws, 0.0, residual=rs)
    assert torch.equal(nr, torch.tensor([[3.0, 4.0]]).half())
    assert torch.allclose(n, torch.tensor([[3.0 / 12.5 ** 0.5, 8.0 / 12.5 ** 0.5]]), rtol=1e-6)
    n0, _ = O.rmsnorm(xs, ws, 0.0, gate=torch.zeros(1, 2).half())
    assert torch.equal(n0, torch.zeros(1, 2))
    # heads: each head of len(weight) elements is normalised on its own
    xh = torch.tensor([[3.0, 4.0, 6.0, 8.0]]).half()
    nh, _ = O.rmsnorm(xh, torch.ones(2).half(), 0.0, heads=2)
    assert torch.allclose(nh, torch.tensor([[3 / 12.5 ** 0.5, 4 / 12.5 ** 0.5, 6 / 50 ** 0.5, 8 / 50 ** 0.5]]), rtol=1e-6)


def test_gelu_tanh_mul_closed_form():
    # the tanh form written out (exp-based tanh as the reference's kernel computes it), gate = first half
    gu = torch.tensor([[0.0, 1.0, -2.0, 3.0, 2.0, 2.0, 2.0, 0.5]])
    out = O.gelu_tanh_mul(gu)
    g = gu[0, :4].double()
    z = 0.7978845608 * (g + 0.044715 * g ** 3)
    e = torch.exp(2 * z)
    exp = 0.5 * g * (1 + (e - 1) / (e + 1)) * gu[0, 4:].double()
    assert torch.allclose(out[0].double(), exp, rtol=1e-6, atol=1e-7)
    assert out[0, 0] == 0 and abs(out[0, 1].item() - 0.8411920 * 2.0) < 1e-5    # gelu_tanh(1) = 0.841192


def test_moe_forward_full_kmajor_against_block_oracle():
    """The K-major per-tensor forward equals the (separately pinned) block-scaled forward on the
    transposed weights with every block of expert e carrying scale[e]: a transposed index, a scale
    taken from the wrong expert or a gate / up swap fails this."""
    g = torch.Generator().manual_seed(6)
    T, E, H, I, k = 4, 6, 256, 128, 2
    x = (torch.randn(T, H, generator=g) * 0.2).half()
    logits = (torch.randn(T, E, generator=g) * 0.4).half()
    w13 = O.e4m3_quantize(torch.randn(E, H, 2 * I, generator=g))           # K-major
    w2 = O.e4m3_quantize(torch.randn(E, I, H, generator=g))
    s13 = 0.01 * (1 + torch.rand(E, generator=g))
    s2 = 0.01 * (1 + torch.rand(E, generator=g))
    sw13 = O.e4m3_quantize(torch.randn(2 * I, H, generator=g))
    sw2 = O.e4m3_quantize(torch.randn(H, I, generator=g))
    ss13, ss2 = torch.tensor([0.013]), torch.tensor([0.017])
    gate = (torch.randn(1, H, generator=g) * 0.1).half()
    got = O.moe_forward_full_kmajor(x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate, k)
    blk = lambda sc, n, kk: sc.reshape(-1, 1, 1).expand(-1, n // 128, kk // 128).contiguous()
    want = O.moe_forward_full(x, logits, w13.transpose(1, 2).contiguous(), blk(s13, 2 * I, H), sw13,
                              ss13.expand(2 * I // 128, H // 128).contiguous(), w2.transpose(1, 2).contiguous(),
                              blk(s2, H, I), sw2, ss2.expand(H // 128, I // 128).contiguous(), gate, k)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


# ---- K-major W4A16 operands (the reference's int4_gemm_w4a16 call) ----
def test_w4a16_kmajor_matches_the_esimd_bytes():
    """vllm/patches/vllm_for_multi_arc.patch:5516-5523: the [K/8, N] tensor with strides (1, K/8)
    is the N-major ESIMD weight, byte for byte; so the transposed K-major words must equal the
    int32 view of int4_pack's bytes."""
    g = torch.Generator().manual_seed(3)
    N, K = 24, 256
    q = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    packed = O.int4_pack(q)
    scale = (torch.rand(N, K // 128, generator=g) * 0.01 + 0.005).half()
    zp = torch.randint(0, 16, (N, K // 128), generator=g, dtype=torch.int32).to(torch.uint8)
    qw, sc, qz = O.w4a16_kmajor_pack(q + 8, scale, zp)
    assert qw.shape == (K // 8, N) and sc.shape == (K // 128, N) and qz.shape == (K // 128, N // 8)
    assert torch.equal(qw.t().contiguous(), packed.view(torch.int32))
    u4, s2, z2 = O.w4a16_kmajor_unpack(qw, sc, qz)
    assert torch.equal(u4, q + 8) and torch.equal(s2, scale) and torch.equal(z2, zp)
    assert torch.equal(O.w4a16_kmajor_dequant(qw, sc, qz), O.int4_dequant(packed, scale, zp=zp))
    # symmetric form: one value for every group
    assert torch.equal(O.w4a16_kmajor_dequant(qw, sc, torch.tensor([8], dtype=torch.int32)), O.int4_dequant(packed, scale))


def test_w4a16_kmajor_hand_placed_nibbles():
    N, K = 16, 128
    u4 = torch.zeros(N, K, dtype=torch.int32)
    u4[5, 13] = 0xF                              # k = 13 = 8 * 1 + 5: word (1, 5), nibble 5
    u4[0, 7] = 0x9                               # the top nibble of word (0, 0): sign bit set
    zp = torch.zeros(N, 1, dtype=torch.uint8)
    zp[11, 0] = 9                                # column 11 = 8 * 1 + 3: word (0, 1), nibble 3
    qw, sc, qz = O.w4a16_kmajor_pack(u4, torch.ones(N, 1).half(), zp)
    assert qw[1, 5].item() == 0x00F00000 and qw[0, 0].item() == 0x90000000 - (1 << 32)
    assert int((qw != 0).sum()) == 2
    assert qz[0, 1].item() == 9 << 12 and int((qz != 0).sum()) == 1
    w = O.w4a16_kmajor_dequant(qw, sc, qz, out_dtype=torch.float32)
    assert w[5, 13].item() == 15.0 and w[0, 7].item() == 9.0 and w[11, 0].item() == -9.0 and w[11, 127].item() == -9.0
    assert O.w4a16_kmajor_unpack(qw, sc, qz, zero_bias=1)[2][11, 0].item() == 10
