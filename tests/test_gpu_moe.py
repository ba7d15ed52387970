"""GPU parity for the MoE path: routing ids and the expert-sorted permutation are
bit-exact against the oracle; activation quantisation codes and scales are
bit-exact; grouped GEMMs and the full forward are within max relative error
1e-2 (denominator floored at the mean magnitude) of the oracle that quantises
the same activations."""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def s(dev):
    import custom_esimd_kernels_sglang as sg
    return sg


@pytest.fixture(scope="module")
def v(dev):
    import custom_esimd_kernels_vllm as mod
    return mod


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("T,E,K,dt", [(512, 128, 8, torch.bfloat16), (7, 16, 4, torch.float16),
                                      (33, 64, 6, torch.float16), (5, 256, 8, torch.bfloat16),
                                      (3, 8, 8, torch.float16), (1, 1024, 2, torch.float16)])
def test_topk_ids_exact_weights_close(v, dev, T, E, K, dt):
    g = torch.Generator().manual_seed(T * 131 + E)
    logits = torch.randn(T, E, generator=g).to(dt)
    if T > 2 and E >= 8:
        logits[1, 5] = logits[1, 2]                 # a tie inside the top range
        logits[1, 2] = logits[1].max()
        logits[1, 5] = logits[1, 2]
        logits[2, :] = 0.5                          # all equal: ids 0..K-1
    tw = torch.empty(T, K, dtype=dt, device=dev)
    ti = torch.empty(T, K, dtype=torch.int32, device=dev)
    r = v.esimd_moe_topk(logits.to(dev), tw, ti, T)
    assert r.data_ptr() == tw.data_ptr()
    rw, ri = O.moe_topk(logits, K)
    assert torch.equal(ti.cpu(), ri)
    ulp = 2.0 ** -8 if dt == torch.bfloat16 else 2.0 ** -11
    assert ((tw.cpu().float() - rw.float()).abs() <= 2 * ulp * rw.float().abs() + 1e-7).all()
    w2, i2 = v.moe_topk(logits.to(dev), K, True)
    assert torch.equal(i2.cpu(), ri) and torch.equal(w2, tw)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_topk_signed_zero_ties(v, dev, dt):
    """+0 and -0 logits are equal to a float compare, so the lowest index wins among them
    (V/csrc/xpu/esimd_kernels/moe_ops.h:77-104): a -0 at a lower index must beat a +0 further on."""
    T, E, K = 4, 64, 4
    logits = torch.full((T, E), -1.0).to(dt)
    logits[0, 3], logits[0, 9], logits[0, 20], logits[0, 40], logits[0, 50] = -0.0, 0.0, -0.0, 0.0, 0.0
    logits[1, :] = -0.0
    logits[1, 7], logits[1, 30] = 0.0, 0.0
    logits[2, 10], logits[2, 11] = 2.0, 2.0
    logits[2, 60], logits[2, 61], logits[2, 62] = 0.0, -0.0, 0.0
    logits[2, 5] = -0.0
    logits[3, :] = 0.0
    logits[3, 0] = -0.0
    tw = torch.empty(T, K, dtype=dt, device=dev)
    ti = torch.empty(T, K, dtype=torch.int32, device=dev)
    v.esimd_moe_topk(logits.to(dev), tw, ti, T)
    rw, ri = O.moe_topk(logits, K, out_dtype=dt)
    assert ri.tolist() == [[3, 9, 20, 40], [0, 1, 2, 3], [10, 11, 5, 60], [0, 1, 2, 3]]
    assert torch.equal(ti.cpu(), ri)
    ulp = 2.0 ** -8 if dt == torch.bfloat16 else 2.0 ** -11
    assert ((tw.cpu().float() - rw.float()).abs() <= 2 * ulp * rw.float().abs() + 1e-7).all()


def test_topk_v2_matches_topk(v, dev):
    T, E, K = 9, 128, 8
    logits = torch.randn(T, E, generator=torch.Generator().manual_seed(5)).half().to(dev)
    tw = torch.empty(T, K, dtype=torch.float16, device=dev)
    ti = torch.empty(T, K, dtype=torch.int32, device=dev)
    r = torch.ops.esimd_topk_v2.topk_v2(logits, tw, ti, T, E, K)
    assert r.data_ptr() == tw.data_ptr()
    rw, ri = O.moe_topk(logits.cpu(), K)
    assert torch.equal(ti.cpu(), ri)
    assert ((tw.cpu().float() - rw.float()).abs() <= 2 * 2.0 ** -11 * rw.float().abs() + 1e-7).all()
    with pytest.raises(RuntimeError):
        torch.ops.esimd_topk_v2.topk_v2(logits, tw, ti, T, E + 1, K)


@pytest.mark.parametrize("T,E,H,dt", [(1, 128, 2048, torch.float16), (4, 64, 512, torch.float16), (12, 256, 1024, torch.bfloat16)])
def test_moe_router_forward(v, dev, T, E, H, dt):
    """logits = x @ (scale * e4m3(w))^T (V/csrc/moe_batch/moe.sycl:302-358)."""
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=g).to(dt)
    w8 = O.e4m3_quantize(torch.randn(E, H, generator=g).clamp(-3, 3) / 3)
    sc = torch.tensor([0.037], dtype=torch.float32)
    got = torch.ops.moe_ops.moe_router_forward(x.to(dev), w8.view(torch.float8_e4m3fn).to(dev), sc.to(dev))
    assert got.shape == (T, E) and got.dtype == dt
    want = (x.float() @ O.e4m3_decode(w8).t()) * sc[0]
    assert O.max_rel_err(got.cpu().float(), want) < TOL


@pytest.mark.parametrize("T,k,ns,H,dt", [(1, 8, 1, 2048, torch.float16), (5, 2, 0, 136, torch.bfloat16), (0, 4, 1, 64, torch.float16)])
def test_moe_accumulate(v, dev, T, k, ns, H, dt):
    """Unweighted fp32 sum over each token's top_k + shared rows, one rounding
    (V/csrc/moe_batch/moe.sycl:1177-1230)."""
    rows = k + ns
    p = torch.randn(T * rows, H, generator=torch.Generator().manual_seed(T + H)).to(dt)
    got = torch.ops.moe_ops.moe_accumulate(p.to(dev), k, ns)
    assert got.shape == (T, H) and got.dtype == dt
    want = p.float().reshape(T, rows, H).sum(1).to(dt)
    assert torch.equal(got.cpu(), want) or (got.cpu().float() - want.float()).abs().max() <= 2.0 ** -7 * want.float().abs().max()


@pytest.mark.parametrize("T,E,K", [(512, 128, 8), (1, 8, 2), (37, 16, 4), (4096, 128, 8), (300, 1000, 6),
                                   (2500, 64, 2), (0, 8, 2)])
def test_sort_bit_exact(v, dev, T, E, K):
    g = torch.Generator().manual_seed(T + E + K)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(max(T, 1))])[:T].to(torch.int32).reshape(T, K)
    if T >= 20:
        for t in range(T // 2):                     # skew: half the tokens route to expert 3
            if 3 not in ids[t].tolist():
                ids[t, 0] = 3
        assert all(len(set(ids[t].tolist())) == K for t in range(min(T, 50)))
    P = T * K
    sp = torch.full((max(P, 1),), -1, dtype=torch.int32, device=dev)
    st = torch.full((E + 1,), -1, dtype=torch.int32, device=dev)
    inv = torch.full((max(P, 1),), -1, dtype=torch.int32, device=dev)
    tok = torch.full((max(P, 1),), -1, dtype=torch.int32, device=dev)
    mx = torch.full((1,), -1, dtype=torch.int32, device=dev)
    v.moe_sort(ids.to(dev), E, sp, st, inv, tok, mx)
    ro, rs, ri = O.moe_sort(ids, E)
    assert torch.equal(st.cpu(), rs)
    assert torch.equal(sp.cpu()[:P], ro)
    assert torch.equal(inv.cpu()[:P], ri)
    assert torch.equal(tok.cpu()[:P], ro // K)
    assert int(mx.cpu()) == int((rs[1:] - rs[:-1]).max())


@pytest.mark.parametrize("T,E,K", [(40, 16, 4), (3000, 32, 2)])
def test_sort_bad_ids_stay_in_bounds(v, dev, T, E, K):
    # ids a top-k selection never produces (out of range, repeated inside a token) give unspecified
    # results for their tokens, but every index the sort writes stays valid and the other tokens'
    # experts keep their pairs (single-pass and chunked path)
    g = torch.Generator().manual_seed(T)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    ids[1, 0] = -7
    ids[2, 1] = E + 100
    ids[3, :] = 5                                   # one expert K times
    ids[T - 1, 0] = ids[T - 1, 1]
    P = T * K
    sp = torch.full((P,), -1, dtype=torch.int32, device=dev)
    st = torch.full((E + 1,), -1, dtype=torch.int32, device=dev)
    inv = torch.full((P,), -1, dtype=torch.int32, device=dev)
    tok = torch.full((P,), -1, dtype=torch.int32, device=dev)
    v.moe_sort(ids.to(dev), E, sp, st, inv, tok)
    sp, st, inv, tok = sp.cpu(), st.cpu(), inv.cpu(), tok.cpu()
    assert st[0] == 0 and bool((st[1:] >= st[:-1]).all()) and int(st[E]) <= P
    assert bool(((sp >= 0) & (sp < P)).all()) and bool(((inv >= 0) & (inv < P)).all())
    assert bool(((tok >= 0) & (tok < T)).all())
    good = [t for t in range(T) if t not in (1, 2, 3, T - 1)]
    for t in good[:64]:
        for j in range(K):
            pos = int(inv[t * K + j])
            e = int(ids[t, j])
            assert int(st[e]) <= pos < int(st[e + 1]) and int(sp[pos]) == t * K + j and int(tok[pos]) == t


def test_sort_golden_fixture(v, dev):
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "routing_4tok_8exp.json")) as f:
        fx = json.load(f)
    ids = torch.tensor(fx["top_ids"], dtype=torch.int32)
    sp = torch.empty(8, dtype=torch.int32, device=dev)
    st = torch.empty(9, dtype=torch.int32, device=dev)
    inv = torch.empty(8, dtype=torch.int32, device=dev)
    v.moe_sort(ids.to(dev), 8, sp, st, inv)
    assert sp.cpu().tolist() == fx["sorted_pairs"]
    assert st.cpu().tolist() == fx["expert_start"]
    assert inv.cpu().tolist() == fx["inv"]


def test_scatter_fused_and_gather_roundtrip(v, dev):
    # scatter rows by expert, then gather with weights: final[t] = sum_j w[t,j] * x[t] = x[t] (weights sum to 1)
    T, E, K, H = 50, 16, 4, 256
    g = torch.Generator().manual_seed(9)
    x = torch.randn(T, H, generator=g).to(torch.float16)
    logits = torch.randn(T, E, generator=g).to(torch.float16)
    tw, ti = O.moe_topk(logits, K)
    sh = torch.empty(T * K, H, dtype=torch.float16, device=dev)
    sw = torch.empty(T * K, dtype=torch.float16, device=dev)
    topk_ids = torch.empty(T * K, dtype=torch.int32, device=dev)
    est = torch.empty(E + 1, dtype=torch.int32, device=dev)
    mx = torch.empty(1, dtype=torch.int32, device=dev)
    v.esimd_moe_scatter_fused(x.to(dev), tw.to(dev), ti.to(dev), sh, sw, topk_ids, est, mx, H, K, T, E)
    order, start, inv = O.moe_sort(ti, E)
    assert torch.equal(est.cpu(), start) and torch.equal(topk_ids.cpu(), inv)
    assert torch.equal(sh.cpu(), x[(order // K).long()])
    assert torch.equal(sw.cpu(), tw.reshape(-1)[order.long()])
    out = torch.empty(T, H, dtype=torch.float16, device=dev)
    v.esimd_moe_gather(sh, topk_ids.reshape(T, K), sw, out, H, K, T)
    ref = (tw.float().sum(-1, keepdim=True) * x.float())
    assert O.max_rel_err(out.cpu(), ref) < 5e-3


# ------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_act_quant_bit_exact(v, dev, dt):
    g = torch.Generator().manual_seed(13)
    x = (torch.randn(77, 768, generator=g) * torch.rand(77, 1, generator=g) * 3).to(dt)
    x[3, :128] = 0                                   # an all-zero group
    x[4, 5] = 1e-30 if dt == torch.bfloat16 else 6e-8
    q = torch.empty(77, 768, dtype=torch.uint8, device=dev)
    s = torch.empty(77, 6, dtype=torch.float32, device=dev)
    v.act_quant_fp8(x.to(dev), q, s)
    rq, rs = O.act_quant_per_token_group(x)
    assert torch.equal(s.cpu(), rs)
    assert torch.equal(q.cpu(), rq)


def test_silu_mul(v, dev):
    g = torch.Generator().manual_seed(14)
    x = (torch.randn(37, 512, generator=g) * 3).to(torch.bfloat16)
    out = torch.empty(37, 256, dtype=torch.bfloat16, device=dev)
    v.esimd_moe_silu_mul(x.to(dev), out, 512, 256, 37)
    ref = O.silu_mul(x)
    assert O.max_rel_err(out.cpu(), ref) < 8e-3     # bf16 output rounding is 2^-9


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("gelu", [False, True])
def test_act_mul_vector_and_element_paths_agree(v, dev, dt, gelu):
    """act(gate) * up runs eight columns per thread when the width and the alignment allow 16-byte accesses and
    element-wise otherwise; the same input through both (the second from a buffer that starts 2 bytes off) must
    give identical bits, and both must match the oracle."""
    rows, I = 301, 264
    g = torch.Generator().manual_seed(16 + gelu)
    x = (torch.randn(rows, 2 * I, generator=g) * 3).to(dt)
    fn = v.esimd_moe_gelu_tanh_mul if gelu else v.esimd_moe_silu_mul
    out = torch.empty(rows, I, dtype=dt, device=dev)
    fn(x.to(dev), out, 2 * I, I, rows)
    buf = torch.empty(rows * 2 * I + 8, dtype=dt, device=dev)
    xin = buf[1:1 + rows * 2 * I].view(rows, 2 * I)
    xin.copy_(x)
    assert xin.data_ptr() % 16 != 0
    out2 = torch.empty(rows, I, dtype=dt, device=dev)
    fn(xin, out2, 2 * I, I, rows)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    ref = O.gelu_tanh_mul(x) if gelu else O.silu_mul(x)
    assert O.max_rel_err(out.cpu(), ref) < (8e-3 if dt == torch.bfloat16 else 2e-3)


def test_gelu_tanh_mul(v, dev):
    g = torch.Generator().manual_seed(15)
    x = (torch.randn(29, 384, generator=g) * 3).half()
    x[0, :8] = torch.tensor([40.0, -40.0, 11.5, -11.5, 0.0, 1e-4, 60000.0, -60000.0]).half()   # saturating gates
    x[0, 192:200] = 1.0
    out = torch.empty(29, 192, dtype=torch.float16, device=dev)
    v.esimd_moe_gelu_tanh_mul(x.to(dev), out, 384, 192, 29)
    ref = O.gelu_tanh_mul(x)
    assert torch.isfinite(out.cpu().float()).all()
    assert out[0, 1].item() == 0.0 and out[0, 7].item() == 0.0          # gelu(-large) = -0
    assert O.max_rel_err(out.cpu(), ref) < 2e-3


# ------------------------------------------------------------------ grouped GEMM
def _grouped_ref(x, dw, counts):
    ref = torch.empty(x.shape[0], dw.shape[1], dtype=torch.float32)
    s = 0
    for e, c in enumerate(counts):
        ref[s:s + c] = x[s:s + c].float() @ dw[e].t()
        s += c
    return ref


def test_moe_gemm_w8a16_reference_case(v, dev):
    # V/tests/test_fp8_blockscale_moe_prefill.py:93-144: 4 experts, counts 33/40/27/36, n = k = 256
    torch.manual_seed(20260713)
    experts, n, k = 4, 256, 256
    counts = [33, 40, 27, 36]
    offsets = torch.tensor([0, 33, 73, 100, 136], dtype=torch.int32)
    x = (torch.randn(136, k) * 0.2).half()
    w8, ws = O.fp8_quantize_block(torch.randn(experts, n, k) * 0.15)
    out = torch.empty(136, n, dtype=torch.float16, device=dev)
    v.esimd_moe_gemm_fp8_blockscale(x.to(dev), w8.view(torch.float8_e4m3fn).to(dev), ws.to(dev), out,
                                    offsets.to(dev), n, k, experts)
    ref = _grouped_ref(x, O.fp8_dequant_block(w8, ws), counts)
    o = out.cpu().float()
    assert O.max_rel_err(o, ref) < TOL
    mean_rel = ((o - ref).abs().mean() / ref.abs().mean()).item()
    assert mean_rel < 3e-3                           # the reference's own bar


@pytest.mark.parametrize("total", [1, 128])
def test_moe_gemm_all_e4m3_codes_exact(v, dev, total):
    # V/tests/test_fp8_blockscale_moe_prefill.py:54-90
    raw = torch.arange(256, dtype=torch.uint8).view(1, 256, 1).expand(1, 256, 128).contiguous()
    reference = raw[0, :, 0].view(torch.float8_e4m3fn).float() * 128
    finite = torch.isfinite(reference)
    scale = torch.ones(1, 2, 1)
    x = torch.ones(total, 128, dtype=torch.float16)
    out = torch.empty(total, 256, dtype=torch.float16, device=dev)
    offsets = torch.tensor([0, total], dtype=torch.int32)
    v.esimd_moe_gemm_fp8_blockscale(x.to(dev), raw.to(dev), scale.to(dev), out, offsets.to(dev), 256, 128, 1, 128, 128)
    for row in (0, total - 1):
        actual = out[row].cpu().float()
        assert torch.equal(actual[finite], reference[finite])
        assert actual[0x80].item() == 0.0


@pytest.mark.parametrize("counts", [[0, 5, 0, 70, 1, 16, 17, 0], [33, 40, 27, 36], [300, 0, 129, 257]])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_moe_gemm_one_hot_rows_return_the_experts_weights(v, dev, counts, dt):
    """One 1.0 per activation row: every output of the grouped w8a16 GEMM is a single block-scaled weight of the
    row's expert rounded to the activation type — the streaming kernel (few rows per expert) and the grouped
    tiled GEMM (96 and more on average), value for value."""
    E, N, K = len(counts), 256, 512
    total = sum(counts)
    st = torch.zeros(E + 1, dtype=torch.int32)
    st[1:] = torch.tensor(counts).cumsum(0)
    g = torch.Generator().manual_seed(total)
    w8, ws = O.fp8_quantize_block(torch.randn(E, N, K, generator=g) * 0.05)
    dw = O.fp8_dequant_block(w8, ws).to(dt).float()           # [E, N, K]
    ks = (5 + 37 * torch.arange(total)) % K
    x = torch.zeros(total, K, dtype=dt)
    x[torch.arange(total), ks] = 1.0
    e_of = torch.repeat_interleave(torch.arange(E), torch.tensor(counts))
    out = torch.full((total, N), float("nan"), dtype=dt, device=dev)
    v.esimd_moe_gemm_fp8_blockscale(x.to(dev), w8.to(dev), ws.to(dev), out, st.to(dev), N, K, E)
    assert torch.equal(out.cpu().float(), dw[e_of, :, ks])


@pytest.mark.parametrize("counts", [[0, 5, 0, 70, 1, 16, 17, 0], [130, 0, 0, 3]])
@pytest.mark.parametrize("a8", [False, True])
def test_moe_gemm_skewed_experts(v, dev, counts, a8):
    E, N, K = len(counts), 272, 384                  # N not a multiple of 128: ragged scale rows
    g = torch.Generator().manual_seed(sum(counts) + a8)
    total = sum(counts)
    st = torch.zeros(E + 1, dtype=torch.int32)
    st[1:] = torch.tensor(counts).cumsum(0)
    x = torch.randn(total, K, generator=g).to(torch.bfloat16)
    w = torch.randn(E, 384, K, generator=g) * 0.05
    w8, ws = O.fp8_quantize_block(w)
    w8 = w8[:, :N].contiguous()
    dw = O.fp8_dequant_block(w8, ws)
    out = torch.empty(total, N, dtype=torch.bfloat16, device=dev)
    if a8:
        xq, xs = O.act_quant_per_token_group(x)
        v.moe_gemm_fp8_block(xq.to(dev), xs.to(dev), None, w8.to(dev), ws.to(dev), st.to(dev), out, N, K, E, False)
        ref = _grouped_ref(O.act_dequant_per_token_group(xq, xs), dw, counts)
    else:
        v.esimd_moe_gemm_fp8_blockscale(x.to(dev), w8.to(dev), ws.to(dev), out, st.to(dev), N, K, E)
        ref = _grouped_ref(x, dw, counts)
    assert O.max_rel_err(out.cpu(), ref) < TOL


@pytest.mark.parametrize("counts,dt,fuse,gather", [
    ([300, 0, 129, 257], torch.float16, False, False), ([97, 260, 100, 511, 16], torch.bfloat16, False, True),
    ([400, 33, 290], torch.bfloat16, True, True), ([256, 256, 256, 256], torch.float16, True, False),
    ([1, 0, 700], torch.float16, False, False)])
def test_moe_gemm_prefill_tiled(v, dev, counts, dt, fuse, gather):
    # experts averaging 96 rows or more (w8a16): the grouped launch of the tiled matrix-core GEMM, with
    # empty experts, partial last tiles, a row gather and the fused SiLU * up epilogue
    E, N, K = len(counts), 384, 512
    g = torch.Generator().manual_seed(sum(counts) + fuse)
    total = sum(counts)
    st = torch.zeros(E + 1, dtype=torch.int32)
    st[1:] = torch.tensor(counts).cumsum(0)
    nsrc = total // 2 if gather else total
    src = (torch.randn(nsrc, K, generator=g) * 0.5).to(dt)
    row_map = torch.randint(0, nsrc, (total,), generator=g).to(torch.int32) if gather else None
    x = src[row_map.long()] if gather else src
    w8, ws = O.fp8_quantize_block(torch.randn(E, N, K, generator=g) * 0.05)
    dw = O.fp8_dequant_block(w8, ws, out_dtype=dt)     # the block scale is folded into 16-bit weights on this path
    n_out = N // 2 if fuse else N
    out = torch.full((total, n_out), float("nan"), dtype=dt, device=dev)
    v.moe_gemm_fp8_block(src.to(dev), None, None if row_map is None else row_map.to(dev), w8.to(dev), ws.to(dev),
                         st.to(dev), out, N, K, E, fuse)
    ref = _grouped_ref(x, dw, counts)
    if fuse:
        ref = torch.nn.functional.silu(ref[:, :N // 2]) * ref[:, N // 2:]
    o = out.cpu()
    assert torch.isfinite(o.float()).all()
    assert O.max_rel_err(o, ref) < TOL


def test_moe_gemm_prefill_tiled_matches_streaming_kernel(v, dev):
    # the same problem through both grouped kernels (the streaming one keeps fp32 output): agreement
    # to the rounding of the 16-bit output and of the folded block scale
    counts = [200, 150, 333]
    E, N, K = len(counts), 256, 768
    g = torch.Generator().manual_seed(5)
    total = sum(counts)
    st = torch.zeros(E + 1, dtype=torch.int32)
    st[1:] = torch.tensor(counts).cumsum(0)
    x = (torch.randn(total, K, generator=g) * 0.5).half().to(dev)
    w8, ws = O.fp8_quantize_block(torch.randn(E, N, K, generator=g) * 0.05)
    a = torch.empty(total, N, dtype=torch.float16, device=dev)
    b = torch.empty(total, N, dtype=torch.float32, device=dev)
    v.moe_gemm_fp8_block(x, None, None, w8.to(dev), ws.to(dev), st.to(dev), a, N, K, E, False)
    v.moe_gemm_fp8_block(x, None, None, w8.to(dev), ws.to(dev), st.to(dev), b, N, K, E, False)
    assert O.max_rel_err(a.cpu(), b.cpu()) < 5e-3


# ------------------------------------------------------------------ full forward
@pytest.mark.parametrize("T,E,k,H,I,dt,skew,offset", [
    (512, 128, 8, 2048, 768, torch.bfloat16, False, 0),     # cfg3's gate_up
    (1, 8, 2, 256, 128, torch.float16, False, 0),
    (37, 16, 4, 384, 64, torch.float16, True, 0),           # 80 rows on one expert: two passes, empty experts
    (200, 4, 2, 256, 128, torch.bfloat16, True, 1),         # ids on a 4-byte boundary only (scalar id loads)
    (1024, 32, 8, 256, 48, torch.float16, True, 0),         # 8192 pairs: 32 per thread
])
def test_routed_gate_up_equals_sort_then_gemm(v, dev, T, E, k, H, I, dt, skew, offset):
    """The launch that sorts the pairs itself writes the same expert_start / inv / sorted_pairs as
    moe_sort (bit for bit, against the oracle's permutation too) and the same intermediate as the
    grouped GEMM on moe_sort's row map (same kernel arithmetic: bit-equal)."""
    g = torch.Generator().manual_seed(T * 7 + E + k)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if skew:
        for t in range(T // 2):
            if 3 % E not in ids[t].tolist():
                ids[t, 0] = 3 % E
        ids[::5, -1] = torch.where(ids[::5, -1] == 3 % E, ids[::5, -1], torch.full_like(ids[::5, -1], E + 7))  # out of range
    P = T * k
    x = (torch.randn(T, H, generator=g) * 0.5).to(dt)
    w = O.e4m3_quantize(torch.randn(E, 2 * I, H, generator=g) * 0.05)
    ws = torch.rand(E, (2 * I + 127) // 128, H // 128, generator=g) * 0.02 + 0.005
    xd, wd, wsd = x.to(dev), w.to(dev), ws.to(dev)
    xq = torch.empty(T, H, dtype=torch.uint8, device=dev)
    xs = torch.empty(T, H // 128, dtype=torch.float32, device=dev)
    v.act_quant_fp8(xd, xq, xs)
    buf = torch.zeros(P + 4, dtype=torch.int32, device=dev)
    ids_d = buf[offset:offset + P].view(T, k)
    ids_d.copy_(ids.to(dev))
    # separate sort + GEMM
    sp = torch.empty(P, dtype=torch.int32, device=dev)
    st = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    tok = torch.empty(P, dtype=torch.int32, device=dev)
    v.moe_sort(ids_d, E, sp, st, inv, tok)
    ref = torch.full((P, I), 7.0, dtype=dt, device=dev)
    v.moe_gemm_fp8_block(xq, xs, tok, wd, wsd, st, ref, 2 * I, H, E, True)
    # one launch
    sp2 = torch.full((P,), -1, dtype=torch.int32, device=dev)
    st2 = torch.full((E + 1,), -1, dtype=torch.int32, device=dev)
    inv2 = torch.full((P,), -1, dtype=torch.int32, device=dev)
    out = torch.full((P, I), 7.0, dtype=dt, device=dev)
    v.moe_gate_up_fp8_routed(xq, xs, ids_d, wd, wsd, st2, inv2, sp2, out, E)
    ro, rs, ri = O.moe_sort(ids.clamp(0, E - 1), E)
    assert torch.equal(st2.cpu(), rs) and torch.equal(st2, st)
    assert torch.equal(sp2.cpu(), ro) and torch.equal(inv2.cpu(), ri)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    # without the optional sorted_pairs
    out3 = torch.full((P, I), 7.0, dtype=dt, device=dev)
    v.moe_gate_up_fp8_routed(xq, xs, ids_d, wd, wsd, st2, inv2, None, out3, E)
    assert torch.equal(out3.view(torch.int16), ref.view(torch.int16))


def test_routed_gate_up_argument_errors(v, dev):
    T, E, k, H, I = 4, 8, 2, 256, 64
    xq = torch.zeros(T, H, dtype=torch.uint8, device=dev)
    xs = torch.ones(T, H // 128, dtype=torch.float32, device=dev)
    ids = torch.zeros(T, k, dtype=torch.int32, device=dev)
    w = torch.zeros(E, 2 * I, H, dtype=torch.uint8, device=dev)
    ws = torch.ones(E, 1, H // 128, dtype=torch.float32, device=dev)
    st = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(T * k, dtype=torch.int32, device=dev)
    out = torch.empty(T * k, I, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError, match="pairs"):
        big = torch.zeros(8192 // k + 1, k, dtype=torch.int32, device=dev)
        v.moe_gate_up_fp8_routed(xq, xs, big, w, ws, st, inv, None, out, E)
    with pytest.raises(RuntimeError, match="K="):
        v.moe_gate_up_fp8_routed(xq[:, :128].contiguous(), xs[:, :1].contiguous(), ids, w[:, :, :128].contiguous(),
                                 ws[:, :, :1].contiguous(), st, inv, None, out, E)
    with pytest.raises(RuntimeError, match="inv"):
        v.moe_gate_up_fp8_routed(xq, xs, ids, w, ws, st, inv[:3], None, out, E)


def _staged_forward(v, dev, x, logits, w13q, w13s, w2q, w2s, E, K, aq):
    """The fused op's own pipeline, run stage by stage through the same ops, so that the
    quantised intermediate is visible."""
    T, H = x.shape
    I = w2q.shape[-1]
    P = T * K
    dt = x.dtype
    xd = x.to(dev)
    tw = torch.empty(T, K, dtype=dt, device=dev)
    ti = torch.empty(T, K, dtype=torch.int32, device=dev)
    v.esimd_moe_topk(logits.to(dev), tw, ti, T)
    sp = torch.empty(P, dtype=torch.int32, device=dev)
    st = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    tok = torch.empty(P, dtype=torch.int32, device=dev)
    v.moe_sort(ti, E, sp, st, inv, tok)
    inter = torch.empty(P, I, dtype=dt, device=dev)
    y = torch.empty(P, H, dtype=torch.float32, device=dev)
    w13d, s13d, w2d, s2d = w13q.to(dev), w13s.to(dev), w2q.to(dev), w2s.to(dev)
    iq = isc = None
    if aq:
        xq = torch.empty(T, H, dtype=torch.uint8, device=dev)
        xs = torch.empty(T, H // 128, dtype=torch.float32, device=dev)
        v.act_quant_fp8(xd, xq, xs)
        v.moe_gemm_fp8_block(xq, xs, tok, w13d, s13d, st, inter, 2 * I, H, E, True)
        iq = torch.empty(P, I, dtype=torch.uint8, device=dev)
        isc = torch.empty(P, I // 128, dtype=torch.float32, device=dev)
        v.act_quant_fp8(inter, iq, isc)
        v.moe_gemm_fp8_block(iq, isc, None, w2d, s2d, st, y, H, I, E, False)
    else:
        v.moe_gemm_fp8_block(xd, None, tok, w13d, s13d, st, inter, 2 * I, H, E, True)
        v.moe_gemm_fp8_block(inter, None, None, w2d, s2d, st, y, H, I, E, False)
    out = torch.empty(T, H, dtype=dt, device=dev)
    v.moe_combine(y, inv, tw, out, K)
    return dict(tw=tw, ti=ti, inter=inter, iq=iq, isc=isc, y=y, out=out)


def _check_forward(v, dev, T, E, K, H, I, aq, seed, free_bar=None):
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, K, H, I, seed=seed)
    g = _staged_forward(v, dev, x, logits, w13q, w13s, w2q, w2s, E, K, aq)
    rtw, rti = O.moe_topk(logits, K)
    assert torch.equal(g["ti"].cpu(), rti)
    # oracle forward that starts the down GEMM from the kernel's own quantised intermediate
    iq_override = (g["iq"].cpu(), g["isc"].cpu()) if aq else None
    ref, ref_inter, ref_y = O.moe_forward_grouped(x, g["tw"].cpu(), rti, w13q, w13s, w2q, w2s, E, act_quant=aq,
                                                  inter_q=iq_override, return_parts=True)
    if aq:
        # stage 1: gate_up GEMM + SiLU*mul from the same quantised x
        assert O.max_rel_err(g["inter"].cpu(), ref_inter.float()) < TOL
        # stage 2: the kernel's quantisation of its own intermediate is bit-exact
        rq, rs = O.act_quant_per_token_group(g["inter"].cpu())
        assert torch.equal(g["iq"].cpu(), rq) and torch.equal(g["isc"].cpu(), rs)
    # stage 3: down GEMM, stage 4: weighted combine
    assert O.max_rel_err(g["y"].cpu(), ref_y) < TOL
    assert O.max_rel_err(g["out"].cpu(), ref) < TOL
    # the reference's 1e-3-floor form on the same teacher-forced output (near-zero outputs are judged on
    # the absolute error of an 8-expert weighted sum rounded to 16 bit)
    assert O.max_rel_err_abs_floor(g["out"].cpu(), ref) < 3e-2
    # the fused op runs the same kernels; with fused SiLU (act-quant mode) it is bit-identical
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    r = v.moe_forward_fp8_block(x.to(dev), logits.to(dev), w13q.view(torch.float8_e4m3fn).to(dev), w13s.to(dev),
                                w2q.view(torch.float8_e4m3fn).to(dev), w2s.to(dev), out, K, aq)
    assert r.data_ptr() == out.data_ptr()
    assert torch.equal(out, g["out"])
    # free-running oracle (quantises its own intermediate): the reference's looser, mean-based bar
    free = O.moe_forward_grouped(x, rtw, rti, w13q, w13s, w2q, w2s, E, act_quant=aq)
    o = out.cpu().float()
    mean_rel = ((o - free).abs().mean() / free.abs().mean()).item()
    cos = torch.nn.functional.cosine_similarity(o.flatten(), free.flatten(), dim=0).item()
    assert mean_rel < 1e-2 and cos > 0.9995, (mean_rel, cos)
    # recorded, not asserted (re-quantising the intermediate is discontinuous): the free-running
    # maximum under both denominators, and the staged (teacher-forced) output under the reference's floor
    print(f"moe forward T={T} E={E} aq={aq}: staged out max-rel (mean floor) {O.max_rel_err(g['out'].cpu(), ref):.3e}, "
          f"(1e-3 floor) {O.max_rel_err_abs_floor(g['out'].cpu(), ref):.3e}; free-running max-rel (mean floor) "
          f"{O.max_rel_err(out.cpu(), free):.3e}, (1e-3 floor) {O.max_rel_err_abs_floor(out.cpu(), free):.3e}, "
          f"mean-rel {mean_rel:.3e}, cos {cos:.6f}", flush=True)
    if free_bar is not None:
        # the free-running maximum is discontinuous in the intermediate's quantisation grid, so it cannot
        # meet the staged bar; it is held to twice the recorded figure instead, which still fails on a
        # regression of the forward as a whole
        assert O.max_rel_err(out.cpu(), free) < free_bar
    return out


@pytest.mark.parametrize("T,E,K,H,I,aq", [(5, 8, 2, 256, 128, True), (5, 8, 2, 256, 128, False),
                                          (12, 16, 4, 256, 128, True), (40, 16, 4, 512, 256, True),
                                          (12, 16, 4, 256, 128, False), (1, 16, 4, 256, 128, True)])
def test_moe_forward_small(v, dev, T, E, K, H, I, aq):
    _check_forward(v, dev, T, E, K, H, I, aq, seed=T + E)


@pytest.mark.parametrize("T,E,K,H,I,dt", [(800, 8, 2, 256, 128, torch.bfloat16), (1100, 4, 2, 384, 256, torch.float16)])
def test_moe_forward_w8a16_prefill(v, dev, T, E, K, H, I, dt):
    """16-bit activations with >= 96 rows per expert on average: both grouped GEMMs take the tiled
    matrix-core route and the expert outputs are kept in the activation type before the combine."""
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, K, H, I, seed=T, act_dtype=dt)
    out = torch.empty(T, H, dtype=dt, device=dev)
    v.moe_forward_fp8_block(x.to(dev), logits.to(dev), w13q.view(torch.float8_e4m3fn).to(dev), w13s.to(dev),
                            w2q.view(torch.float8_e4m3fn).to(dev), w2s.to(dev), out, K, False)
    rtw, rti = O.moe_topk(logits, K)
    free = O.moe_forward_grouped(x, rtw, rti, w13q, w13s, w2q, w2s, E, act_quant=False, act_dtype=dt)
    o = out.cpu().float()
    mean_rel = ((o - free).abs().mean() / free.abs().mean()).item()
    cos = torch.nn.functional.cosine_similarity(o.flatten(), free.flatten(), dim=0).item()
    assert mean_rel < (3e-3 if dt == torch.float16 else 1e-2) and cos > 0.9999, (mean_rel, cos)
    # element-wise, against the same arithmetic: block scales folded into weights of the activation type (as the
    # tiled kernel feeds the matrix core), plus one rounding of each expert output to that type (the reference's
    # grouped GEMM writes it too), which cancellation between a token's experts can make visible
    ref, _, y = O.moe_forward_grouped(x, rtw, rti, w13q, w13s, w2q, w2s, E, act_quant=False, act_dtype=dt,
                                      return_parts=True, weight_dtype=dt)
    order, _, _ = O.moe_sort(rti, E)
    mag = torch.zeros(T, H).index_add_(0, (order // K).long(), y.abs() * rtw.reshape(-1).float()[order.long()][:, None])
    ulp = 2.0 ** -8 if dt == torch.bfloat16 else 2.0 ** -11
    bound = TOL * ref.abs().clamp(min=ref.abs().mean()) + ulp * mag
    assert bool(((o - ref).abs() <= bound).all()), ((o - ref).abs() / bound).max()


def test_moe_prefill_full_size_properties(v, dev):
    """The w8a16 forward at the prefill benchmark's size (4096 tokens, 128 experts, top 8, H = 2048, I = 768,
    bf16: 256 +- 16 rows per expert, so full tiles and a few-row tail tile per expert), checked through what
    does not depend on the size: (1) a permutation of the tokens permutes the output rows bit for bit (a row's
    arithmetic does not depend on which tile, wavefront or lane it lands in); (2) sampled tokens against the
    oracle's per-token forward with the weights of their experts."""
    T, E, K, H, I = 4096, 128, 8, 2048, 768
    dt = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(77)
    # finite E4M3 codes drawn directly (a CPU quantisation of 600 M weights takes minutes): |code| <= 0x6F
    codes = lambda *s: (torch.randint(0, 0x70, s, generator=g, device=dev, dtype=torch.uint8) |
                        (torch.randint(0, 2, s, generator=g, device=dev, dtype=torch.uint8) << 7))
    w13, w2 = codes(E, 2 * I, H), codes(E, H, I)
    s13 = torch.rand(E, 2 * I // 128, H // 128, generator=g, device=dev) * 2e-3 + 5e-4
    s2 = torch.rand(E, H // 128, I // 128, generator=g, device=dev) * 2e-3 + 5e-4
    x = (torch.randn(T, H, generator=g, device=dev) * 0.5).to(dt)
    logits = torch.randn(T, E, generator=g, device=dev).to(dt)
    f8 = lambda t: t.view(torch.float8_e4m3fn)
    out = torch.empty(T, H, dtype=dt, device=dev)
    v.moe_forward_fp8_block(x, logits, f8(w13), s13, f8(w2), s2, out, K, False)
    assert torch.isfinite(out.float()).all()
    perm = torch.randperm(T, generator=g, device=dev)
    out_p = torch.empty_like(out)
    v.moe_forward_fp8_block(x[perm].contiguous(), logits[perm].contiguous(), f8(w13), s13, f8(w2), s2, out_p, K, False)
    assert torch.equal(out_p.view(torch.int16), out[perm].view(torch.int16))
    # sampled tokens: block scales folded into weights of the activation type (the tiled kernel's arithmetic),
    # the intermediate and every expert output rounded to it, fp32 sum of the routes
    xc, lc = x.cpu(), logits.cpu()
    rtw, rti = O.moe_topk(lc, K)
    for t in (0, 1733, T - 1):
        want = torch.zeros(H)
        mag = torch.zeros(H)
        for jr in range(K):
            e = int(rti[t, jr])
            d13 = O.fp8_dequant_block(w13[e].cpu(), s13[e].cpu(), out_dtype=dt)
            d2 = O.fp8_dequant_block(w2[e].cpu(), s2[e].cpu(), out_dtype=dt)
            h = O.silu_mul((xc[t].float() @ d13.t())[None, :]).to(dt).float()
            y = (h @ d2.t())[0].to(dt).float()
            want += rtw[t, jr].float() * y
            mag += rtw[t, jr].float() * y.abs()
        got = out[t].cpu().float()
        bound = TOL * want.abs().clamp(min=want.abs().mean()) + 2.0 ** -8 * mag
        assert bool(((got - want).abs() <= bound).all()), (t, ((got - want).abs() / bound).max())


@pytest.mark.parametrize("T", [512, 37])
def test_cfg3_forward_token_permutation(v, dev, T):
    """cfg3's forward (fp8 activations; the gate_up launch sorts the pairs itself): permuting the tokens
    permutes the output rows bit for bit, at the benchmark's size and at a ragged one."""
    E, K, H, I = 128, 8, 2048, 768
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, K, H, I, seed=4242)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    args = (f8(w13q), w13s.to(dev), f8(w2q), w2s.to(dev))
    xd, ld = x.to(dev), logits.to(dev)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    v.moe_forward_fp8_block(xd, ld, *args, out, K, True)
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(T)).to(dev)
    out_p = torch.empty_like(out)
    v.moe_forward_fp8_block(xd[perm].contiguous(), ld[perm].contiguous(), *args, out_p, K, True)
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out_p.view(torch.int16), out[perm].view(torch.int16))


@pytest.mark.parametrize("counts,H,I,dt,per_expert,act", [
    ([300, 0, 17, 256, 0, 0, 513, 1], 256, 128, torch.bfloat16, 0, 1),       # empty experts, one row, tile edges
    ([120, 200, 90, 310], 384, 256, torch.float16, 0, 2),                      # tanh-GELU
    ([260, 250], 256, 384, torch.bfloat16, 2, 1),                              # gate / up scalars, one for down
    ([100] * 40, 128, 128, torch.float16, 1, 1)])
def test_moe_mlp_tiled_equals_two_grouped_gemms(v, dev, counts, H, I, dt, per_expert, act):
    """The expert MLP as one library call (tile table built once, the intermediate written straight into the
    second GEMM's operand order) against two calls of the tiled grouped GEMM with a row-major intermediate:
    the same bits, with a row map on the input and a row map + row weights on the output; and the
    two-call result against the oracle."""
    import ctypes
    from mi355x_qlinear import capi
    E = len(counts)
    total = sum(counts)
    g = torch.Generator().manual_seed(total + H)
    start = torch.zeros(E + 1, dtype=torch.int32)
    start[1:] = torch.tensor(counts).cumsum(0).to(torch.int32)
    T = total // 2 + 3
    x = (torch.randn(T, H, generator=g) * 0.3).to(dt)
    row_map = torch.randint(0, T, (total,), generator=g, dtype=torch.int32)
    out_map = torch.randperm(total, generator=g).to(torch.int32)
    row_w = (torch.rand(total, generator=g) + 0.5).to(dt)
    if per_expert:
        w13 = (torch.randn(E, 2 * I, H, generator=g) * 20).to(torch.float8_e4m3fn)
        w2 = (torch.randn(E, H, I, generator=g) * 20).to(torch.float8_e4m3fn)
        s13 = torch.rand(E, per_expert, generator=g) * 0.004 + 0.002
        s2 = torch.rand(E, generator=g) * 0.004 + 0.002
        w13b, w2b = w13.view(torch.uint8), w2.view(torch.uint8)
    else:
        w13b, s13 = O.fp8_quantize_block(torch.randn(E, 2 * I, H, generator=g) * 0.15)
        w2b, s2 = O.fp8_quantize_block(torch.randn(E, H, I, generator=g) * 0.15)
    xd, rmd, omd, rwd, std = x.to(dev), row_map.to(dev), out_map.to(dev), row_w.to(dev), start.to(dev)
    w13d, s13d, w2d, s2d = w13b.to(dev), s13.to(dev), w2b.to(dev), s2.to(dev)
    adt = capi.act_dtype(xd)

    def ws_of(fn, *dims):
        need = ctypes.c_longlong(0)
        assert getattr(capi.lib(), fn)(*dims, ctypes.byref(need)) == 0
        return torch.empty(need.value, dtype=torch.uint8, device=dev), need.value

    inter = torch.empty(total, I, dtype=dt, device=dev)
    two = torch.full((total, H), 3.0, dtype=dt, device=dev)
    b1, n1 = ws_of("mi_moe_gemm_fp8_tiled_workspace", total, E, H)
    capi.call("mi_moe_gemm_fp8_tiled_ws", xd, capi.ptr(xd), capi.ptr(rmd), 1, capi.ptr(w13d), capi.ptr(s13d), per_expert,
              capi.ptr(std), capi.ptr(inter), None, None, T, total, E, 2 * I, H, act, adt, capi.ptr(b1), n1)
    b2, n2 = ws_of("mi_moe_gemm_fp8_tiled_workspace", total, E, I)
    capi.call("mi_moe_gemm_fp8_tiled_ws", xd, capi.ptr(inter), None, 1, capi.ptr(w2d), capi.ptr(s2d), min(per_expert, 1),
              capi.ptr(std), capi.ptr(two), capi.ptr(omd), capi.ptr(rwd), total, total, E, H, I, 0, adt, capi.ptr(b2), n2)
    one = torch.full((total, H), 5.0, dtype=dt, device=dev)
    b3, n3 = ws_of("mi_moe_mlp_fp8_tiled_workspace", total, E, H, I)
    capi.call("mi_moe_mlp_fp8_tiled_ws", xd, capi.ptr(xd), capi.ptr(rmd), 1, capi.ptr(w13d), capi.ptr(s13d), capi.ptr(w2d),
              capi.ptr(s2d), per_expert, capi.ptr(std), capi.ptr(one), capi.ptr(omd), capi.ptr(rwd), T, total, E, H, I, act,
              adt, capi.ptr(b3), n3)
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    # the two-call result against the oracle: per expert, weights with their scales folded in and rounded to
    # the activation type where the scales are blocks (as the tiled kernel feeds the matrix core)
    want = torch.zeros(total, H)
    for e in range(E):
        lo, hi = int(start[e]), int(start[e + 1])
        if hi == lo:
            continue
        if per_expert:
            d13 = w13[e].float()
            d13 = torch.cat([d13[:I] * s13[e, 0], d13[I:] * s13[e, per_expert - 1]])
            d2 = w2[e].float() * s2[e]
        else:
            d13 = O.fp8_dequant_block(w13b[e], s13[e], out_dtype=dt).float()
            d2 = O.fp8_dequant_block(w2b[e], s2[e], out_dtype=dt).float()
        gu = x[row_map[lo:hi].long()].float() @ d13.t()
        h = (O.gelu_tanh_mul(gu) if act == 2 else O.silu_mul(gu)).to(dt).float()
        want[out_map[lo:hi].long()] = ((h @ d2.t()) * row_w[out_map[lo:hi].long()].float()[:, None])
    assert O.max_rel_err(two.cpu(), want) < TOL


@pytest.mark.parametrize("aq", [True, False])
def test_expert_outputs_in_fp16_beside_bf16(v, dev, aq):
    """The grouped GEMM can write fp16 whatever the activation type and the combine reads it: half the bytes
    of fp32 rows at 11 significant bits.  The fused forward keeps fp32 (near-zero outputs, sums of cancelling
    terms, are 6 x closer to the oracle with it); this covers the mode for callers that trade that for speed."""
    T, E, K, H, I = 24, 8, 2, 256, 128
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, K, H, I, seed=77)
    assert x.dtype == torch.bfloat16
    g = _staged_forward(v, dev, x, logits, w13q, w13s, w2q, w2s, E, K, aq)
    P = T * K
    st = torch.empty(E + 1, dtype=torch.int32, device=dev)
    sp, inv, tok = (torch.empty(P, dtype=torch.int32, device=dev) for _ in range(3))
    v.moe_sort(g["ti"], E, sp, st, inv, tok)
    y16 = torch.empty(P, H, dtype=torch.float16, device=dev)
    if aq:
        v.moe_gemm_fp8_block(g["iq"], g["isc"], None, w2q.to(dev), w2s.to(dev), st, y16, H, I, E, False)
    else:
        v.moe_gemm_fp8_block(g["inter"], None, None, w2q.to(dev), w2s.to(dev), st, y16, H, I, E, False)
    assert torch.equal(y16, g["y"].half())                     # the fp32 result, rounded once
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    v.moe_combine(y16, inv, g["tw"], out, K)
    ref = (g["tw"].float().reshape(T, K, 1) * y16.float()[inv.long()].reshape(T, K, H)).sum(1)
    assert O.max_rel_err(out.cpu(), ref.cpu()) < 4e-3          # one bf16 rounding of the fp32 sum
    assert O.max_rel_err(out.cpu(), g["out"].float().cpu()) < TOL


def test_cfg3_moe_forward(v, dev):
    # the stage-wise 1e-2 bars (mean floor) are inside _check_forward; it also prints the staged and the
    # free-running maxima under both denominators (free-running, this shape: 4e-2 with the mean floor)
    # and asserts the free-running maximum at twice the recorded 4.1e-2
    out = _check_forward(v, dev, 512, 128, 8, 2048, 768, True, seed=1237, free_bar=8e-2)
    assert torch.isfinite(out.float()).all()


# ----------------------------------------------------------------- fused decode op with shared expert
def _full_case(T, seed, dtype, experts=16, hidden=256, inter=128):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, hidden, generator=g) * 0.2).to(dtype)
    logits = (torch.randn(T, experts, generator=g) * 0.4).to(dtype)
    w13, s13 = O.fp8_quantize_block(torch.randn(experts, 2 * inter, hidden, generator=g) * 0.15)
    w2, s2 = O.fp8_quantize_block(torch.randn(experts, hidden, inter, generator=g) * 0.15)
    sw13, ss13 = O.fp8_quantize_block(torch.randn(2 * inter, hidden, generator=g) * 0.15)
    sw2, ss2 = O.fp8_quantize_block(torch.randn(hidden, inter, generator=g) * 0.15)
    gate = (torch.randn(1, hidden, generator=g) * 0.1).to(dtype)
    return x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate


@pytest.mark.parametrize("T", [1, 2, 3, 4, 8, 10, 12, 20, 24, 25, 40])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_moe_forward_full_fp8_block(v, dev, T, dtype):
    # V/tests/test_moe_forward_full_fp8_block.py:83-150 (same sizes, same bars); T = 20 .. 40 are beyond
    # the reference's 12-token limit: up to 96 (token, route) pairs (T = 24 here) run one GEMV per route,
    # more (T = 25, 40) the grouped GEMMs
    top_k = 4
    x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate = _full_case(T, 100 + T, dtype)
    expected = O.moe_forward_full(x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate, top_k)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    out = torch.empty(T, x.shape[1], dtype=dtype, device=dev)
    r = torch.ops.moe_ops.moe_forward_full_fp8_block(
        x.to(dev), logits.to(dev), out, f8(w13), s13.to(dev), f8(sw13), ss13.to(dev), f8(w2), s2.to(dev),
        f8(sw2), ss2.to(dev), gate.to(dev), top_k, 1, 16)
    assert r.data_ptr() == out.data_ptr()
    actual = out.cpu().float()
    mean_rel = ((actual - expected).abs().mean() / expected.abs().mean()).item()
    cos = torch.nn.functional.cosine_similarity(actual.flatten(), expected.flatten(), dim=0).item()
    bar = 3e-3 if dtype == torch.float16 else 1e-2     # the reference's bar is for fp16
    assert mean_rel < bar and cos > (0.9999 if dtype == torch.float16 else 0.999)


@pytest.mark.parametrize("routes,E,N,K,dt,weighted", [(8, 16, 1536, 2048, torch.bfloat16, False),
                                                      (12, 8, 384, 256, torch.float16, True),
                                                      (1, 4, 128, 1152, torch.float16, True)])
def test_routed_fp8_block_gemv(dev, routes, E, N, K, dt, weighted):
    """One block-scaled FP8 GEMV per (token, expert) route in one launch: each route's row against
    the oracle's dequantised expert matrix (1e-2 with the mean floor), ids outside the range held
    into it, the optional routing weight applied before the rounding."""
    from mi355x_qlinear import capi
    g = torch.Generator().manual_seed(routes * 31 + N)
    k = 2 if routes % 2 == 0 else 1
    T = routes // k
    x = (torch.randn(T, K, generator=g) * 0.5).to(dt)
    w, ws = O.fp8_quantize_block(torch.randn(E, N, K, generator=g) * 0.1)
    ids = torch.randint(0, E, (routes,), generator=g).to(torch.int32)
    ids[0] = E + 3                                          # held into the range: expert E - 1
    rw = (torch.rand(routes, generator=g) + 0.25).to(dt) if weighted else None
    xd, wd, wsd, idd = x.to(dev), w.to(dev), ws.to(dev), ids.to(dev)
    rwd = rw.to(dev) if weighted else None
    out = torch.full((routes, N + 8), 7.0, dtype=dt, device=dev)       # rows 8 elements apart from dense
    capi.call("mi_moe_gemv_fp8_block_routed", xd, capi.ptr(xd), k, 0, capi.ptr(wd), capi.ptr(wsd), capi.ptr(out), N + 8,
              capi.ptr(idd), capi.ptr(rwd), routes, E, None, None, 0, 0, N, K, capi.act_dtype(xd))
    dw = O.fp8_dequant_block(w, ws)
    for r in range(routes):
        e = min(max(int(ids[r]), 0), E - 1)
        ref = x[r // k].float() @ dw[e].t()
        if weighted:
            ref = ref * rw[r].float()
        assert O.max_rel_err(out[r, :N].cpu(), ref) < TOL, (r, e)
    assert bool((out[:, N:] == 7.0).all())
    # rows of a shared matrix in the same launch, and SiLU(gate) * up fused into the staging of x:
    # x2 rows are [gate | up], 2 K wide; shared row i reads x2 row 1 + i
    sw, sws = O.fp8_quantize_block(torch.randn(N, K, generator=g) * 0.1)
    x2 = (torch.randn(routes + 3, 2 * K, generator=g) * 0.7).to(dt)
    act = O.silu_mul(x2).to(dt)
    x2d, swd, swsd = x2.to(dev), sw.to(dev), sws.to(dev)
    out2 = torch.full((routes + 2, N), 7.0, dtype=dt, device=dev)
    capi.call("mi_moe_gemv_fp8_block_routed", x2d, capi.ptr(x2d), 1, 1, capi.ptr(wd), capi.ptr(wsd), capi.ptr(out2), N,
              capi.ptr(idd), capi.ptr(rwd), routes, E, capi.ptr(swd), capi.ptr(swsd), 2, 1, N, K, capi.act_dtype(xd))
    dsw = O.fp8_dequant_block(sw, sws)
    for r in range(routes):
        e = min(max(int(ids[r]), 0), E - 1)
        ref = act[r].float() @ dw[e].t()
        if weighted:
            ref = ref * rw[r].float()
        assert O.max_rel_err(out2[r].cpu(), ref) < TOL, (r, e)
    for i in range(2):
        assert O.max_rel_err(out2[routes + i].cpu(), act[1 + i].float() @ dsw.t()) < TOL, i


def test_moe_forward_full_fp8_block_errors(v, dev):
    top_k = 4
    x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate = _full_case(4, 7, torch.float16)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    xd = x.to(dev)
    args = [xd, logits.to(dev), torch.empty_like(xd), f8(w13), s13.to(dev), f8(sw13), ss13.to(dev), f8(w2),
            s2.to(dev), f8(sw2), ss2.to(dev), gate.to(dev), top_k, 1, 16]
    op = torch.ops.moe_ops.moe_forward_full_fp8_block
    bad = list(args); bad[2] = xd                                  # output aliases x
    with pytest.raises(RuntimeError, match="alias"):
        op(*bad)
    bad = list(args); bad[13] = 2                                  # two shared experts
    with pytest.raises(RuntimeError, match="one shared expert"):
        op(*bad)
    bad = list(args); bad[12] = 17                                 # top_k > experts
    with pytest.raises(RuntimeError, match="top_k"):
        op(*bad)
    bad = list(args); bad[4] = s13.to(dev).double()                # scale dtype
    with pytest.raises(RuntimeError):
        op(*bad)


# ----------------------------------------------------------------- sglang prefill ops, per-expert scalar scales
def _prefill_case(T, E, H, I, k, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * 0.3).to(dtype)
    logits = torch.randn(T, E, generator=g).to(dtype)
    tw, ti = O.moe_topk(logits, k)
    w13f = torch.randn(E, 2 * I, H, generator=g) * 0.05
    w2f = torch.randn(E, H, I, generator=g) * 0.05
    s13 = torch.stack([w13f[:, :I].abs().amax((1, 2)), w13f[:, I:].abs().amax((1, 2))], 1) / 448.0
    s2 = w2f.abs().amax((1, 2)) / 448.0
    w13 = torch.cat([O.e4m3_quantize(w13f[:, :I] / s13[:, 0].view(E, 1, 1)), O.e4m3_quantize(w13f[:, I:] / s13[:, 1].view(E, 1, 1))], 1)
    w2 = O.e4m3_quantize(w2f / s2.view(E, 1, 1))
    return x, tw, ti, w13, s13.float().contiguous(), w2, s2.float().contiguous()


@pytest.mark.parametrize("T,E,H,I,k,dtype", [(64, 8, 256, 128, 2, torch.float16), (200, 16, 512, 256, 4, torch.bfloat16),
                                             (1, 4, 128, 128, 1, torch.float16),
                                             # sizes that are multiples of 16 / 32 only, as the reference accepts
                                             (50, 8, 144, 80, 2, torch.float16), (33, 4, 2816 // 8, 704 // 4, 2, torch.float16),
                                             # hundreds of rows per expert: both GEMMs on the tiled matrix-core route
                                             (700, 4, 256, 128, 2, torch.float16)])
def test_moe_prefill_full_fp8(s, dev, T, E, H, I, k, dtype):
    x, tw, ti, w13, s13, w2, s2 = _prefill_case(T, E, H, I, k, 300 + T, dtype)
    want, inter_ref, y_ref = O.moe_prefill_scalar(x, tw, ti, w13, s13, w2, s2, return_parts=True)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    op = torch.ops.moe_fp8_prefill_ops
    got = op.moe_prefill_full_fp8(x.to(dev), tw.to(dev), ti.to(dev), f8(w13), s13.to(dev), f8(w2), s2.to(dev), k, E)
    assert got.shape == (T, H) and got.dtype == dtype
    # the intermediate is a 16-bit tensor by the op's contract (w8a16): the reference value of the
    # output is the down projection of the oracle's intermediate rounded to that dtype
    ids = ti.reshape(-1).long()
    d2 = O.e4m3_decode(w2.reshape(-1, I)).reshape(E, H, I)
    y_r = torch.einsum("pi,phi->ph", inter_ref.to(dtype).float(), d2[ids]) * s2[ids].view(-1, 1)
    want_r = (tw.float().reshape(T, k, 1) * y_r.reshape(T, k, H)).sum(1)
    assert O.max_rel_err(got.cpu().float(), want_r) < TOL
    mean_rel = ((got.cpu().float() - want).abs().mean() / want.abs().mean()).item()
    assert mean_rel < 5e-3                                      # against the all-fp32 oracle
    # the staged ops, each against the oracle's pair-ordered intermediates (teacher forcing:
    # the down op is fed the up op's own rounded output)
    offs, toks, perm, rows = op.moe_prefill_gather_forward_fp8(ti.to(dev), E)
    inter = op.moe_prefill_up_forward_fp8(x.to(dev), f8(w13), s13.to(dev), offs, toks, k)
    assert inter.shape == (T * k, I)
    assert O.max_rel_err(inter.cpu().float(), inter_ref) < TOL
    y = op.moe_prefill_down_forward_fp8(inter, f8(w2), s2.to(dev), offs, toks)
    y_forced = torch.einsum("pi,phi->ph", inter.cpu().float(), d2[ids]) * s2[ids].view(-1, 1)
    assert O.max_rel_err(y.cpu().float(), y_forced) < TOL
    acc = op.moe_prefill_accumulate_forward_fp8(y, tw.to(dev))
    acc_ref = (tw.float().reshape(T, k, 1) * y.cpu().float().reshape(T, k, H)).sum(1)
    assert O.max_rel_err(acc.cpu().float(), acc_ref) < TOL
    assert O.max_rel_err(acc.cpu().float(), want) < 3 * TOL     # free-running chain: three 16-bit roundings


def test_permute_rows_roundtrip(v, dev):
    from mi355x_qlinear import capi
    g = torch.Generator().manual_seed(9)
    rows, cols = 777, 264
    src = torch.randn(rows, cols, generator=g).half().to(dev)
    perm = torch.randperm(rows, generator=g).to(torch.int32).to(dev)
    a = torch.empty_like(src)
    b = torch.empty_like(src)
    capi.call("mi_permute_rows", src, capi.ptr(src), capi.ptr(perm), capi.ptr(a), rows, cols * 2, 0)
    assert torch.equal(a.cpu(), src.cpu()[perm.cpu().long()])
    capi.call("mi_permute_rows", a, capi.ptr(a), capi.ptr(perm), capi.ptr(b), rows, cols * 2, 1)
    assert torch.equal(b.cpu(), src.cpu())


# ----------------------------------------------------------------- per-expert-scale ops with the tanh-GELU gate (moe_ops)
def _pert_case(T, E, H, I, k, seed, dtype):
    """Weights as V/tests/test_moe_full_gelu_tanh.py:39-44 draws them (clamped normal / 0.3 -> e4m3, with
    per-expert scales varied here so that a wrong scale index shows)."""
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * 0.05).to(dtype)
    logits = torch.randn(T, E, generator=g).to(dtype)
    tw, ti = O.moe_topk(logits, k)
    w13 = O.e4m3_quantize((torch.randn(E, 2 * I, H, generator=g) * 0.05).clamp(-0.3, 0.3) / 0.3)
    w2 = O.e4m3_quantize((torch.randn(E, H, I, generator=g) * 0.05).clamp(-0.3, 0.3) / 0.3)
    s13 = (0.3 * (0.5 + torch.rand(E, generator=g))).float()
    s2 = (0.3 * (0.5 + torch.rand(E, generator=g))).float()
    return x, logits, tw.to(dtype), ti, w13, s13, w2, s2


@pytest.mark.parametrize("T,E,H,I,k,dtype", [(1, 16, 2048, 768, 8, torch.float16), (8, 8, 512, 256, 2, torch.float16),
                                             (3, 4, 384, 80, 2, torch.bfloat16), (40, 8, 256, 144, 2, torch.float16)])
def test_moe_silu_routed(v, dev, T, E, H, I, k, dtype):
    """moe_forward_full_silu_routed_sglang (N-major w13) and moe_forward_full_silu_routed (w13 transposed to
    [E, H, 2I]) against the per-route loop with the intermediate rounded to the activation dtype."""
    x, logits, tw, ti, w13, s13, w2, s2 = _pert_case(T, E, H, I, k, 900 + T, dtype)
    want, inter_ref, y_ref = O.moe_prefill_scalar(x, tw, ti, w13, s13, w2, s2, return_parts=True, act="silu")
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    d = lambda t: t.to(dev)
    ids = ti.reshape(-1).long()
    d2 = O.e4m3_decode(w2.reshape(-1, I)).reshape(E, H, I)
    y_r = torch.einsum("pi,phi->ph", inter_ref.to(dtype).float(), d2[ids]) * s2[ids].view(-1, 1)
    want_r = (tw.float().reshape(T, k, 1) * y_r.reshape(T, k, H)).sum(1)
    import custom_esimd_kernels_sglang.moe_ops as sg_moe
    got = sg_moe.moe_forward_full_silu_routed_sglang(d(x), d(tw), d(ti), f8(w13), d(s13), f8(w2), d(s2), k, E)
    assert got.shape == (T, H) and got.dtype == dtype
    assert O.max_rel_err(got.cpu().float(), want_r) < TOL
    assert ((got.cpu().float() - want).abs().mean() / want.abs().mean()).item() < 5e-3
    w13_km = w13.transpose(1, 2).contiguous()          # [E, H, 2I]
    got2 = sg_moe.moe_forward_full_silu_routed(d(x), d(tw), d(ti), f8(w13_km), d(s13), f8(w2), d(s2), k, E)
    assert got2.shape == (T, H) and got2.dtype == dtype
    assert O.max_rel_err(got2.cpu().float(), want_r) < TOL
    if 2 * I != H:
      with pytest.raises(RuntimeError):                # N-major w13 handed to the K-major op
        sg_moe.moe_forward_full_silu_routed(d(x), d(tw), d(ti), f8(w13), d(s13), f8(w2), d(s2), k, E)


@pytest.mark.parametrize("T,E,H,I,k,dtype", [(2, 16, 2816, 704, 8, torch.float16), (40, 8, 256, 144, 2, torch.float16),
                                             (1, 16, 512, 256, 4, torch.float16), (70, 4, 384, 80, 2, torch.bfloat16)])
def test_moe_gelu_tanh_family(v, dev, T, E, H, I, k, dtype):
    """K = 704, 144, 80 end in a partial 128-granule; I = 704, 144, 80 put the gate / up boundary inside a
    128-row block."""
    x, logits, tw, ti, w13, s13, w2, s2 = _pert_case(T, E, H, I, k, 500 + T, dtype)
    want, inter_ref, y_ref = O.moe_prefill_scalar(x, tw, ti, w13, s13, w2, s2, return_parts=True, act="gelu_tanh")
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    op = torch.ops.moe_ops
    d = lambda t: t.to(dev)
    # down projection of the rounded intermediate: the value a w8a16 chain should produce
    ids = ti.reshape(-1).long()
    d2 = O.e4m3_decode(w2.reshape(-1, I)).reshape(E, H, I)
    y_r = torch.einsum("pi,phi->ph", inter_ref.to(dtype).float(), d2[ids]) * s2[ids].view(-1, 1)
    want_r = (tw.float().reshape(T, k, 1) * y_r.reshape(T, k, H)).sum(1)

    got = op.moe_forward_full_gelu_tanh_routed(d(x), d(tw), d(ti), f8(w13), d(s13), f8(w2), d(s2), k, E)
    assert got.shape == (T, H) and got.dtype == dtype
    assert O.max_rel_err(got.cpu().float(), want_r) < TOL
    assert ((got.cpu().float() - want).abs().mean() / want.abs().mean()).item() < 5e-3
    # internal softmax top-k
    got2 = op.moe_forward_full_gelu_tanh(d(x), d(logits), f8(w13), d(s13), f8(w2), d(s2), k, E)
    assert O.max_rel_err(got2.cpu().float(), want_r) < TOL
    # per-route rows, weighted, in pair order
    rows = op.moe_forward_full_gelu_tanh_routed_no_accum(d(x), d(tw), d(ti), f8(w13), d(s13), f8(w2), d(s2), k, E)
    assert rows.shape == (T * k, H)
    assert O.max_rel_err(rows.cpu().float(), y_r * tw.float().reshape(-1, 1)) < TOL
    if T == 1:
        got3 = op.moe_forward_full_gelu_tanh_routed_decode(d(x), d(tw), d(ti), f8(w13), d(s13), f8(w2), d(s2), k, E)
        assert torch.equal(got3.cpu(), got.cpu())
        pes = (0.5 + torch.rand(E, generator=torch.Generator().manual_seed(3))).float()
        got4 = op.moe_forward_full_gelu_tanh_decode(d(x), d(logits), f8(w13), d(s13), f8(w2), d(s2), d(pes), k, E)
        tw_f = (tw.float() * pes[ti.long()]).to(dtype)
        want4 = (tw_f.float().reshape(T, k, 1) * y_r.reshape(T, k, H)).sum(1)
        assert O.max_rel_err(got4.cpu().float(), want4) < TOL
    # the grouped ops on the sglang gather's expert grouping
    offs, toks, _, _ = torch.ops.moe_fp8_prefill_ops.moe_prefill_gather_forward_fp8(d(ti), E)
    inter = op.moe_up_fp8_grouped(d(x), f8(w13), d(s13), offs, toks, k, E)
    assert inter.shape == (T * k, I)
    assert O.max_rel_err(inter.cpu().float(), inter_ref) < TOL
    rw = d(tw.reshape(-1).contiguous())
    part = op.moe_down_fp8_grouped(inter, f8(w2), d(s2), rw, offs, toks, k, E)
    forced = torch.einsum("pi,phi->ph", inter.cpu().float(), d2[ids]) * s2[ids].view(-1, 1) * tw.float().reshape(-1, 1)
    assert O.max_rel_err(part.cpu().float(), forced) < TOL
    full = op.moe_forward_full_fp8_grouped(d(x), f8(w13), d(s13), f8(w2), d(s2), rw, offs, toks, k, E)
    assert O.max_rel_err(full.cpu().float(), want_r) < TOL


def test_moe_fp8_grouped_vllm_call_chain(v, dev):
    """The call sequence of the patched vLLM's grouped FP8 MoE forward
    (vllm/patches/vllm_for_multi_arc.patch:8216-8246): module import, softmax top-k, gather v2 of the
    moe_int4_prefill_ops namespace, grouped up / down on uint8 views, sum over the routes."""
    import custom_esimd_kernels_vllm.moe_int4_prefill_ops  # noqa: F401  (registers the gather)
    T, E, H, I, k = 20, 16, 512, 256, 4
    x, logits, tw, ti, w13, s13, w2, s2 = _pert_case(T, E, H, I, k, 77, torch.float16)
    d = lambda t: t.to(dev)
    weights, indices = torch.ops.moe_int4_prefill_ops.moe_topk_softmax(d(logits), k, E)
    assert torch.equal(indices.cpu(), ti)
    go = torch.ops.moe_int4_prefill_ops.moe_prefill_gather_forward_v2(indices.contiguous(), E)
    expert_offsets, expert_tokens = go[0], go[1]
    assert len(go) == 4 and expert_offsets.numel() == E and expert_tokens.numel() == T * k
    w13u, w2u = d(w13).view(torch.uint8), d(w2).view(torch.uint8)
    rw_flat = weights.reshape(-1).contiguous()
    inter = torch.ops.moe_ops.moe_up_fp8_grouped(d(x), w13u, d(s13), expert_offsets, expert_tokens, k, E)
    outp = torch.ops.moe_ops.moe_down_fp8_grouped(inter, w2u, d(s2), rw_flat, expert_offsets, expert_tokens, k, E)
    out = outp.view(T, k, -1).sum(1)
    want = O.moe_prefill_scalar(x, weights.cpu(), ti, w13, s13, w2, s2, act="gelu_tanh")
    assert ((out.cpu().float() - want).abs().mean() / want.abs().mean()).item() < 1e-2


def test_moe_fp8_grouped_reference_shape(v, dev):
    """E=128, top_k=8, H=2816, I=704, T=256 (V/tests/test_moe_fp8_grouped.py:16-37): the three routes through
    the kernels agree, and a sample of tokens matches the fp32 per-route loop."""
    T, E, H, I, k = 256, 128, 2816, 704, 8
    g = torch.Generator(device=dev).manual_seed(42)
    x = (torch.randn(T, H, generator=g, device=dev) * 0.05).half()
    logits = torch.randn(T, E, generator=g, device=dev).half()
    w13 = ((torch.randn(E, 2 * I, H, generator=g, device=dev) * 0.05).clamp(-0.3, 0.3) / 0.3).to(torch.float8_e4m3fn)
    w2 = ((torch.randn(E, H, I, generator=g, device=dev) * 0.05).clamp(-0.3, 0.3) / 0.3).to(torch.float8_e4m3fn)
    s13 = torch.full((E,), 0.3, device=dev)
    s2 = torch.full((E,), 0.3, device=dev)
    op = torch.ops.moe_ops
    tw, ti = op.moe_topk(logits, k, True)
    offs, toks, _, _ = torch.ops.moe_fp8_prefill_ops.moe_prefill_gather_forward_fp8(ti, E)
    rw = tw.reshape(-1).contiguous()
    inter = op.moe_up_fp8_grouped(x, w13, s13, offs, toks, k, E)
    part = op.moe_down_fp8_grouped(inter, w2, s2, rw, offs, toks, k, E)
    staged = part.view(T, k, H).float().sum(1)
    full = op.moe_forward_full_fp8_grouped(x, w13, s13, w2, s2, rw, offs, toks, k, E)
    routed = op.moe_forward_full_gelu_tanh_routed(x, tw, ti, w13, s13, w2, s2, k, E)
    assert O.max_rel_err(full.cpu().float(), staged.cpu()) < TOL
    assert O.max_rel_err(routed.cpu().float(), full.cpu().float()) < 2e-3
    sample = [0, 101, 255]
    tic = ti.cpu()
    used = sorted(set(tic[sample].reshape(-1).tolist()))
    remap = {e: i for i, e in enumerate(used)}
    ti_s = torch.tensor([[remap[int(e)] for e in tic[t]] for t in sample], dtype=torch.int32)
    w13_s = w13.view(torch.uint8)[used].cpu()
    w2_s = w2.view(torch.uint8)[used].cpu()
    want = O.moe_prefill_scalar(x.cpu()[sample], tw.cpu()[sample], ti_s, w13_s, torch.full((len(used),), 0.3), w2_s,
                                torch.full((len(used),), 0.3), act="gelu_tanh")
    assert O.max_rel_err(full.cpu().float()[sample], want) < 2 * TOL      # intermediate rounded to fp16 on the device


def test_moe_gemm_grouped_argument_errors(v, dev):
    from mi355x_qlinear import capi
    E, N, K, R = 2, 64, 72, 4          # K not a multiple of 16
    a = torch.zeros(R, K, dtype=torch.float16, device=dev)
    w = torch.zeros(E, N, K, dtype=torch.uint8, device=dev)
    sc = torch.ones(E, device=dev)
    start = torch.tensor([0, 2, 4], dtype=torch.int32, device=dev)
    out = torch.zeros(R, N, dtype=torch.float16, device=dev)
    args = lambda k, act, se=1, div=1: (capi.ptr(a), None, None, div, capi.ptr(w), capi.ptr(sc), se, capi.ptr(start),
                                        capi.ptr(out), None, None, R, R, E, N, k, act, capi.DT_F16, 0)
    with pytest.raises(RuntimeError):
        capi.call("mi_moe_gemm_fp8_grouped", a, *args(K, 0))
    with pytest.raises(RuntimeError):
        capi.call("mi_moe_gemm_fp8_grouped", a, *args(64, 3))
    with pytest.raises(RuntimeError):
        capi.call("mi_moe_gemm_fp8_grouped", a, *args(64, 0, 3))          # no such scale form
    # block scales with the fused epilogue: N/2 = 500 would put 16-row tiles of the up half across two scale blocks
    with pytest.raises(RuntimeError):
        v.moe_gemm_fp8_block(torch.zeros(4, 128, dtype=torch.float16, device=dev), None, None,
                             torch.zeros(2, 1000, 128, dtype=torch.uint8, device=dev),
                             torch.ones(2, 8, 1, device=dev), start, torch.zeros(4, 500, dtype=torch.float16, device=dev),
                             1000, 128, 2, True)
    with pytest.raises(RuntimeError):
        capi.call("mi_moe_gemm_fp8_grouped", a, *args(64, 0, 1, 0))       # row-map divisor below 1


# ----------------------------------------------------------------- per-tensor decode op on K-major routed weights
def _kmajor_case(T, E, H, I, k, seed, dtype, shared=True):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * 0.3).to(dtype)
    logits = torch.randn(T, E, generator=g).to(dtype)
    w13 = O.e4m3_quantize(torch.randn(E, H, 2 * I, generator=g))
    w2 = O.e4m3_quantize(torch.randn(E, I, H, generator=g))
    s13 = (0.004 * (1 + torch.rand(E, generator=g))).float()
    s2 = (0.004 * (1 + torch.rand(E, generator=g))).float()
    if not shared:
        return x, logits, w13, s13, None, None, w2, s2, None, None, None
    sw13 = O.e4m3_quantize(torch.randn(1, 2 * I, H, generator=g))
    sw2 = O.e4m3_quantize(torch.randn(1, H, I, generator=g))
    ss13, ss2 = torch.tensor([0.0051]), torch.tensor([0.0047])
    gate = (torch.randn(1, H, generator=g) * 0.05).to(dtype)
    return x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate


@pytest.mark.parametrize("T,E,H,I,k,dtype", [(1, 512, 2048, 512, 10, torch.float16), (1, 16, 256, 128, 4, torch.bfloat16),
                                             (3, 16, 1056, 288, 2, torch.float16), (9, 8, 2048, 768, 3, torch.float16)])
def test_moe_forward_full_kmajor(v, dev, T, E, H, I, k, dtype):
    """Qwen3-Next decode sizes (512 experts, top 10, H 2048, I 512), sizes that are not multiples of the
    1024-column block or of the 8-row batch, and several tokens; shared expert included."""
    case = _kmajor_case(T, E, H, I, k, 700 + T, dtype)
    want = O.moe_forward_full_kmajor(*case, k)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    x, logits, w13, s13, sw13, ss13, w2, s2, sw2, ss2, gate = case
    args = (x.to(dev), logits.to(dev), f8(w13), s13.to(dev), f8(sw13), ss13.to(dev), f8(w2), s2.to(dev), f8(sw2),
            ss2.to(dev), gate.to(dev), k, 1, E)
    got = torch.ops.moe_ops.moe_forward_full(*args)
    assert got.shape == (T, H) and got.dtype == dtype
    # the op rounds the routed and the shared intermediates to the activation type (w8a16 chain):
    # the mean-based bar of the reference's block-FP8 test plus a max bar three roundings wide
    diff = (got.cpu().float() - want).abs()
    assert (diff.mean() / want.abs().mean()).item() < 3e-3
    assert O.max_rel_err(got.cpu().float(), want) < 3 * TOL
    again = torch.ops.moe_ops.moe_forward_full_v2(*args)
    assert torch.equal(again.cpu(), got.cpu())                  # fixed summation order


def test_moe_forward_full_kmajor_no_shared_expert(v, dev):
    T, E, H, I, k = 2, 8, 512, 256, 2
    x, logits, w13, s13, _, _, w2, s2, _, _, _ = _kmajor_case(T, E, H, I, k, 41, torch.float16, shared=False)
    want = O.moe_forward_full_kmajor(x, logits, w13, s13, None, None, w2, s2, None, None, None, k)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    e = torch.empty(0, device=dev)
    got = torch.ops.moe_ops.moe_forward_full(x.to(dev), logits.to(dev), f8(w13), s13.to(dev), e, e, f8(w2), s2.to(dev), e, e,
                                             e, k, 0, E)
    assert O.max_rel_err(got.cpu().float(), want) < 2 * TOL


def test_kmajor_out_of_range_expert_ids_contribute_zero(v, dev):
    """Routes whose expert id is not in [0, E) must not be dereferenced: their partial rows are zero and
    they add nothing to the output (the host forces the condition; every kernel exits normally)."""
    from mi355x_qlinear import capi
    g = torch.Generator().manual_seed(8)
    E, H, I, k = 2, 256, 64, 3
    x = (torch.randn(1, H, generator=g) * 0.3).half()
    w13 = O.e4m3_quantize(torch.randn(E, H, 2 * I, generator=g))
    w2 = O.e4m3_quantize(torch.randn(E, I, H, generator=g))
    s13 = torch.tensor([0.01, 0.02])
    s2 = torch.tensor([0.03, 0.015])
    ids = torch.tensor([1, -1, 99], dtype=torch.int32)
    tw = torch.tensor([[0.5, 0.3, 0.2]]).half()
    d = lambda t: t.to(dev)
    xd, w13d, w2d, idd, twd, s13d, s2d = d(x), d(w13), d(w2), d(ids), d(tw), d(s13), d(s2)
    su, sd = 2, 2
    up = torch.full((k, su, 2 * I), float("nan"), device=dev)
    capi.call("mi_moe_kmajor_up", xd, capi.ptr(xd), capi.ptr(w13d), capi.ptr(idd), capi.ptr(up), k, k, E, H, 2 * I, su,
              capi.DT_F16)
    assert torch.isfinite(up).all() and (up[1:] == 0).all() and (up[0] != 0).any()
    dn = torch.full((k, sd, H), float("nan"), device=dev)
    capi.call("mi_moe_kmajor_down", xd, capi.ptr(up), su, capi.ptr(s13d), capi.ptr(w2d), capi.ptr(idd), capi.ptr(dn), k, E, I, H,
              sd, 0, capi.DT_F16)
    assert torch.isfinite(dn).all() and (dn[1:] == 0).all()
    out = torch.empty(1, H, dtype=torch.float16, device=dev)
    capi.call("mi_moe_kmajor_finalize", xd, capi.ptr(dn), sd, capi.ptr(s2d), capi.ptr(idd), capi.ptr(twd), None, None,
              capi.ptr(out), 1, k, E, H, capi.DT_F16)
    d13 = O.e4m3_decode(w13[1].reshape(-1, 2 * I)).reshape(H, 2 * I)
    gu = (x.float()[0] @ d13) * s13[1]
    inter = (torch.nn.functional.silu(gu[:I]) * gu[I:]).half().float()
    want = 0.5 * s2[1] * (inter @ O.e4m3_decode(w2[1].reshape(-1, H)).reshape(I, H))
    assert O.max_rel_err(out.cpu().float()[0], want) < TOL


def test_package_level_moe_batch_helpers(v, dev):
    """moe_router_forward / moe_batch_topk / moe_accumulate as attributes of both packages, the names the
    reference packages re-export (V/python/custom_esimd_kernels_vllm/ops.py:931-1030): same results as the
    torch.ops.moe_ops operators they call."""
    import custom_esimd_kernels_sglang as s
    T, E, H, k = 5, 64, 256, 4
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g).half().to(dev)
    w8, sc = O.fp8_quantize_per_channel(torch.randn(E, H, generator=g) * 0.05)
    sc1 = sc.mean().reshape(1).expand(E).contiguous()        # per-tensor: one value for every expert
    for pkg in (v, s):
        logits = pkg.moe_router_forward(x, w8.view(torch.float8_e4m3fn).to(dev), sc1.to(dev))
        want = torch.ops.moe_ops.moe_router_forward(x, w8.view(torch.float8_e4m3fn).to(dev), sc1.to(dev))
        assert torch.equal(logits, want) and logits.shape == (T, E)
        tv, ti = pkg.moe_batch_topk(logits, k)
        wv, wi = O.moe_topk(logits.cpu(), k)
        assert torch.equal(ti.cpu(), wi.to(torch.int32)) and O.max_rel_err(tv.cpu(), wv) < TOL
        parts = torch.randn(T * k, H, generator=g).half().to(dev)
        acc = pkg.moe_accumulate(parts, k, 0)
        assert O.max_rel_err(acc.cpu(), parts.cpu().float().view(T, k, H).sum(1)) < TOL
