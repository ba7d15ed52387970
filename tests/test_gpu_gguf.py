"""GPU parity for the weight-preparation side: GGUF Q4_0 / Q8_0 / Q5_K / Q6_K repack,
dequant and decode GEMV, and the group-128 Q4_0 quantizer, through torch.ops ->
ctypes -> the C ABI, against the CPU oracle.

Bars: repack outputs, dequantized weights and quantizer outputs bit-exact; GEMV
outputs within max relative error 1e-2 of the fp32-accumulated reference on the
oracle's dequantized weights.
"""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as G
from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def ops(dev):
    import custom_esimd_kernels_vllm as v
    import custom_esimd_kernels_sglang as s
    return v, s


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def _f16u(rng, shape, lo, hi):
    return rng.uniform(lo, hi, size=shape).astype(np.float16)


def _raw_case(kind, N, K, seed):
    rng = np.random.default_rng(seed)
    if kind == "q4_0":
        d = _f16u(rng, (N, K // 32), -0.02, 0.02)
        return G.q4_0_build_raw(rng.integers(0, 16, size=(N, K), dtype=np.uint8), d)
    if kind == "q8_0":
        d = _f16u(rng, (N, K // 32), -0.002, 0.002)
        return G.q8_0_build_raw(rng.integers(-128, 128, size=(N, K)).astype(np.int8), d)
    nsb = K // 256
    if kind == "q5_k":
        sc12 = O.q4k_pack_scales(rng.integers(0, 64, size=(N, nsb, 8)), rng.integers(0, 64, size=(N, nsb, 8)))
        return G.q5k_build_raw(rng.integers(0, 32, size=(N, K)), sc12, _f16u(rng, (N, nsb), 0.0005, 0.005),
                               _f16u(rng, (N, nsb), 0.0, 0.003))
    sc = rng.integers(-128, 128, size=(N, nsb, 16)).astype(np.int8)
    return G.q6k_build_raw(rng.integers(0, 64, size=(N, K)), sc, _f16u(rng, (N, nsb), 0.00002, 0.0002))


def _repack_oracle(kind, raw):
    return {"q4_0": G.q4_0_repack, "q8_0": G.q8_0_repack, "q5_k": G.q5k_repack, "q6_k": G.q6k_repack}[kind](raw)


def _dequant_oracle(kind, rep):
    return {"q4_0": G.q4_0_dequant, "q8_0": G.q8_0_dequant, "q5_k": G.q5k_dequant, "q6_k": G.q6k_dequant}[kind](*rep)


def _repack_gpu(s, kind, raw, dev):
    N = raw.shape[0]
    r = _t(raw).to(dev)
    if kind == "q4_0":
        K = raw.shape[1] // 18 * 32
        out = (torch.empty(N, K // 2, dtype=torch.uint8, device=dev), torch.empty(N, K // 32, dtype=torch.float16, device=dev))
        s.q4_0_repack(r, *out)
    elif kind == "q8_0":
        K = raw.shape[1] // 34 * 32
        out = (torch.empty(N, K, dtype=torch.int8, device=dev), torch.empty(N, K // 32, dtype=torch.float16, device=dev))
        s.q8_0_repack(r, *out)
    elif kind == "q5_k":
        K = raw.shape[1] // 176 * 256
        out = (torch.empty(N, K // 2, dtype=torch.uint8, device=dev), torch.empty(N, K // 8, dtype=torch.uint8, device=dev),
               torch.empty(N, K // 32, dtype=torch.float16, device=dev), torch.empty(N, K // 32, dtype=torch.float16, device=dev))
        s.q5_k_repack(r, *out)
    else:
        K = raw.shape[1] // 210 * 256
        out = (torch.empty(N, K // 2, dtype=torch.uint8, device=dev), torch.empty(N, K // 4, dtype=torch.uint8, device=dev),
               torch.empty(N, K // 16, dtype=torch.float16, device=dev))
        s.q6_k_repack(r, *out)
    return out, K


def _same(a_gpu, b_np):
    a = a_gpu.cpu().numpy()
    if a.dtype == np.float16:
        return np.array_equal(a.view(np.uint16), np.asarray(b_np).view(np.uint16))
    return np.array_equal(a.view(np.uint8), np.asarray(b_np).view(np.uint8))


KINDS = ["q4_0", "q8_0", "q5_k", "q6_k"]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("N,K", [(3, 512), (64, 2048), (17, 5120)])
def test_repack_and_dequant_bit_exact(ops, dev, kind, N, K):
    _, s = ops
    raw = _raw_case(kind, N, K, seed=N + K)
    ref = _repack_oracle(kind, raw)
    got, K2 = _repack_gpu(s, kind, raw, dev)
    assert K2 == K
    for g, r in zip(got, ref):
        assert _same(g, r)
    dense = torch.empty(N, K, dtype=torch.float16, device=dev)
    getattr(s, f"{kind}_dequant")(*got, dense)
    assert _same(dense, _dequant_oracle(kind, ref))


@pytest.mark.parametrize("kind", KINDS)
def test_dequant_extreme_scales(ops, dev, kind):
    # negative, subnormal-product and large scales / mins: roundings must still match bit for bit
    _, s = ops
    N, K = 8, 1024
    raw = _raw_case(kind, N, K, seed=99)
    rep = [np.array(a) for a in _repack_oracle(kind, raw)]
    sc = rep[-2] if kind == "q5_k" else rep[-1]
    sc[0, :4] = np.array([-0.875, 6.0e-5, 1.0e-7, 300.0], dtype=np.float16)
    if kind == "q5_k":
        rep[-1][0, :4] = np.array([0.3333, -2.5, 6.0e-8, 1000.0], dtype=np.float16)
    dense = torch.empty(N, K, dtype=torch.float16, device=dev)
    getattr(s, f"{kind}_dequant")(*[_t(a).to(dev) for a in rep], dense)
    assert _same(dense, _dequant_oracle(kind, rep))


def _gemv(s, kind, x, rep, out, name=None):
    name = name or f"esimd_gemv_{kind}"
    return getattr(s, name)(x, *rep, out)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,N,K", [(1, 64, 512), (1, 1000, 4096), (1, 520, 5120), (2, 96, 2048), (3, 33, 1024),
                                   (4, 256, 8192), (1, 40, 14336), (7, 48, 1536), (16, 130, 2048), (33, 72, 1024),
                                   (64, 520, 5120), (100, 40, 512),
                                   # Q4_0 / Q8_0 with few rows and K % 128 == 0: x resident in registers, K sliced over wavefronts
                                   (12, 300, 5120), (40, 96, 2048), (5, 64, 1024), (16, 1000, 4096)])
def test_gemv(ops, dev, kind, M, N, K):
    _, s = ops
    raw = _raw_case(kind, N, K, seed=7 * M + N + K)
    rep = _repack_oracle(kind, raw)
    wd = torch.from_numpy(_dequant_oracle(kind, rep).astype(np.float32))
    g = torch.Generator().manual_seed(K + M)
    x = torch.randn(M, K, generator=g).half()
    out = torch.empty(M, N, dtype=torch.float16, device=dev)
    ret = _gemv(s, kind, x.to(dev), [_t(a).to(dev) for a in rep], out)
    assert ret.data_ptr() == out.data_ptr()
    ref = O.matmul_ref(x, wd)
    assert O.max_rel_err(out.cpu(), ref) < TOL


@pytest.mark.parametrize("kind", ["q5_k", "q6_k"])
@pytest.mark.parametrize("N,K", [(3, 256), (40, 768), (17, 2048)])
def test_repack_plain_bit_exact(ops, dev, kind, N, K):
    # element-order high bits of the MoE down stacks (sglang_for_multi_arc.patch:2736-2765)
    _, s = ops
    raw = _raw_case(kind, N, K, seed=3 * N + K)
    r = _t(raw).to(dev)
    u8 = lambda *sh: torch.empty(*sh, dtype=torch.uint8, device=dev)
    f16 = lambda *sh: torch.empty(*sh, dtype=torch.float16, device=dev)
    if kind == "q5_k":
        ref = G.q5k_repack_plain(raw)
        got = (u8(N, K // 2), u8(N, K // 8), f16(N, K // 32), f16(N, K // 32))
        s.q5_k_repack_plain(r, *got)
    else:
        ref = G.q6k_repack_plain(raw)
        got = (u8(N, K // 2), u8(N, K // 4), f16(N, K // 16))
        s.q6_k_repack_plain(r, *got)
    for g_, r_ in zip(got, ref):
        assert _same(g_, r_)


@pytest.mark.parametrize("T,E,k,H,I", [(1, 8, 4, 2048, 512), (3, 16, 2, 512, 1024), (2, 4, 4, 5120, 512),
                                       (1, 128, 8, 2048, 768), (5, 6, 3, 512, 96), (2, 8, 2, 256, 2080)])
def test_moe_gguf_routed_stages(ops, dev, T, E, k, H, I):
    """esimd_moe_up_q4k -> esimd_moe_down_q5k / _q6k (S/csrc/xpu/torch_extension.cc:86-101): per-route
    GEMVs on expert stacks of the repacked representations, against the per-route loop on the oracle's
    dequantized weights."""
    _, s = ops
    rng = np.random.default_rng(T + E + H)
    g = torch.Generator().manual_seed(H + I)
    x = (torch.randn(T, H, generator=g) * 0.1).half()   # keeps silu(gate) * up inside fp16 range
    sel = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).reshape(-1)
    P = T * k
    # Large expert counts: U distinct experts are generated and decoded on the CPU, and the
    # device stack of E experts repeats them through a scrambled map (expert e holds distinct
    # expert (7e + 3) % U), so the operands keep their full [E, ...] shape.
    U = min(E, 16)
    emap = (7 * torch.arange(E) + 3) % U if U < E else torch.arange(E)
    stack = lambda a: _t(a).reshape(U, -1, a.shape[-1]).to(dev)[emap.to(dev)].contiguous()
    # gate / up: Q4_K stacks [E, I, ...]
    reps, deq = [], []
    for seed in (11, 12):
        _, raw = O.make_q4k_case(1, H, U * I, seed=seed + H)
        rep = O.q4k_repack(raw)
        reps.append([stack(a) for a in rep])
        deq.append(torch.from_numpy(O.q4k_dequant(*rep).astype(np.float32)).reshape(U, I, H))
    inter = torch.empty(P, I, dtype=torch.float16, device=dev)
    ret = s.esimd_moe_up_q4k(x.to(dev), *reps[0], *reps[1], sel.to(dev), inter, T, H, I, k)
    assert ret.data_ptr() == inter.data_ptr()
    tok = torch.arange(P) // k
    e_of = emap[sel.long()]
    gate = torch.einsum("ph,pih->pi", x.float()[tok], deq[0][e_of])
    up = torch.einsum("ph,pih->pi", x.float()[tok], deq[1][e_of])
    want = torch.nn.functional.silu(gate.half().float()) * up.half().float()
    assert O.max_rel_err(inter.cpu(), want) < 2 * TOL           # gate / up are rounded to fp16 before SiLU * up
    free = torch.nn.functional.silu(gate) * up
    assert ((inter.cpu().float() - free).abs().mean() / free.abs().mean()).item() < 5e-3
    # down: Q5_K and Q6_K stacks [E, H, ...] on an intermediate of a size that keeps fp16 outputs finite
    tw = torch.rand(P, generator=g).half()
    inter = (torch.randn(P, I, generator=g) * 0.1).half().to(dev)
    for kind in ("q5_k", "q6_k"):
        # element-order ("plain") high bits: the representation the reference's down kernels
        # read and the patched loader passes (moe_kquant_GEMV.h:109-116, 159-166)
        Ip = (I + 255) // 256 * 256                       # raw super-blocks hold 256 elements
        raw = _raw_case(kind, U * H, Ip, seed=31 + I)
        full = G.q5k_repack_plain(raw) if kind == "q5_k" else G.q6k_repack_plain(raw)
        if Ip != I:                                       # K % 32 == 0: cut every row to its first I elements
            per = (2, 8, 32, 32) if kind == "q5_k" else (2, 4, 16)
            full = tuple(np.ascontiguousarray(a[:, :I // d]) for a, d in zip(full, per))
        rep = full
        deq = G.q5k_dequant_plain(*rep) if kind == "q5_k" else G.q6k_dequant_plain(*rep)
        wd = torch.from_numpy(deq.astype(np.float32)).reshape(U, H, I)
        out = torch.empty(P, H, dtype=torch.float16, device=dev)
        args = [stack(a) for a in rep]
        fn = s.esimd_moe_down_q5k if kind == "q5_k" else s.esimd_moe_down_q6k
        ret = fn(inter, *args, sel.to(dev), tw.to(dev), out, T, H, I, k)
        assert ret.data_ptr() == out.data_ptr()
        ref = torch.einsum("pi,phi->ph", inter.cpu().float(), wd[e_of]) * tw.float().view(-1, 1)
        assert O.max_rel_err(out.cpu(), ref) < TOL


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,K", [(1, 1024), (2, 4096), (4, 1024), (8, 1024), (16, 4096), (40, 2048), (64, 4096), (100, 1024)])
def test_one_hot_activations_return_the_dequantized_weights(ops, dev, kind, M, K):
    """With one 1.0 per activation row every output is a single weight: row GEMV, K-sliced and skinny kernels
    must return exactly the oracle's dequantized fp16 weight (decode, high-bit planes, scale and min
    arithmetic, output rounding), value for value.  The row GEMV (up to 4 rows for these formats) multiplies
    weights that are not rounded to fp16, like the reference's decode kernels (fp32 `d sc q - dmin m`,
    S/csrc/xpu/esimd_kernels/q4_k_GEMV.h:84-88): for Q5_K, the one format here with two roundings, its output
    is the single rounding of fp32(v5 * scale - min)."""
    _, s = ops
    N = 72
    raw = _raw_case(kind, N, K, seed=3 * M + K)
    rep = _repack_oracle(kind, raw)
    wd = torch.from_numpy(_dequant_oracle(kind, rep).astype(np.float32))
    if kind == "q5_k" and M <= 4:
        v5, sc, mn = G.q5k_elem(raw)
        one = v5.astype(np.float32) * np.repeat(sc.astype(np.float32), 32, 1) - np.repeat(mn.astype(np.float32), 32, 1)
        wd = torch.from_numpy(one.astype(np.float16).astype(np.float32))
    ks = (9 + 37 * torch.arange(M)) % K                        # 37 is coprime to K: distinct k per row
    x = torch.zeros(M, K, dtype=torch.float16)
    x[torch.arange(M), ks] = 1.0
    out = torch.empty(M, N, dtype=torch.float16, device=dev)
    _gemv(s, kind, x.to(dev), [_t(a).to(dev) for a in rep], out)
    assert torch.equal(out.cpu().float(), wd[:, ks].t())


@pytest.mark.parametrize("name,kind", [("esimd_gemm_q4_0", "q4_0"), ("esimd_gemv_q8_0_m", "q8_0"), ("esimd_gemv_q6_k_m", "q6_k")])
def test_small_m_variants(ops, dev, name, kind):
    _, s = ops
    M, N, K = 6, 200, 2048
    raw = _raw_case(kind, N, K, seed=5)
    rep = _repack_oracle(kind, raw)
    wd = torch.from_numpy(_dequant_oracle(kind, rep).astype(np.float32))
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3)).half()
    out = torch.empty(M, N, dtype=torch.float16, device=dev)
    _gemv(s, kind, x.to(dev), [_t(a).to(dev) for a in rep], out, name)
    assert O.max_rel_err(out.cpu(), O.matmul_ref(x, wd)) < TOL


@pytest.mark.parametrize("M", [1, 8])
@pytest.mark.parametrize("kind", ["q5_k", "q6_k"])
def test_gemv_every_high_bit_field(ops, dev, kind, M):
    # weights whose low nibbles are zero: the output depends on the high bits alone,
    # one 64- (Q5_K) or 128-element (Q6_K) field of one 512-tile at a time (M = 1: the row
    # kernel, M = 8: the MFMA kernel)
    _, s = ops
    N, K = 16, 1024
    span = 64 if kind == "q5_k" else 128
    for f in range(K // span):
        v = np.zeros((N, K), dtype=np.int64)
        v[:, f * span:(f + 1) * span] = 16 if kind == "q5_k" else 48
        if kind == "q5_k":
            sc12 = O.q4k_pack_scales(np.full((N, K // 256, 8), 1), np.zeros((N, K // 256, 8), dtype=np.int64))
            raw = G.q5k_build_raw(v, sc12, np.full((N, K // 256), 0.5, np.float16), np.zeros((N, K // 256), np.float16))
        else:
            raw = G.q6k_build_raw(v, np.ones((N, K // 256, 16), np.int8), np.full((N, K // 256), 0.5, np.float16))
        rep = _repack_oracle(kind, raw)
        wd = torch.from_numpy(_dequant_oracle(kind, rep).astype(np.float32))
        x = torch.randn(M, K, generator=torch.Generator().manual_seed(f)).half()
        out = torch.empty(M, N, dtype=torch.float16, device=dev)
        _gemv(s, kind, x.to(dev), [_t(a).to(dev) for a in rep], out)
        assert O.max_rel_err(out.cpu(), O.matmul_ref(x, wd)) < TOL, f"field {f}"


def test_gguf_shape_errors(ops, dev):
    _, s = ops
    x = torch.zeros(1, 256, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):          # Q5_K needs whole 512-tiles
        s.esimd_gemv_q5_k(x, torch.zeros(4, 128, dtype=torch.uint8, device=dev), torch.zeros(4, 32, dtype=torch.uint8, device=dev),
                          torch.zeros(4, 8, dtype=torch.float16, device=dev), torch.zeros(4, 8, dtype=torch.float16, device=dev),
                          torch.zeros(1, 4, dtype=torch.float16, device=dev))
    with pytest.raises(RuntimeError):          # bf16 activations are not part of the GGUF path
        s.esimd_gemv_q8_0(x.bfloat16(), torch.zeros(4, 256, dtype=torch.int8, device=dev),
                          torch.zeros(4, 8, dtype=torch.float16, device=dev), torch.zeros(1, 4, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):
        s.q4_0_repack(torch.zeros(4, 19, dtype=torch.uint8, device=dev), torch.zeros(4, 16, dtype=torch.uint8, device=dev),
                      torch.zeros(4, 1, dtype=torch.float16, device=dev))


# ------------------------------------------------------------- quantizer ----
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(1, 128), (4, 256), (16, 128), (256, 512), (1024, 2048), (512, 5120)])
def test_q4_0_quantize_bit_exact(ops, dev, dt, M, K):
    # shapes of V/tests/test_q4_0_quant_xpu.py:52-61
    v, _ = ops
    g = torch.Generator().manual_seed(M * 7 + K)
    x = (torch.randn(M, K, generator=g) * 0.5).to(dt)
    x[0, :4] = torch.tensor([7.0, -7.0, 3.0, -3.0]).to(dt)          # known-answer block when K == 128 ... and ties
    if M > 1:
        x[1, :] = 0                                                  # all-zero blocks
    q = torch.empty(M, K // 8, dtype=torch.int32, device=dev)
    sc = torch.empty(M, K // 128, dtype=torch.float16, device=dev)
    assert v.q4_0_quantize(x.to(dev), q, sc) is None
    rq, rs = G.q4_0_quantize(x.float().numpy())
    assert np.array_equal(sc.cpu().numpy().view(np.uint16), rs.view(np.uint16))
    assert np.array_equal(q.cpu().numpy(), rq)


def test_q4_0_quantize_feeds_int4_gemv(ops, dev):
    # quantize on the device, run the int4 GEMV on the result, compare with the dense product
    v, _ = ops
    N, K = 512, 4096
    g = torch.Generator().manual_seed(11)
    w = (torch.randn(N, K, generator=g) * 0.05).half()
    x = torch.randn(1, K, generator=g).half()
    q = torch.empty(N, K // 8, dtype=torch.int32, device=dev)
    sc = torch.empty(N, K // 128, dtype=torch.float16, device=dev)
    v.q4_0_quantize(w.to(dev), q, sc)
    out = torch.empty(1, N, dtype=torch.float16, device=dev)
    v.esimd_gemv_int4(x.to(dev), q.view(torch.uint8), sc, out)
    wd = O.int4_dequant(q.cpu().view(torch.uint8), sc.cpu(), out_dtype=torch.float16)
    assert O.max_rel_err(out.cpu(), O.matmul_ref(x, wd)) < TOL
    # and the quantization itself stays inside the Q4_0 envelope: |w - deq| <= |d|
    err = (wd.float() - w.float()).abs()
    assert bool((err <= sc.cpu().float().abs().repeat_interleave(128, dim=1) + 1e-4).all())


# ---- grouped MoE GEMMs over chunks of expert-sorted rows (the reference's moe_grouped_gguf_xpu module) ----
def _expert_chunks(topk_ids, E, max_m, fixed):
    """The caller's chunk list (sglang_for_multi_arc.patch:2810-2887): routes sorted by expert (stable),
    one {expert, first sorted row, rows} triple per non-empty expert, experts with more than max_m rows split;
    `fixed` = the [E, 3] table with empty chunks that the small-M branch builds."""
    T, k = topk_ids.shape
    flat = topk_ids.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    tok_sorted = (torch.arange(T).repeat_interleave(k))[order].to(torch.int32)
    counts = torch.bincount(flat, minlength=E)
    start = torch.cumsum(counts, 0) - counts
    rows = []
    for e in range(E):
        s, n = int(start[e]), int(counts[e])
        if fixed:
            rows.append([e, s, n])
            continue
        while n > 0:
            c = min(max_m, n)
            rows.append([e, s, c])
            s += c
            n -= c
    return torch.tensor(rows, dtype=torch.int32).reshape(-1, 3), tok_sorted, order


def _q4k_expert_stacks(U, I, H, seeds, emap, dev):
    """Two Q4_K stacks (gate, up) of U distinct experts spread over len(emap) experts; returns the device
    representations and the oracle's dequantized weights [U, I, H]."""
    stack = lambda a: _t(a).reshape(U, -1, a.shape[-1]).to(dev)[emap.to(dev)].contiguous()
    reps, deq = [], []
    for seed in seeds:
        Hp = (H + 255) // 256 * 256                       # raw super-blocks hold 256 elements
        _, raw = O.make_q4k_case(1, Hp, U * I, seed=seed + H)
        rep = O.q4k_repack(raw)
        if Hp != H:                                       # K % 32 == 0: cut every row to its first H elements
            rep = tuple(np.ascontiguousarray(a[:, :H // d]) for a, d in zip(rep, (2, 32, 32)))
        reps.append([stack(a) for a in rep])
        deq.append(torch.from_numpy(O.q4k_dequant(*rep).astype(np.float32)).reshape(U, I, H))
    return reps, deq


@pytest.mark.parametrize("T,E,k,H,I,smallm,gathered", [
    (4, 16, 4, 2048, 512, True, False),      # multi-token verify: fixed [E, 3] table with empty chunks
    (16, 8, 2, 512, 96, True, False),        # 16 rows per chunk at most; I not a multiple of the 64-row block
    (200, 8, 2, 2048, 512, False, False),    # prefill: experts with more than 64 rows split into sub-chunks
    (90, 6, 3, 2080, 128, False, False),     # K not a multiple of 128 (partial last granule), no LDS tables
    (64, 4, 2, 256, 64, False, True),        # rows gathered by the caller (no token list)
    (300, 128, 8, 2048, 768, False, False),  # many experts, few rows each
])
def test_moe_grouped_q4k_up(ops, dev, T, E, k, H, I, smallm, gathered):
    """moe_up_q4k_ggemv (S/csrc/moe_grouped/moe_grouped_entry.sycl:24-60, moe_q4k_ggemv.h:47-201): gate and up
    projections of every chunk against the per-chunk product on the oracle's dequantized weights; rows no
    chunk covers keep the caller's zeros."""
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    g = torch.Generator().manual_seed(T + H + I)
    x = (torch.randn(T, H, generator=g) * 0.1).half()
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    chunks, tok_sorted, _ = _expert_chunks(ids, E, 16 if smallm else 64, fixed=smallm)
    U = min(E, 8)
    emap = (7 * torch.arange(E) + 3) % U if U < E else torch.arange(E)
    reps, deq = _q4k_expert_stacks(U, I, H, (21, 22), emap, dev)
    P = T * k
    buf = torch.zeros(P, 2 * I, dtype=torch.float16, device=dev)
    if gathered:
        xin = x[tok_sorted.long()].contiguous().to(dev)
        ret = mg.moe_up_q4k_ggemv(xin, *reps[0], *reps[1], buf, chunks.to(dev), H, I)
    else:
        ret = mg.moe_up_q4k_ggemv(x.to(dev), *reps[0], *reps[1], buf, chunks.to(dev), H, I, tok_sorted.to(dev),
                                  smallm=smallm)
    assert ret.data_ptr() == buf.data_ptr()
    want = torch.zeros(P, 2 * I)
    for e, t0, nt in chunks.tolist():
        if nt <= 0:
            continue
        xs = x.float()[tok_sorted[t0:t0 + nt].long()]
        u = int(emap[e])
        want[t0:t0 + nt, :I] = xs @ deq[0][u].t()
        want[t0:t0 + nt, I:] = xs @ deq[1][u].t()
    assert O.max_rel_err(buf.cpu(), want) < TOL
    assert int(chunks[:, 2].sum()) == P                   # every row belongs to a chunk in these cases


def test_moe_grouped_q4k_up_chunk_semantics(ops, dev):
    """Chunks as the reference kernel treats them (moe_q4k_ggemv.h:70-73, 79-92, 173-186): nt <= 0 skipped, rows
    past the tile height (64, or 16 with smallm) not computed, rows outside every chunk untouched; here also
    experts outside [0, E), rows outside the output and token ids outside x are skipped or read as zero rows."""
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    E, H, I, R = 4, 512, 128, 200
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(50, H, generator=g) * 0.1).half()
    tok = torch.randint(0, 50, (R,), generator=g).to(torch.int32)
    tok[7] = 50                                           # past the rows of x: a zero row
    tok[8] = -3
    reps, deq = _q4k_expert_stacks(E, I, H, (31, 32), torch.arange(E), dev)
    chunks = torch.tensor([[1, 0, 20], [2, 20, 0], [0, 30, 80], [5, 120, 10], [-1, 130, 5], [3, 190, 30],
                           [2, 150, -4], [1, 400, 3]], dtype=torch.int32)
    for smallm in (False, True):
        cap = 16 if smallm else 64
        buf = torch.full((R, 2 * I), 7.0, dtype=torch.float16, device=dev)
        mg.moe_up_q4k_ggemv(x.to(dev), *reps[0], *reps[1], buf, chunks.to(dev), H, I, tok.to(dev), smallm=smallm)
        want = torch.full((R, 2 * I), 7.0)
        for e, t0, nt in chunks.tolist():
            if nt <= 0 or not 0 <= e < E or not 0 <= t0 < R:
                continue
            n = min(nt, cap, R - t0)
            ids = tok[t0:t0 + n].long()
            ok = (ids >= 0) & (ids < 50)
            xs = torch.where(ok[:, None], x.float()[ids.clamp(0, 49)], torch.zeros(1))
            want[t0:t0 + n, :I] = xs @ deq[0][e].t()
            want[t0:t0 + n, I:] = xs @ deq[1][e].t()
        got = buf.cpu().float()
        untouched = want == 7.0
        assert torch.equal(got[untouched], want[untouched])
        assert O.max_rel_err(got, want) < TOL


def _down_stack(kind, U, H, I, seed, emap, dev):
    """Q5_K / Q6_K down stack [E, H, ...] with element-order high bits and its dequantized weights [U, H, I]."""
    Ip = (I + 255) // 256 * 256                           # raw super-blocks hold 256 elements
    raw = _raw_case(kind, U * H, Ip, seed=seed)
    full = G.q5k_repack_plain(raw) if kind == "q5_k" else G.q6k_repack_plain(raw)
    if Ip != I:                                           # K % 32 == 0: cut every row to its first I elements
        per = (2, 8, 32, 32) if kind == "q5_k" else (2, 4, 16)
        full = tuple(np.ascontiguousarray(a[:, :I // d]) for a, d in zip(full, per))
    deq = G.q5k_dequant_plain(*full) if kind == "q5_k" else G.q6k_dequant_plain(*full)
    stack = lambda a: _t(a).reshape(U, -1, a.shape[-1]).to(dev)[emap.to(dev)].contiguous()
    return [stack(a) for a in full], torch.from_numpy(deq.astype(np.float32)).reshape(U, H, I)


@pytest.mark.parametrize("kind", ["q5_k", "q6_k"])
@pytest.mark.parametrize("T,E,k,H,I,smallm", [
    (4, 16, 4, 2048, 512, True),
    (16, 8, 2, 96, 512, True),               # H not a multiple of the 64-row block
    (200, 8, 2, 2048, 512, False),
    (90, 6, 3, 128, 2080 // 32 * 32, False),  # K = 2080: partial last granule
    (70, 4, 2, 256, 96, False),              # K = 96: one partial granule, rows cut inside a super-block
    (300, 128, 8, 2048, 768, False),
])
def test_moe_grouped_down(ops, dev, kind, T, E, k, H, I, smallm):
    """moe_down_q5k_ggemv / moe_down_q6k_ggemv (S/csrc/moe_grouped/moe_grouped_entry.sycl:62-106): rows of the
    intermediate in sorted order against the chunk's expert, element-order high bits."""
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    g = torch.Generator().manual_seed(T + H + I)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    chunks, _, _ = _expert_chunks(ids, E, 16 if smallm else 64, fixed=smallm)
    U = min(E, 8)
    emap = (7 * torch.arange(E) + 3) % U if U < E else torch.arange(E)
    args, wd = _down_stack(kind, U, H, I, 41 + I, emap, dev)
    P = T * k
    inter = (torch.randn(P, I, generator=g) * 0.1).half()
    out = torch.zeros(P, H, dtype=torch.float16, device=dev)
    fn = mg.moe_down_q5k_ggemv if kind == "q5_k" else mg.moe_down_q6k_ggemv
    ret = fn(inter.to(dev), *args, out, chunks.to(dev), I, H, smallm=smallm)
    assert ret.data_ptr() == out.data_ptr()
    want = torch.zeros(P, H)
    for e, t0, nt in chunks.tolist():
        if nt > 0:
            want[t0:t0 + nt] = inter.float()[t0:t0 + nt] @ wd[int(emap[e])].t()
    assert O.max_rel_err(out.cpu(), want) < TOL


@pytest.mark.parametrize("kind", ["q5_k", "q6_k"])
def test_moe_grouped_down_every_high_bit(ops, dev, kind):
    """Weights whose low nibbles are zero and whose high bits are set for ONE element per row at a time: the
    output then is that element's activation times (16 or 48 - 32) * scale, so a high-bit field read for the
    wrong element shows up as a wrong column of the intermediate."""
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    E, H, I = 1, 16, 256
    chunks = torch.tensor([[0, 0, 3]], dtype=torch.int32, device=dev)
    inter = (torch.arange(3 * I).reshape(3, I) % 97 + 1).half() / 64          # distinct per element within a row
    for e0 in list(range(0, 40)) + [63, 64, 127, 128, 200, 255]:
        v = np.zeros((H, I), dtype=np.int64)
        v[:, e0] = 16 if kind == "q5_k" else 48
        if kind == "q5_k":
            sc12 = O.q4k_pack_scales(np.full((H, 1, 8), 1), np.zeros((H, 1, 8), dtype=np.int64))
            raw = G.q5k_build_raw(v + 0, sc12, np.full((H, 1), 0.5, np.float16), np.zeros((H, 1), np.float16))
            rep = G.q5k_repack_plain(raw)
            wd = G.q5k_dequant_plain(*rep)
        else:
            raw = G.q6k_build_raw(v + 32 * (v == 0), np.full((H, 1, 16), 1, np.int8), np.full((H, 1), 0.5, np.float16))
            rep = G.q6k_repack_plain(raw)
            wd = G.q6k_dequant_plain(*rep)
        wd = torch.from_numpy(wd.astype(np.float32))
        assert int((wd != 0).sum()) == H and bool((wd[:, e0] != 0).all())
        out = torch.zeros(3, H, dtype=torch.float16, device=dev)
        args = [_t(a).unsqueeze(0).to(dev) for a in rep]
        fn = mg.moe_down_q5k_ggemv if kind == "q5_k" else mg.moe_down_q6k_ggemv
        fn(inter.to(dev), *args, out, chunks, I, H)
        assert torch.equal(out.cpu().float(), (inter.float() @ wd.t()).half().float()), e0


def test_moe_grouped_prefill_flow(ops, dev):
    """The caller's whole grouped prefill (sglang_for_multi_arc.patch:2810-2950): sort routes by expert -> Q4_K up
    over chunks with the gather folded in -> SiLU * up -> Q5_K down -> gather + weighted sum per token, against
    the same chain on the oracle's dequantized weights."""
    v, s = ops
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    # the caller takes these names from the sglang package first (patch :2077-2087, :2134-2138)
    silu_mul, gather = s.esimd_moe_silu_mul, s.esimd_moe_gather
    T, E, k, H, I = 150, 8, 2, 512, 256
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(T, H, generator=g) * 0.1).half()
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    tw = torch.rand(T, k, generator=g).half()
    chunks, tok_sorted, order = _expert_chunks(ids, E, 64, fixed=False)
    reps, deq = _q4k_expert_stacks(E, I, H, (51, 52), torch.arange(E), dev)
    dargs, wd = _down_stack("q5_k", E, H, I, 53, torch.arange(E), dev)
    P = T * k
    gate_buf = torch.zeros(P, 2 * I, dtype=torch.float16, device=dev)
    mg.moe_up_q4k_ggemv(x.to(dev), *reps[0], *reps[1], gate_buf, chunks.to(dev), H, I, tok_sorted.to(dev))
    inter = torch.empty(P, I, dtype=torch.float16, device=dev)
    silu_mul(gate_buf, inter, 2 * I, I, P)
    out_route = torch.zeros(P, H, dtype=torch.float16, device=dev)
    mg.moe_down_q5k_ggemv(inter, *dargs, out_route, chunks.to(dev), I, H)
    inv = torch.argsort(order)
    pos = inv.to(torch.int32).reshape(T, k).contiguous()
    w_sorted = tw.reshape(-1)[order].contiguous()
    final = torch.empty(T, H, dtype=torch.float16, device=dev)
    gather(out_route, pos.to(dev), w_sorted.to(dev), final, H, k, T)
    want = torch.zeros(T, H)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            gu = x.float()[t] @ deq[0][e].t(), x.float()[t] @ deq[1][e].t()
            h = (torch.nn.functional.silu(gu[0].half().float()) * gu[1].half().float()).half().float()
            want[t] += float(tw[t, j]) * (h @ wd[e].t()).half().float()
    assert O.max_rel_err(final.cpu(), want) < 2 * TOL      # three fp16 roundings on the way


@pytest.mark.parametrize("smallm", [False, True])
def test_moe_grouped_one_hot_rows_return_the_experts_weights(ops, dev, smallm):
    """One 1.0 per row of x: every output of the grouped launches is a single dequantized weight of the chunk's
    expert — Q4_K gate / up, Q5_K and Q6_K down with element-order high bits — compared value for value."""
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    E, H, I, T, k = 6, 768, 512, 40, 2
    g = torch.Generator().manual_seed(77)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    chunks, tok_sorted, _ = _expert_chunks(ids, E, 16 if smallm else 64, fixed=False)
    P = T * k
    e_of = torch.empty(P, dtype=torch.long)
    for e, t0, nt in chunks.tolist():
        e_of[t0:t0 + nt] = e
    # up: x [T, H] one-hot per token, gathered through the token list
    kx = (3 + 37 * torch.arange(T)) % H
    x = torch.zeros(T, H, dtype=torch.float16)
    x[torch.arange(T), kx] = 1.0
    reps, deq = _q4k_expert_stacks(E, I, H, (61, 62), torch.arange(E), dev)
    buf = torch.zeros(P, 2 * I, dtype=torch.float16, device=dev)
    mg.moe_up_q4k_ggemv(x.to(dev), *reps[0], *reps[1], buf, chunks.to(dev), H, I, tok_sorted.to(dev), smallm=smallm)
    kk = kx[tok_sorted.long()]
    want = torch.cat([deq[0][e_of, :, kk], deq[1][e_of, :, kk]], 1)
    assert torch.equal(buf.cpu().float(), want)
    # down: the intermediate [P, I] one-hot per route
    ki = (7 + 37 * torch.arange(P)) % I
    inter = torch.zeros(P, I, dtype=torch.float16)
    inter[torch.arange(P), ki] = 1.0
    for kind in ("q5_k", "q6_k"):
        args, wd = _down_stack(kind, E, H, I, 63, torch.arange(E), dev)
        out = torch.zeros(P, H, dtype=torch.float16, device=dev)
        fn = mg.moe_down_q5k_ggemv if kind == "q5_k" else mg.moe_down_q6k_ggemv
        fn(inter.to(dev), *args, out, chunks.to(dev), I, H, smallm=smallm)
        assert torch.equal(out.cpu().float(), wd[e_of, :, ki]), kind
