"""HIP-graph capture parity: one operator of each family is captured into a graph after one
warm-up call, the graph is replayed several times with eager work and synchronisations in
between, and every replay must reproduce the eager result bit for bit
(vllm/patches/vllm_for_multi_arc.patch:2793-2937 registers the operators for graph use).
"""
import numpy as np
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    import custom_esimd_kernels_vllm as v
    import custom_esimd_kernels_sglang as s
    return v, s


def _check_graph(dev, run, outputs, reset=None, replays=3):
    """run(): launches the operator on the current stream writing `outputs` (tensors);
    reset(): restores inputs the operator updates in place."""
    if reset:
        reset()
    run()                                                 # eager: the expected result (also the warm-up)
    torch.cuda.synchronize()
    want = [o.clone() for o in outputs]
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    if reset:
        reset()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            run()
    for r in range(replays):
        for o in outputs:
            o.fill_(float("nan")) if o.is_floating_point() else o.zero_()
        if reset:
            reset()
        # eager work of the program's own between the replays
        junk = torch.randn(256, 256, device=dev) @ torch.randn(256, 256, device=dev)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del junk
        for o, w in zip(outputs, want):
            assert torch.equal(o.view(torch.uint8), w.view(torch.uint8)), f"replay {r} differs from the eager call"


def test_graph_int4_gemv(ops, dev):
    v, _ = ops
    x, packed, scale, _ = O.make_int4_case(1, 4096, 1024, seed=21)
    xd, wd, sd = x.to(dev), packed.to(dev), scale.to(dev)
    out = torch.empty(1, 1024, dtype=torch.float16, device=dev)
    _check_graph(dev, lambda: v.esimd_gemv_int4(xd, wd, sd, out), [out])


def test_graph_fp8_pern_m8(ops, dev):
    v, _ = ops
    M, K, N = 8, 2048, 1536
    x, w8, s = O.make_fp8_pern_case(M, K, N, seed=22)
    xd, wd, sd = x.to(dev), w8.view(torch.float8_e4m3fn).to(dev), s.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _check_graph(dev, lambda: v.esimd_gemv_fp8_pern(xd, wd, sd, out, N, K), [out])


def test_graph_int4_m16_and_fp8_m64(ops, dev):
    # the K-sliced kernel on INT4 (16 rows) and the row-split launch of the skinny kernel (64 rows of x
    # against 16 weight rows per CU)
    v, _ = ops
    x, packed, scale, _ = O.make_int4_case(16, 2048, 1024, seed=31)
    xd, wd, sd = x.to(dev), packed.to(dev), scale.to(dev)
    out = torch.empty(16, 1024, dtype=torch.float16, device=dev)
    _check_graph(dev, lambda: v.esimd_gemm_int4_pgrp(xd, wd, sd, out), [out])
    M, K, N = 64, 4096, 4096
    x, w8, s = O.make_fp8_pern_case(M, K, N, seed=32)
    xf, wf, sf = x.to(dev), w8.view(torch.float8_e4m3fn).to(dev), s.to(dev)
    out2 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _check_graph(dev, lambda: v.esimd_gemv_fp8_pern(xf, wf, sf, out2, N, K), [out2])


def test_graph_int4_gemm(ops, dev):
    v, _ = ops
    M, K, N = 200, 1024, 512
    x, packed, scale, zp = O.make_int4_case(M, K, N, seed=23, act_dtype=torch.bfloat16, asym=True)
    xd, wd, sd, zd = x.to(dev), packed.to(dev), scale.to(dev), zp.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _check_graph(dev, lambda: v.esimd_gemm_int4_pgrp_zp(xd, wd, sd, zd, out), [out])


def test_graph_moe_forward_fp8_block(ops, dev):
    v, _ = ops
    T, E, k, H, I = 48, 16, 4, 512, 256
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, k, H, I, seed=24)
    f8 = lambda t: t.view(torch.float8_e4m3fn).to(dev)
    args = (x.to(dev), logits.to(dev), f8(w13q), w13s.to(dev), f8(w2q), w2s.to(dev))
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    _check_graph(dev, lambda: v.moe_forward_fp8_block(*args, out, k, True), [out])


def test_graph_fused_norm_gemv(ops, dev):
    v, _ = ops
    # a full grid: the arrival counters are in play.  The capture stream has never run the operator
    # (the eager call went to the default stream): its counter block must come from the device's
    # pool without an allocation during the capture.
    K, N = 4096, 14336
    g = torch.Generator().manual_seed(25)
    hidden = torch.randn(1, K, generator=g).half().to(dev)
    res0 = torch.randn(1, K, generator=g).half().to(dev)
    nw = (torch.randn(K, generator=g) * 0.1 + 1.0).half().to(dev)
    w8 = O.e4m3_quantize((torch.randn(N, K, generator=g) * 100).clamp(-448, 448)).view(torch.float8_e4m3fn).to(dev)
    sc = torch.tensor([3.0e-3]).to(dev)
    res = res0.clone()
    out = torch.empty(1, N, dtype=torch.float16, device=dev)
    normed = torch.empty(1, K, dtype=torch.float16, device=dev)
    _check_graph(dev, lambda: v.esimd_resadd_norm_gemv_fp8_pert(hidden, res, nw, w8, sc, out, normed, 1e-6),
                 [out, normed, res], reset=lambda: res.copy_(res0))


def test_graph_q4k_gemv(ops, dev):
    _, s = ops
    x, raw = O.make_q4k_case(1, 2048, 640, seed=26)
    ql, sc, mn = (torch.from_numpy(a).to(dev) for a in O.q4k_repack(raw))
    xd = x.to(dev)
    out = torch.empty(1, 640, dtype=torch.float16, device=dev)
    _check_graph(dev, lambda: s.esimd_gemv_q4_k(xd, ql, sc, mn, out), [out])


def test_graph_grouped_gguf_moe(ops, dev):
    # the verify-step use of the grouped module (fixed [E, 3] chunk table, 16-row tiles) is what the caller
    # captures (sglang/patches/sglang_for_multi_arc.patch:2850-2870); the 64-row form as well
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    E, H, I, T, k = 8, 512, 128, 12, 2
    g = torch.Generator().manual_seed(41)
    u8 = lambda *sh: torch.randint(0, 256, sh, dtype=torch.uint8, generator=g).to(dev)
    f16 = lambda hi, *sh: (torch.rand(*sh, generator=g) * hi).half().to(dev)
    up = [u8(E, I, H // 2), f16(0.01, E, I, H // 32), f16(0.005, E, I, H // 32)] * 2
    down = [u8(E, H, I // 2), u8(E, H, I // 4), f16(0.002, E, H, I // 16)]
    x = (torch.randn(T, H, generator=g) * 0.1).half().to(dev)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    flat = ids.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    tok = torch.arange(T).repeat_interleave(k)[order].to(torch.int32).to(dev)
    counts = torch.bincount(flat, minlength=E)
    chunks = torch.stack([torch.arange(E), torch.cumsum(counts, 0) - counts, counts], 1).to(torch.int32).to(dev)
    P = T * k
    gate_buf = torch.zeros(P, 2 * I, dtype=torch.float16, device=dev)
    out = torch.zeros(P, H, dtype=torch.float16, device=dev)
    inter = (torch.randn(P, I, generator=g) * 0.1).half().to(dev)
    for smallm in (True, False):
        def run():
            mg.moe_up_q4k_ggemv(x, *up, gate_buf, chunks, H, I, tok, smallm=smallm)
            mg.moe_down_q6k_ggemv(inter, *down, out, chunks, I, H, smallm=smallm)
        _check_graph(dev, run, [gate_buf, out])
