#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--all]

A step is one launch of the hot-path op on one batch of seeded synthetic input.
The headline workload (default) is the second benchmark configuration: FP8 per-channel
weight-only GEMV, M=1, K=4096, N=14336, bf16 activations.  Each step uses the
next of R distinct weight copies (R x weight bytes >> the 256 MB Infinity Cache)
so the figure is HBM bandwidth, not cache bandwidth.  The K timed steps are
exactly K launches, all of them nodes of HIP graphs replayed back to back on one
stream and bracketed by a device synchronise on both sides; HIP events recorded
on that same stream give the average per-launch duration used for the roofline
fraction.

Prints ONE JSON line.  `value` is the algorithmic bytes moved per second with
inputs resident in HBM.  `cases` holds the other benchmark configurations (W4A16
GEMV, FP8 GEMV at M = 8 / 32, W4A16 prefill GEMM, block-FP8 MoE forward, Q4_K at
M = 1 / 64), each timed the same way with its own `roofline` and `cpu_baseline`;
`--only` leaves them out, `--all` adds the workloads beyond the configurations.
`cpu_baseline` times the reference's CPU path (torch dequant + fp32 matmul,
restated in oracle/) on this host's cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "llm-scaler_amd"))

import torch  # noqa: E402

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "fp8": 5000.0}
CACHE_BUST_BYTES = 1 << 30       # rotate over >= 1 GiB of distinct weights (4 x Infinity Cache)


# ----------------------------------------------------------------------------
# workloads: each returns (launch(i), alg_bytes, alg_flops, bound, dtype, descr, cpu_fn)
# ----------------------------------------------------------------------------
_CACHE = {}


def _copies(nbytes: int) -> int:
    return max(2, -(-CACHE_BUST_BYTES // nbytes))


def wl_fp8_pern(M: int, dev):
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    K, N = 4096, 14336
    R = _copies(N * K)
    if "fp8_pern" not in _CACHE:    # the three M of this configuration share the weights
        _, w8, s = O.make_fp8_pern_case(1, K, N)
        g = torch.Generator().manual_seed(99)
        ws = [w8.to(dev)]
        for _ in range(R - 1):      # distinct contents per copy, same distribution (row permutation)
            ws.append(w8[torch.randperm(N, generator=g)].to(dev))
        _CACHE["fp8_pern"] = (w8, s, [w.view(torch.float8_e4m3fn) for w in ws])
    w8, s, ws = _CACHE["fp8_pern"]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(1235)).to(torch.bfloat16)
    xd, sd = x.to(dev), s.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    def launch(i):
        v.esimd_gemv_fp8_pern(xd, ws[i % R], sd, out, N, K)

    def cpu():
        return O.matmul_ref(x, O.fp8_dequant_per_channel(w8, s)).to(torch.bfloat16)

    alg_bytes = N * K + 4 * N + 2 * M * K + 2 * M * N
    return dict(launch=launch, R=R, bytes=alg_bytes, flops=2 * M * N * K, bound="hbm", dtype="bf16",
                name=f"cfg1 FP8 e4m3 per-channel weight-only GEMV M={M} K={K} N={N} bf16",
                kernel="gemv_rows_kernel" if M <= 4 else "kslice_kernel", cpu=cpu)


def wl_int4_gemv(dev, M=1, N=4096):
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    K = 4096
    x, packed, scale, _ = O.make_int4_case(M, K, N)
    R = _copies(N * K // 2)
    g = torch.Generator().manual_seed(98)
    ws, ss = [packed.to(dev)], [scale.to(dev)]
    for _ in range(R - 1):
        p = torch.randperm(N, generator=g)
        ws.append(packed[p].to(dev))
        ss.append(scale[p].to(dev))
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)

    def launch(i):
        v.esimd_gemv_int4(xd, ws[i % R], ss[i % R], out)

    def cpu():
        return O.matmul_ref(x, O.int4_dequant(packed, scale)).to(torch.float16)

    alg_bytes = N * K // 2 + N * (K // 128) * 2 + M * K * 2 + M * N * 2
    cfg0 = M == 1 and N == 4096
    return dict(launch=launch, R=R, bytes=alg_bytes, flops=2 * M * N * K, bound="hbm", dtype="f16",
                name=("cfg0" if cfg0 else "next:") + f" W4A16 group-128 GEMV M={M} K={K} N={N} fp16",
                kernel="gemv_rows_kernel" if M <= 2 else "kslice_kernel", cpu=cpu)


def wl_q4k(M: int, dev):
    import custom_esimd_kernels_sglang as s
    from oracle import qlinear_oracle as O
    K = N = 5120
    x, raw = O.make_q4k_case(M, K, N)
    ql, sc, mn = O.q4k_repack(raw)
    qlt, sct, mnt = torch.from_numpy(ql), torch.from_numpy(sc), torch.from_numpy(mn)
    per = N * K // 2 + 2 * N * (K // 32) * 2
    R = _copies(per)
    g = torch.Generator().manual_seed(97)
    W = [(qlt.to(dev), sct.to(dev), mnt.to(dev))]
    for _ in range(R - 1):
        p = torch.randperm(N, generator=g)
        W.append((qlt[p].to(dev), sct[p].to(dev), mnt[p].to(dev)))
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)

    def launch(i):
        a, b, c = W[i % R]
        s.esimd_gemv_q4_k(xd, a, b, c, out)

    n_cpu = N                                     # weight rows of the CPU sample (all of them)

    def cpu():
        return O.matmul_ref(x, torch.from_numpy(O.q4k_dequant(ql[:n_cpu], sc[:n_cpu], mn[:n_cpu]))).to(torch.float16)

    alg_bytes = per + 2 * M * K + 2 * M * N
    return dict(launch=launch, R=R, bytes=alg_bytes, flops=2 * M * N * K, bound="hbm", dtype="f16",
                name=f"cfg4 GGUF Q4_K (repacked) dequant-matmul M={M} K={K} N={N} fp16",
                kernel="gemv_rows_kernel" if M <= 4 else "skinny_kernel", cpu=cpu, cpu_scale=n_cpu / N,
                cpu_what=f"{n_cpu} of the {N} weight rows")


def wl_gguf(kind: str, M: int, dev):
    """Decode GEMV on the other GGUF formats at the cfg4 shape (next-row workloads)."""
    import custom_esimd_kernels_sglang as s
    import numpy as np
    from oracle import gguf_oracle as G
    from oracle import qlinear_oracle as O
    K = N = 5120
    rng = np.random.default_rng(1240)
    f16u = lambda shape, lo, hi: rng.uniform(lo, hi, size=shape).astype(np.float16)
    nsb = K // 256
    if kind == "q4_0":
        raw = G.q4_0_build_raw(rng.integers(0, 16, size=(N, K), dtype=np.uint8), f16u((N, K // 32), -0.02, 0.02))
        rep, deq, op = G.q4_0_repack(raw), G.q4_0_dequant, s.esimd_gemv_q4_0
    elif kind == "q8_0":
        raw = G.q8_0_build_raw(rng.integers(-128, 128, size=(N, K)).astype(np.int8), f16u((N, K // 32), -0.002, 0.002))
        rep, deq, op = G.q8_0_repack(raw), G.q8_0_dequant, s.esimd_gemv_q8_0
    elif kind == "q5_k":
        sc12 = O.q4k_pack_scales(rng.integers(0, 64, size=(N, nsb, 8)), rng.integers(0, 64, size=(N, nsb, 8)))
        raw = G.q5k_build_raw(rng.integers(0, 32, size=(N, K)), sc12, f16u((N, nsb), 0.0005, 0.005), f16u((N, nsb), 0.0, 0.003))
        rep, deq, op = G.q5k_repack(raw), G.q5k_dequant, s.esimd_gemv_q5_k
    else:
        raw = G.q6k_build_raw(rng.integers(0, 64, size=(N, K)), rng.integers(-128, 128, size=(N, nsb, 16)).astype(np.int8),
                              f16u((N, nsb), 0.00002, 0.0002))
        rep, deq, op = G.q6k_repack(raw), G.q6k_dequant, s.esimd_gemv_q6_k
    rep_t = [torch.from_numpy(np.ascontiguousarray(a)) for a in rep]
    per = sum(t.numel() * t.element_size() for t in rep_t)
    R = _copies(per)
    g = torch.Generator().manual_seed(96)
    W = [[t.to(dev) for t in rep_t]]
    for _ in range(R - 1):
        p = torch.randperm(N, generator=g)
        W.append([t[p].to(dev) for t in rep_t])
    x = torch.randn(M, K, generator=g).half()
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)

    def launch(i):
        op(xd, *W[i % R], out)

    def cpu():
        return O.matmul_ref(x, torch.from_numpy(deq(*rep).astype(np.float32))).to(torch.float16)

    return dict(launch=launch, R=R, bytes=per + 2 * M * K + 2 * M * N, flops=2 * M * N * K, bound="hbm", dtype="f16",
                name=f"next: GGUF {kind} (repacked) decode GEMV M={M} K={K} N={N} fp16", kernel="gemv_rows_kernel", cpu=cpu)


def wl_moe_gguf(dev):
    """One decode token through the routed GGUF MoE stages (next-row workload): Q4_K gate / up,
    SiLU * up, Q6_K down over top-8 of 256 experts, H = 2048, I = 1024.  Consecutive launches route to
    consecutive groups of eight experts, so 32 launches walk the whole 1.2 GB stack once.  The stacks
    hold random codes and scales (timing only; parity is tests/test_gpu_gguf.py)."""
    import custom_esimd_kernels_sglang as s
    E, k, H, I = 256, 8, 2048, 1024
    g = torch.Generator(device="cpu").manual_seed(97)
    u8 = lambda *shape: torch.randint(0, 256, shape, dtype=torch.uint8, generator=g).to(dev)
    f16 = lambda hi, *shape: (torch.rand(*shape, generator=g) * hi).half().to(dev)
    gq, uq = u8(E, I, H // 2), u8(E, I, H // 2)
    gs, gm, us, um = f16(0.01, E, I, H // 32), f16(0.005, E, I, H // 32), f16(0.01, E, I, H // 32), f16(0.005, E, I, H // 32)
    dq, dh, ds = u8(E, H, I // 2), u8(E, H, I // 4), f16(0.002, E, H, I // 16)
    x = (torch.randn(1, H, generator=g) * 0.1).half().to(dev)
    tw = torch.full((k,), 1.0 / k, dtype=torch.float16, device=dev)
    R = E // k
    sels = [(torch.arange(k, dtype=torch.int32) + k * i).to(dev) for i in range(R)]
    inter = torch.empty(k, I, dtype=torch.float16, device=dev)
    out = torch.empty(k, H, dtype=torch.float16, device=dev)

    def launch(i):
        sel = sels[i % R]
        s.esimd_moe_up_q4k(x, gq, gs, gm, uq, us, um, sel, inter, 1, H, I, k)
        s.esimd_moe_down_q6k(inter, dq, dh, ds, sel, tw, out, 1, H, I, k)

    per = k * (2 * (I * H // 2 + 2 * I * (H // 32) * 2) + H * I // 2 + H * I // 4 + H * (I // 16) * 2)
    return dict(launch=launch, R=R, bytes=per + 2 * H + 2 * k * (3 * I + H) * 2, flops=2 * k * 3 * I * H, bound="hbm",
                dtype="f16", name=f"next: GGUF MoE decode stages T=1 top-{k} of {E} experts H={H} I={I} "
                                   "(Q4_K gate, Q4_K up, SiLU*up, Q6_K down: 4 launches)", kernel="gemv_rows_kernel", cpu=lambda: None)


def wl_moe_gguf_grouped(dev, T=2048):
    """Prefill through the grouped GGUF MoE stages (next-row workload): routes sorted by expert, Q4_K gate / up
    over chunks of at most 64 rows with the token gather inside the launch, SiLU * up, Q6_K down, weighted
    gather per token; top-8 of 128 experts, H = 2048, I = 768.  Random codes and scales (timing only; parity is
    tests/test_gpu_gguf.py)."""
    import custom_esimd_kernels_vllm as v
    from custom_esimd_kernels_sglang import moe_grouped_gguf_xpu as mg
    E, k, H, I = 128, 8, 2048, 768
    g = torch.Generator(device="cpu").manual_seed(98)
    u8 = lambda *shape: torch.randint(0, 256, shape, dtype=torch.uint8, generator=g).to(dev)
    f16 = lambda hi, *shape: (torch.rand(*shape, generator=g) * hi).half().to(dev)
    gq, uq = u8(E, I, H // 2), u8(E, I, H // 2)
    gs, gm, us, um = f16(0.01, E, I, H // 32), f16(0.005, E, I, H // 32), f16(0.01, E, I, H // 32), f16(0.005, E, I, H // 32)
    dq, dh, ds = u8(E, H, I // 2), u8(E, H, I // 4), f16(0.002, E, H, I // 16)
    x = (torch.randn(T, H, generator=g) * 0.1).half().to(dev)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    flat = ids.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    tok_sorted = torch.arange(T).repeat_interleave(k)[order].to(torch.int32).to(dev)
    counts = torch.bincount(flat, minlength=E)
    rows, s0 = [], 0
    smallm = T <= 16                                      # the caller's verify branch: fixed [E, 3] table, 16-row tiles
    for e in range(E):
        n = int(counts[e])
        if smallm:
            rows.append([e, s0, n])
            s0 += n
            continue
        while n > 0:
            c = min(64, n)
            rows.append([e, s0, c])
            s0 += c
            n -= c
    chunks = torch.tensor(rows, dtype=torch.int32).to(dev)
    P = T * k
    pos = torch.argsort(order).to(torch.int32).reshape(T, k).contiguous().to(dev)
    w_sorted = torch.full((P,), 1.0 / k, dtype=torch.float16, device=dev)
    gate_buf = torch.zeros(P, 2 * I, dtype=torch.float16, device=dev)
    inter = torch.empty(P, I, dtype=torch.float16, device=dev)
    out_route = torch.zeros(P, H, dtype=torch.float16, device=dev)
    final = torch.empty(T, H, dtype=torch.float16, device=dev)

    def launch(i):
        mg.moe_up_q4k_ggemv(x, gq, gs, gm, uq, us, um, gate_buf, chunks, H, I, tok_sorted, smallm=smallm)
        v.esimd_moe_silu_mul(gate_buf, inter, 2 * I, I, P)
        mg.moe_down_q6k_ggemv(inter, dq, dh, ds, out_route, chunks, I, H, smallm=smallm)
        v.esimd_moe_gather(out_route, pos, w_sorted, final, H, k, T)

    used = int((counts > 0).sum())                        # experts with rows: their matrices are what a launch reads
    wbytes = used * (2 * (I * H // 2 + 2 * I * (H // 32) * 2) + H * I // 2 + H * I // 4 + H * (I // 16) * 2)
    return dict(launch=launch, R=1, bytes=wbytes + 2 * T * H * 2, flops=2 * P * 3 * I * H,
                bound="hbm" if smallm else "mfma", dtype="f16",
                name=f"next: grouped GGUF MoE prefill T={T} top-{k} of {E} experts H={H} I={I} ({len(rows)} chunks; "
                     "Q4_K gate / up, SiLU*up, Q6_K down, gather: 4 launches)", kernel="skinny_kernel", cpu=lambda: None)


def wl_q4_0_quantize(dev):
    """On-device group-128 Q4_0 quantization of a [14336, 4096] bf16 weight (next-row workload)."""
    import custom_esimd_kernels_vllm as v
    from oracle import gguf_oracle as G
    rows, K = 14336, 4096
    g = torch.Generator().manual_seed(95)
    w = (torch.randn(rows, K, generator=g) * 0.02).bfloat16()
    R = _copies(rows * K * 2)
    ws = [w.to(dev)] + [w[torch.randperm(rows, generator=g)].to(dev) for _ in range(R - 1)]
    q = torch.empty(rows, K // 8, dtype=torch.int32, device=dev)
    sc = torch.empty(rows, K // 128, dtype=torch.float16, device=dev)

    def launch(i):
        v.q4_0_quantize(ws[i % R], q, sc)

    def cpu():
        return G.q4_0_quantize(w.float().numpy())

    return dict(launch=launch, R=R, bytes=rows * K * 2 + rows * K // 2 + rows * (K // 128) * 2, flops=0, bound="hbm",
                dtype="f32", name=f"next: q4_0_quantize (group 128) [{rows}, {K}] bf16 -> int4 + fp16 scales",
                kernel="q4_0_quantize_kernel", cpu=cpu)


def wl_resadd_norm_gemv(dev):
    """Residual add + RMS norm fused into the FP8 per-tensor GEMV, K=4096 N=14336 fp16 (next-row workload)."""
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    K, N = 4096, 14336
    g = torch.Generator().manual_seed(94)
    w8 = O.e4m3_quantize((torch.randn(N, K, generator=g) * 100).clamp(-448, 448))
    R = _copies(N * K)
    ws = [w8.to(dev).view(torch.float8_e4m3fn)] + [w8[torch.randperm(N, generator=g)].to(dev).view(torch.float8_e4m3fn)
                                                    for _ in range(R - 1)]
    h = torch.zeros(1, K).half()       # the op adds it into `residual` in place on every launch: keep that stationary
    res = torch.randn(1, K, generator=g).half()
    nw = (torch.randn(K, generator=g) * 0.1 + 1.0).half()
    sc = torch.tensor([2.0e-4])
    hd, nwd, scd = h.to(dev), nw.to(dev), sc.to(dev)
    resd = res.to(dev)
    out = torch.empty(1, N, dtype=torch.float16, device=dev)
    normed = torch.empty(1, K, dtype=torch.float16, device=dev)

    def launch(i):
        v.esimd_resadd_norm_gemv_fp8_pert(hd, resd, nwd, ws[i % R], scd, out, normed, 1e-6)

    def cpu():
        nr, _ = O.rmsnorm(h, nw, 1e-6, residual=res)
        return O.matmul_ref(nr.half(), O.fp8_dequant_per_tensor(w8, sc)).half()

    return dict(launch=launch, R=R, bytes=N * K + 4 + 2 * N + 5 * 2 * K, flops=2 * N * K, bound="hbm", dtype="f16",
                name=f"next: resadd + RMS norm + FP8 per-tensor GEMV M=1 K={K} N={N} fp16 (one fused launch)",
                kernel="gemv_rows_kernel", cpu=cpu)


def wl_gemm_w4a16(dev):
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    M, K, N = 2048, 4096, 14336
    x, packed, scale, zp = O.make_int4_case(M, K, N, seed=1236, act_dtype=torch.bfloat16, asym=True)
    xd, wd, sd, zd = x.to(dev), packed.to(dev), scale.to(dev), zp.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    def launch(i):
        v.esimd_gemm_int4_pgrp_zp(xd, wd, sd, zd, out)

    def cpu():
        return O.matmul_ref(x, O.int4_dequant(packed, scale, out_dtype=torch.bfloat16, zp=zp)).to(torch.bfloat16)

    alg_bytes = N * K // 2 + N * (K // 128) * 3 + 2 * M * K + 2 * M * N
    return dict(launch=launch, R=1, bytes=alg_bytes, flops=2 * M * N * K, bound="mfma", dtype="bf16",
                name=f"cfg2 W4A16 asymmetric group-128 prefill GEMM M={M} K={K} N={N} bf16",
                kernel="gemm_tiled_kernel", cpu=cpu)


def wl_fp8_prefill(dev, mode="pern"):
    """FP8 weight-only prefill GEMM at the cfg1 shape with 2048 rows (workload beyond the configurations):
    the tiled matrix-core GEMM with the FP8 weight staged through LDS."""
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    M, K, N = 2048, 4096, 14336
    g = torch.Generator().manual_seed(1241)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    if mode == "block":
        _, w8, s = O.make_fp8_block_case(1, K, N, seed=1241)
    else:
        _, w8, s = O.make_fp8_pern_case(1, K, N, seed=1241)
    xd, wd, sd = x.to(dev), w8.view(torch.float8_e4m3fn).to(dev), s.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    def launch(i):
        if mode == "block":
            v.esimd_gemm_fp8_blockscale(xd, wd, sd, out)
        else:
            v.esimd_gemv_fp8_pern(xd, wd, sd, out, N, K)

    def cpu():
        wdq = O.fp8_dequant_block(w8, s) if mode == "block" else O.fp8_dequant_per_channel(w8, s)
        return O.matmul_ref(x[:256], wdq).to(torch.bfloat16)

    alg_bytes = N * K + 4 * N + 2 * M * K + 2 * M * N
    return dict(launch=launch, R=1, bytes=alg_bytes, flops=2 * M * N * K, bound="mfma", dtype="bf16",
                name=f"next: FP8 e4m3 {'128x128-block' if mode == 'block' else 'per-channel'} weight-only prefill GEMM "
                     f"M={M} K={K} N={N} bf16", kernel="gemm_tiled_kernel", cpu=cpu, cpu_scale=256 / M,
                cpu_what=f"256 of the {M} activation rows (the whole weight is dequantized in every pass)")


def wl_q4k_prefill(dev):
    """Q4_K prefill at the cfg4 shape with 2048 rows (workload beyond the configurations)."""
    import custom_esimd_kernels_sglang as s
    from oracle import qlinear_oracle as O
    M, K, N = 2048, 5120, 5120
    x, raw = O.make_q4k_case(M, K, N, seed=1242)
    ql, sc, mn = O.q4k_repack(raw)
    W = (torch.from_numpy(ql).to(dev), torch.from_numpy(sc).to(dev), torch.from_numpy(mn).to(dev))
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)

    def launch(i):
        s.esimd_gemv_q4_k(xd, *W, out)

    def cpu():
        return O.matmul_ref(x[:256], torch.from_numpy(O.q4k_dequant(ql, sc, mn))).to(torch.float16)

    alg_bytes = N * K // 2 + 2 * N * (K // 32) * 2 + 2 * M * K + 2 * M * N
    return dict(launch=launch, R=1, bytes=alg_bytes, flops=2 * M * N * K, bound="mfma", dtype="f16",
                name=f"next: GGUF Q4_K (repacked) prefill GEMM M={M} K={K} N={N} fp16", kernel="gemm_tiled_kernel",
                cpu=cpu, cpu_scale=256 / M, cpu_what=f"256 of the {M} activation rows")


def wl_copy(dev):
    """Plain device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    n = 256 << 20
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)

    def launch(i):
        dst.copy_(src)

    return dict(launch=launch, R=1, bytes=2 * n, flops=0, bound="hbm", dtype="u8",
                name="plain device copy, 256 MiB read + 256 MiB written", kernel="copy", cpu=lambda: None)


def wl_moe(dev, T=512):
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    E, K, H, I = 128, 8, 2048, 768
    x, logits, w13q, w13s, w2q, w2s = O.make_moe_case(T, E, K, H, I)
    wbytes = E * (2 * I * H + H * I)
    R = _copies(wbytes)
    g = torch.Generator().manual_seed(96)
    W = [(w13q.to(dev), w13s.to(dev), w2q.to(dev), w2s.to(dev))]
    for _ in range(R - 1):                      # permute the experts: distinct bytes, same distribution
        p = torch.randperm(E, generator=g)
        W.append((w13q[p].to(dev), w13s[p].to(dev), w2q[p].to(dev), w2s[p].to(dev)))
    xd, ld = x.to(dev), logits.to(dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)

    aq = T <= 512              # the configuration quantises the activations; the 4096-token workload is w8a16 (the reference's mode)

    def launch(i):
        a, b, c, d = W[i % R]
        v.moe_forward_fp8_block(xd, ld, a, b, c, d, out, K, aq)

    e_cpu, t_cpu = 64, 256                        # CPU sample: half of the experts and of the tokens, 32 rows per expert as in the whole

    def cpu():
        tw, ti = O.moe_topk(logits[:t_cpu, :e_cpu], K)
        return O.moe_forward_grouped(x[:t_cpu], tw, ti, w13q[:e_cpu], w13s[:e_cpu], w2q[:e_cpu], w2s[:e_cpu], e_cpu,
                                     act_quant=True).to(torch.bfloat16)

    P = T * K
    # algorithmic bytes: every expert's weights + block scales once, x and logits in, output out
    alg_bytes = wbytes + 4 * E * ((2 * I // 128) * (H // 128) + (H // 128) * (I // 128)) + 2 * T * H + 2 * T * E + 2 * T * H
    flops = 2 * P * (2 * I * H + H * I)
    return dict(launch=launch, R=R, bytes=alg_bytes, flops=flops, bound="hbm" if T <= 512 else "mfma", dtype="fp8" if aq else "bf16",
                name=f"{'cfg3' if T == 512 else 'next:'} FP8 128x128-block MoE forward (topk+sort+quant+gate_up/SiLU+quant+down+combine) "
                     f"T={T} E={E} top{K} H={H} I={I} bf16, {'fp8 activations' if aq else '16-bit activations (w8a16)'}",
                kernel="moe_gemm_kernel", cpu=cpu, cpu_scale=e_cpu / E,
                cpu_what=f"{e_cpu} of the {E} experts and {t_cpu} of the {T} tokens (32 rows per expert, as in the whole)")


def wl_moe_gelu(dev):
    """Per-expert-scale FP8 MoE with the tanh-GELU gate at the shape of the reference's own test
    (vllm/custom-esimd-kernels-vllm/tests/test_moe_fp8_grouped.py:16): routing given, sort + grouped
    gate_up GEMM with the fused GELU * up + grouped down GEMM + weighted sum."""
    import custom_esimd_kernels_vllm  # noqa: F401  (registers torch.ops.moe_ops)
    from oracle import qlinear_oracle as O
    T, E, K, H, I = 256, 128, 8, 2816, 704
    g = torch.Generator(device=dev).manual_seed(97)
    x = (torch.randn(T, H, generator=g, device=dev) * 0.05).half()
    logits = torch.randn(T, E, generator=g, device=dev).half()
    tw, ti = torch.ops.moe_ops.moe_topk(logits, K, True)
    wbytes = E * 3 * H * I
    R = _copies(wbytes)
    W = []
    for _ in range(R):
        w13 = ((torch.randn(E, 2 * I, H, generator=g, device=dev) * 0.05).clamp(-0.3, 0.3) / 0.3).to(torch.float8_e4m3fn)
        w2 = ((torch.randn(E, H, I, generator=g, device=dev) * 0.05).clamp(-0.3, 0.3) / 0.3).to(torch.float8_e4m3fn)
        W.append((w13, w2))
    s13 = torch.full((E,), 0.3, device=dev)
    s2 = torch.full((E,), 0.3, device=dev)

    def launch(i):
        a, b = W[i % R]
        torch.ops.moe_ops.moe_forward_full_gelu_tanh_routed(x, tw, ti, a, s13, b, s2, K, E)

    n_cpu = 2                                    # tokens of the CPU sample

    def cpu():
        tic = ti.cpu()[:n_cpu]
        used = sorted(set(tic.reshape(-1).tolist()))
        remap = {e: i for i, e in enumerate(used)}
        ti_s = torch.tensor([[remap[int(e)] for e in row] for row in tic], dtype=torch.int32)
        a, b = W[0]
        sc = torch.full((len(used),), 0.3)
        return O.moe_prefill_scalar(x.cpu()[:n_cpu], tw.cpu()[:n_cpu], ti_s, a.view(torch.uint8)[used].cpu(), sc,
                                    b.view(torch.uint8)[used].cpu(), sc, act="gelu_tanh")

    P = T * K
    alg_bytes = wbytes + 8 * E + 2 * T * H + 6 * P + 2 * T * H
    flops = 2 * P * 3 * H * I
    return dict(launch=launch, R=R, bytes=alg_bytes, flops=flops, bound="hbm", dtype="fp16",
                name=f"next: per-expert-scale FP8 MoE, tanh-GELU gate (sort+gate_up/GELU+down+combine) "
                     f"T={T} E={E} top{K} H={H} I={I} fp16 (w8a16)",
                kernel="moe_gemm_kernel", cpu=cpu, cpu_scale=n_cpu / T)


def wl_moe_forward_full(dev):
    """Per-tensor FP8 MoE decode step at Qwen3-Next sizes: one token, 512 experts, top 10, one shared
    expert; routed weights K-major (moe_forward_full, vllm/custom-esimd-kernels-vllm/csrc/moe_batch/moe.sycl:1855).
    Each launch routes to ten other experts and another copy of the shared expert, so nothing is
    served from the Infinity Cache."""
    import custom_esimd_kernels_vllm  # noqa: F401
    from oracle import qlinear_oracle as O
    T, E, K, H, I = 1, 512, 10, 2048, 512
    g = torch.Generator(device=dev).manual_seed(98)
    f8 = lambda *shape: ((torch.randn(*shape, generator=g, device=dev)).clamp(-3, 3) * 100).to(torch.float8_e4m3fn)
    x = (torch.randn(T, H, generator=g, device=dev) * 0.3).half()
    w13, w2 = f8(E, H, 2 * I), f8(E, I, H)
    s13 = torch.full((E,), 2e-4, device=dev)
    s2 = torch.full((E,), 2e-4, device=dev)
    R = 96
    sw13 = [f8(1, 2 * I, H) for _ in range(R)]
    sw2 = [f8(1, H, I) for _ in range(R)]
    ss = torch.full((1,), 2e-4, device=dev)
    gate = (torch.randn(1, H, generator=g, device=dev) * 0.05).half()
    sets = E // K
    logits = []
    for i in range(sets):                            # launch i prefers experts [i*K, (i+1)*K)
        l = torch.randn(T, E, generator=g, device=dev) * 0.1
        l[:, i * K:(i + 1) * K] += 8.0
        logits.append(l.half())

    def launch(i):
        torch.ops.moe_ops.moe_forward_full(x, logits[i % sets], w13, s13, sw13[i % R], ss, w2, s2, sw2[i % R], ss, gate,
                                           K, 1, E)

    def cpu():
        u8 = lambda t: t.view(torch.uint8).cpu()
        return O.moe_forward_full_kmajor(x.cpu(), logits[0].cpu(), u8(w13), s13.cpu(), u8(sw13[0]), ss.cpu(), u8(w2),
                                         s2.cpu(), u8(sw2[0]), ss.cpu(), gate.cpu(), K)

    alg_bytes = (K + 1) * 3 * H * I + 2 * T * E + 4 * T * H
    flops = 2 * T * (K + 1) * 3 * H * I
    return dict(launch=launch, R=sets, bytes=alg_bytes, flops=flops, bound="hbm", dtype="fp16",
                name=f"next: per-tensor FP8 MoE decode step, K-major routed weights (topk+up+down+shared+finalize) "
                     f"T={T} E={E} top{K} H={H} I={I} fp16 (w8a16)",
                kernel="km_up_kernel", cpu=cpu)


def wl_moe_fp8_block_decode(dev, T=1):
    """The reference's fused small-batch MoE op for 128x128 block-FP8 weights (moe_forward_full_fp8_block,
    vllm/custom-esimd-kernels-vllm/csrc/moe_batch/moe.sycl:1707-1853; called per layer by the patched
    Qwen3-Next MoE block, vllm/patches/vllm_for_multi_arc.patch:9972-9989) at cfg3's layer shape: T tokens,
    128 experts, top 8, one shared expert.  Each launch prefers eight other experts and runs on another
    copy of the shared expert, so nothing is served from the Infinity Cache."""
    import custom_esimd_kernels_vllm  # noqa: F401
    from oracle import qlinear_oracle as O
    E, K, H, I = 128, 8, 2048, 768
    g = torch.Generator(device=dev).manual_seed(97)
    f8 = lambda *shape: ((torch.randn(*shape, generator=g, device=dev)).clamp(-3, 3) * 60).to(torch.float8_e4m3fn)
    x = (torch.randn(T, H, generator=g, device=dev) * 0.3).to(torch.bfloat16)
    w13, w2 = f8(E, 2 * I, H), f8(E, H, I)
    s13 = torch.rand(E, 2 * I // 128, H // 128, generator=g, device=dev) * 2e-4 + 1e-4
    s2 = torch.rand(E, H // 128, I // 128, generator=g, device=dev) * 2e-4 + 1e-4
    R = 64
    sw13 = [f8(2 * I, H) for _ in range(R)]
    sw2 = [f8(H, I) for _ in range(R)]
    ss13 = torch.full((2 * I // 128, H // 128), 2e-4, device=dev)
    ss2 = torch.full((H // 128, I // 128), 2e-4, device=dev)
    gate = (torch.randn(1, H, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    sets = E // K
    logits = []
    for i in range(sets):                            # launch i prefers experts [i*K, (i+1)*K)
        l = torch.randn(T, E, generator=g, device=dev) * 0.1
        l[:, i * K:(i + 1) * K] += 8.0
        logits.append(l.to(torch.bfloat16))
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)

    def launch(i):
        torch.ops.moe_ops.moe_forward_full_fp8_block(x, logits[i % sets], out, w13, s13, sw13[i % R], ss13, w2, s2,
                                                     sw2[i % R], ss2, gate, K, 1, E)

    def cpu():
        u8 = lambda t: t.view(torch.uint8).cpu()
        return O.moe_forward_full(x.cpu(), logits[0].cpu(), u8(w13), s13.cpu(), u8(sw13[0]), ss13.cpu(), u8(w2),
                                  s2.cpu(), u8(sw2[0]), ss2.cpu(), gate.cpu(), K)

    alg_bytes = (K + 1) * 3 * H * I + 2 * T * E + 4 * T * H      # T = 1: every route is its own expert
    flops = 2 * T * (K + 1) * 3 * H * I
    return dict(launch=launch, R=sets, bytes=alg_bytes, flops=flops, bound="hbm", dtype="bf16",
                name=f"next: fused block-FP8 MoE decode op (topk + routed up/SiLU/down + shared expert + sum) "
                     f"T={T} E={E} top{K} H={H} I={I} bf16 (w8a16)",
                kernel="gemv_rows_kernel (routed)", cpu=cpu)


def wl_gemv_fp16(dev):
    """16-bit weight GEMV at the reference test's largest router shape (tests/test_gemv_fp16.py:62-71)."""
    import custom_esimd_kernels_vllm as v
    M, N, K = 8, 256, 2048
    g = torch.Generator().manual_seed(99)
    x = (torch.randn(M, K, generator=g) * 0.1).half()
    per = N * K * 2
    R = 320                                      # 335 MB of distinct weights: more than the Infinity Cache
    W = [(torch.randn(N, K, generator=g) * 0.05).half().to(dev) for _ in range(R)]
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)

    def launch(i):
        v.esimd_gemv_fp16(xd, W[i % R], out)

    def cpu():
        return (x.float() @ W[0].cpu().float().t()).half()

    return dict(launch=launch, R=R, bytes=per + 2 * M * K + 2 * M * N, flops=2 * M * N * K, bound="hbm", dtype="f16",
                name=f"next: 16-bit weight GEMV (router) M={M} K={K} N={N} fp16", kernel="gemv_w16_kernel", cpu=cpu)


def wl_int4_fused2(dev):
    """The two GDN input projections of a Qwen3-Next decode step in one launch, as the reference's caller
    issues them (vllm/patches/vllm_for_multi_arc.patch:4490-4524): in_proj_qkvz [12288, 2048] and
    in_proj_ba [64, 2048], W4A16 group 128, one token."""
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    K, N0, N1 = 2048, 12288, 64
    x, p0, s0, _ = O.make_int4_case(1, K, N0, seed=31)
    _, p1, s1, _ = O.make_int4_case(1, K, N1, seed=32)
    per = (N0 + N1) * (K // 2 + (K // 128) * 2)
    R = _copies(per)
    g = torch.Generator().manual_seed(97)
    W = []
    for _ in range(R):
        a, b = torch.randperm(N0, generator=g), torch.randperm(N1, generator=g)
        W.append((p0[a].to(dev), s0[a].to(dev), p1[b].to(dev), s1[b].to(dev)))
    xd = x.to(dev)
    o0 = torch.empty(1, N0, dtype=torch.float16, device=dev)
    o1 = torch.empty(1, N1, dtype=torch.float16, device=dev)

    def launch(i):
        a, b, c, d = W[i % R]
        v.esimd_gemv_int4_fused2(xd, a, b, o0, c, d, o1)

    def cpu():
        return O.matmul_ref(x, O.int4_dequant(p0, s0)).half(), O.matmul_ref(x, O.int4_dequant(p1, s1)).half()

    return dict(launch=launch, R=R, bytes=per + 2 * K + 2 * (N0 + N1), flops=2 * (N0 + N1) * K, bound="hbm", dtype="f16",
                name=f"next: W4A16 fused2 GEMV (GDN in_proj_qkvz + in_proj_ba) M=1 K={K} N={N0}+{N1} fp16",
                kernel="gemv_rows_kernel", cpu=cpu)


def wl_fp8_pert_fused(dev, three: bool):
    """Per-tensor FP8 projections sharing one activation row in one launch: fused2 = the GDN in_proj_qkvz +
    in_proj_ba pair the reference's caller issues (vllm/patches/vllm_for_multi_arc.patch:4340-4355,
    10521-10529); fused3 = the q / k / v projections of a Qwen3-Next full-attention layer (gated q:
    16 heads x 256 x 2; 2 kv heads x 256)."""
    import custom_esimd_kernels_vllm as v
    from oracle import qlinear_oracle as O
    K = 2048
    Ns = [8192, 512, 512] if three else [12288, 64]
    g = torch.Generator().manual_seed(96)
    x = torch.randn(1, K, generator=g).half()
    w8 = [O.e4m3_quantize(torch.randn(n, K, generator=g).clamp(-3, 3) * (448.0 / 3)) for n in Ns]
    sc = [torch.tensor([0.02 / 448 * (i + 1)], dtype=torch.float32) for i in range(len(Ns))]
    per = sum(Ns) * K
    R = _copies(per)
    W = []
    for _ in range(R):
        W.append([w[torch.randperm(w.shape[0], generator=g)].to(dev).view(torch.float8_e4m3fn) for w in w8])
    xd = x.to(dev)
    sd = [t.to(dev) for t in sc]
    outs = [torch.empty(1, n, dtype=torch.float16, device=dev) for n in Ns]

    def launch(i):
        w = W[i % R]
        if three:
            v.esimd_gemv_fp8_pert_fused3(xd, w[0], sd[0], outs[0], w[1], sd[1], outs[1], w[2], sd[2], outs[2])
        else:
            v.esimd_gemv_fp8_pert_fused2(xd, w[0], sd[0], outs[0], w[1], sd[1], outs[1])

    def cpu():
        return [O.matmul_ref(x, O.fp8_dequant_per_tensor(w, t)).half() for w, t in zip(w8, sc)]

    n = "+".join(str(t) for t in Ns)
    return dict(launch=launch, R=R, bytes=per + 2 * K + 2 * sum(Ns) + 4 * len(Ns), flops=2 * sum(Ns) * K, bound="hbm",
                dtype="f16", name=f"next: FP8 per-tensor fused{len(Ns)} GEMV M=1 K={K} N={n} fp16",
                kernel="gemv_rows_kernel", cpu=cpu)


WORKLOADS = {
    "cfg1_m1": lambda dev: wl_fp8_pern(1, dev),
    "cfg1_m8": lambda dev: wl_fp8_pern(8, dev),
    "cfg1_m32": lambda dev: wl_fp8_pern(32, dev),
    "cfg0": wl_int4_gemv,
    "copy": wl_copy,
    "cfg2": wl_gemm_w4a16,
    "cfg3": wl_moe,
    "cfg4_m1": lambda dev: wl_q4k(1, dev),
    "cfg4_m64": lambda dev: wl_q4k(64, dev),
    "next_moe_prefill_t4096": lambda dev: wl_moe(dev, 4096),
    "next_fp8_prefill_m2048": wl_fp8_prefill,
    "next_fp8_block_prefill_m2048": lambda dev: wl_fp8_prefill(dev, "block"),
    "next_q4k_prefill_m2048": wl_q4k_prefill,
    "next_int4_fused2": wl_int4_fused2,
    "next_fp8_pert_fused2": lambda dev: wl_fp8_pert_fused(dev, False),
    "next_fp8_pert_fused3": lambda dev: wl_fp8_pert_fused(dev, True),
    "next_int4_m8": lambda dev: wl_int4_gemv(dev, 8, 14336),
    "next_int4_m32": lambda dev: wl_int4_gemv(dev, 32, 14336),
    "next_q4k_m8": lambda dev: wl_q4k(8, dev),
    "next_q4k_m32": lambda dev: wl_q4k(32, dev),
    "next_q4_0_m1": lambda dev: wl_gguf("q4_0", 1, dev),
    "next_q8_0_m1": lambda dev: wl_gguf("q8_0", 1, dev),
    "next_q5_k_m1": lambda dev: wl_gguf("q5_k", 1, dev),
    "next_q6_k_m1": lambda dev: wl_gguf("q6_k", 1, dev),
    "next_q4_0_quantize": wl_q4_0_quantize,
    "next_resadd_norm_gemv": wl_resadd_norm_gemv,
    "next_moe_gelu_grouped": wl_moe_gelu,
    "next_moe_forward_full_t1": wl_moe_forward_full,
    "next_moe_fp8_block_decode_t1": wl_moe_fp8_block_decode,
    "next_gemv_fp16_router": wl_gemv_fp16,
    "next_moe_gguf_t1": wl_moe_gguf,
    "next_moe_gguf_grouped_t2048": wl_moe_gguf_grouped,
    "next_moe_gguf_grouped_t512": lambda dev: wl_moe_gguf_grouped(dev, 512),
    "next_moe_gguf_grouped_t16": lambda dev: wl_moe_gguf_grouped(dev, 16),
}
HEADLINE = "cfg1_m1"
# the other benchmark configurations: reported as `cases` of the default run
BASELINE_CASES = ["cfg0", "cfg1_m8", "cfg1_m32", "cfg2", "cfg3", "cfg4_m1", "cfg4_m64"]
CASE_MIN_STEPS = 200             # a case is timed over at least this many launches


# ----------------------------------------------------------------------------
def run_gpu(wl, steps: int, warmup: int):
    """Times exactly `steps` launches, every one a node of a replayed HIP graph.
    -> (wall seconds for the timed region, event ms for the same region)"""
    R = wl["R"]
    launch = wl["launch"]
    G = min(steps, max(R, 128))                 # launches per graph
    reps, rem = divmod(steps, G)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(max(warmup, 1)):
            launch(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(G):
                launch(i)
        tail = None
        if rem:
            tail = torch.cuda.CUDAGraph()
            with torch.cuda.graph(tail, stream=stream):
                for i in range(rem):
                    launch(G + i)
        graph.replay()                      # untimed replays: graph upload
        if tail is not None:
            tail.replay()
        stream.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(reps):
            graph.replay()
        if tail is not None:
            tail.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    return t1 - t0, e0.elapsed_time(e1)


def floor_us(nbytes: int, dev, steps: int = CASE_MIN_STEPS):
    """Microseconds a pure streaming read of `nbytes` takes on this device (the library's read yardstick over
    cold memory: consecutive launches walk a buffer of at least 1 GiB), timed like a workload."""
    from mi355x_qlinear import capi
    import ctypes
    nbytes = (int(nbytes) + 15) // 16 * 16
    slices = max(2, -(-CACHE_BUST_BYTES // nbytes))
    buf = torch.empty(slices * nbytes, dtype=torch.uint8, device=dev).fill_(3)
    words = ctypes.c_longlong(0)
    if capi.lib().mi_stream_read_sink_words(ctypes.byref(words)) != 0:
        return None
    sink = torch.zeros(words.value, dtype=torch.int32, device=dev)
    base = buf.data_ptr()

    best = None
    for variant in range(capi.lib().mi_stream_read_variants()):     # launch shapes; which is fastest depends on the size
        def launch(i, variant=variant):
            capi.call("mi_stream_read", buf, base + (i % slices) * nbytes, nbytes, capi.ptr(sink), variant)

        _, ev = run_gpu(dict(launch=launch, R=slices), steps, 3)
        best = ev if best is None else min(best, ev)
    del buf
    return best * 1e3 / steps


def measured_traffic(workload_id):
    """(HBM bytes per launch, commit of the kernels they were measured on) from the committed rocprofv3
    --pmc summary, or (None, None).  The counters need a profiler run of their own, so the figure is a
    record, not a measurement of this run: the commit says which kernels it belongs to."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            d = json.load(f)
        e = d.get(workload_id, {})
        return e.get("bytes"), e.get("commit", d.get("commit"))
    except (OSError, ValueError):
        return None, None


def summarize(wl, wid, steps, warmup, wall_s, ev_ms):
    per_launch_s = ev_ms * 1e-3 / steps
    if wl["bound"] == "hbm":
        achieved = wl["bytes"] / per_launch_s / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = wl["flops"] / per_launch_s / 1e12
        peak, unit = MFMA_PEAK_TFLOPS[wl["dtype"]], "TFLOP/s"
    traffic, traffic_commit = measured_traffic(wid)
    return {
        "id": wid,
        "workload": wl["name"],
        "dtype": wl["dtype"],
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": wall_s * 1e3 / steps,
        "us_per_launch_events": per_launch_s * 1e6,
        "GBps": wl["bytes"] / per_launch_s / 1e9,
        "TFLOPs": wl["flops"] / per_launch_s / 1e12,
        "roofline": {"bound": wl["bound"], "achieved": achieved, "peak": peak, "unit": unit,
                     "frac": achieved / peak, "traffic": traffic, "traffic_measured_at_commit": traffic_commit,
                     "launches_timed": steps, "kernel": wl["kernel"],
                     "alg_bytes_per_launch": wl["bytes"], "alg_flops_per_launch": wl["flops"]},
    }


def cpu_baseline(wl, budget_s: float = 20.0):
    """The oracle's torch dequant + fp32 matmul on this host's cores, on a bounded sample."""
    host = os.cpu_count() or 1
    # the GPU box exports OMP_NUM_THREADS = its CPU share for one GPU; never more threads than that
    torch.set_num_threads(min(host, int(os.environ.get("OMP_NUM_THREADS", "16"))))
    cores = torch.get_num_threads()
    times = []
    t_start = time.perf_counter()
    n = 0
    while True:
        t0 = time.perf_counter()
        if wl["cpu"]() is None:                     # this workload has no CPU leg
            return None
        dt = time.perf_counter() - t0
        n += 1
        if n > 2:
            times.append(dt)
        if (n >= 7 or time.perf_counter() - t_start > budget_s) and times:
            break
    times.sort()
    med = times[len(times) // 2]
    frac = wl.get("cpu_scale", 1.0)                 # share of the workload one CPU pass covers
    if wl["bound"] == "hbm":
        value, unit = wl["bytes"] * frac / med / 1e9, "GB/s"
    else:
        value, unit = wl["flops"] * frac / med / 1e12, "TFLOP/s"
    what = "the full workload" if frac == 1.0 else wl.get("cpu_what", f"{frac:.3f} of the workload")
    return {"value": value, "unit": unit, "cores": cores, "host_cpu_count": host, "kind": "port",
            "seconds_per_pass": med,
            "sample": f"{len(times)} timed passes (after 2 warm-ups) over {what}: torch dequant of the "
                      f"sampled weight + fp32 matmul, {wl['name']}"}


def run_case(wid, dev, steps, warmup, with_cpu, cpu_budget_s):
    wl = WORKLOADS[wid](dev)
    wall, ev = run_gpu(wl, steps, warmup)
    c = summarize(wl, wid, steps, warmup, wall, ev)
    if steps < CASE_MIN_STEPS:
        # `ms_per_step` stays the wall clock over exactly `steps` launches; the per-launch average behind
        # `roofline` comes from a second, longer series, like every other case (a handful of launches
        # still carries the first ones' cold instruction cache and clock ramp)
        _, ev2 = run_gpu(wl, CASE_MIN_STEPS, 3)
        long_run = summarize(wl, wid, CASE_MIN_STEPS, 3, wall, ev2)
        for key in ("roofline", "us_per_launch_events", "GBps", "TFLOPs"):
            c[key] = long_run[key]
    if wl["bound"] == "hbm":
        # the same number of bytes through a pure streaming read: what is left of the gap to the HBM peak once
        # the device's own read ceiling and the fixed cost of a launch are taken out
        f = floor_us(wl["bytes"], dev)
        if f:
            c["roofline"]["floor_us"] = f
            c["roofline"]["frac_of_floor"] = f / c["us_per_launch_events"]
    c["cpu_baseline"] = cpu_baseline(wl, cpu_budget_s) if with_cpu else None
    del wl
    torch.cuda.empty_cache()
    return c


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--only", action="store_true", help="time --workload alone (no `cases`)")
    ap.add_argument("--all", action="store_true", help="also time the workloads beyond the benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the path has no multi-GPU leg "
              f"(asked for --gpus {args.gpus}).", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import mi355x_qlinear  # noqa: F401  (raises if the HIP library is not built)
    dev = torch.device("cuda:0")

    head = run_case(args.workload, dev, args.steps, args.warmup, not args.no_cpu, 10.0)

    cases = []
    if not args.only:
        ids = [w for w in BASELINE_CASES if w != args.workload]
        if args.workload != HEADLINE:
            ids.insert(0, HEADLINE)
        if args.all:
            ids += [w for w in sorted(WORKLOADS) if w not in ids and w != args.workload and w != "copy"]
        for wid in ids:
            cases.append(run_case(wid, dev, max(args.steps, CASE_MIN_STEPS), max(args.warmup, 20),
                                  not args.no_cpu and wid in BASELINE_CASES + [HEADLINE], 5.0))

    line = {
        "metric": "HBM GB/s (GEMV) and TFLOP/s (GEMM) as % of MI355X roofline, 1 GPU",
        "value": wl_value(head),
        "unit": head["roofline"]["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic (seeded; weights rotate over >=1 GiB of distinct copies)",
        "config": {"workload": head["workload"], "id": args.workload,
                   "timing": "exactly `steps` launches, all HIP-graph nodes replayed back to back on one stream"},
        "roofline": head["roofline"],
        "cpu_baseline": head["cpu_baseline"],
    }
    if cases:
        line["cases"] = cases
    print(json.dumps(line))


def wl_value(head):
    """Whole-job throughput over the wall-clock timed region."""
    r = head["roofline"]
    per_step_s = head["ms_per_step"] * 1e-3
    if r["bound"] == "hbm":
        return r["alg_bytes_per_launch"] / per_step_s / 1e9
    return r["alg_flops_per_launch"] / per_step_s / 1e12


if __name__ == "__main__":
    main()
