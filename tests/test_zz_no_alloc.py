"""The entry point that allocates nothing, mi_norm_gemv_static, against mi_norm_gemv_scaled.

Both are called through the C ABI (ctypes) on the same inputs; outputs, the in-place
residual and the normalised row must be bit-identical (same kernel, only the arrival
counters live elsewhere).  Two calls in a row share the static counters, the second on
a smaller problem; then sizes beyond the fused launch's limit must be refused.
"""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


def _case(K, Ns, seed, dev, dt=torch.float16):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(1, K, generator=g).to(dt)
    residual = torch.randn(1, K, generator=g).to(dt)
    nw = (torch.randn(K, generator=g) * 0.1 + 1.0).to(dt)
    ws = [O.e4m3_quantize((torch.randn(N, K, generator=g) * 60).clamp(-448, 448)) for N in Ns]
    scs = [torch.tensor([2.0e-3 * (i + 1)]) for i in range(len(Ns))]
    return hidden, residual, nw, ws, scs


def _run(entry, dev, hidden, residual, nw, ws, scs, eps=1e-6, rscale=1.0):
    from mi355x_qlinear import capi
    dt = hidden.dtype
    K = hidden.shape[1]
    x = hidden.to(dev)
    res = residual.to(dev).clone()
    nwd = nw.to(dev)
    wd = [w.view(torch.float8_e4m3fn).to(dev) for w in ws]
    sd = [s.to(dev) for s in scs]
    outs = [torch.full((1, w.shape[0]), float("nan"), dtype=dt, device=dev) for w in ws]
    normed = torch.full((1, K), float("nan"), dtype=dt, device=dev)
    capi.call(entry, x, capi.ptr(x), capi.ptr(res), None, capi.ptr(nwd), capi.ptr(normed), K, float(eps), float(rscale),
              0, len(ws), capi.ptr_array(wd), capi.ptr_array(sd), capi.ptr_array(outs),
              capi.int_array([w.shape[0] for w in ws]), K, capi.act_dtype(x))
    torch.cuda.synchronize()
    return [o.cpu() for o in outs], res.cpu(), normed.cpu()


def _bits(t):
    return t.view(torch.int16)


def test_static_entry_matches_allocating_entry(dev):
    from mi355x_qlinear import capi
    assert capi.lib().mi_static_scratch_setup() == 0
    # first call: a full grid (more workgroups than CUs); second call: a smaller row and fewer rows,
    # run right after it on the counters the first call left behind; third: bf16, two matrices
    for K, Ns, seed, dt, rscale in ((4096, [14336], 1, torch.float16, 1.0), (512, [200], 2, torch.float16, 1.0),
                                    (2048, [96, 640], 3, torch.bfloat16, 0.5)):
        case = _case(K, Ns, seed, dev, dt)
        want = _run("mi_norm_gemv_scaled", dev, *case, rscale=rscale)
        got = _run("mi_norm_gemv_static", dev, *case, rscale=rscale)
        for a, b in zip(got[0], want[0]):
            assert torch.equal(_bits(a), _bits(b)), f"K={K} Ns={Ns}: outputs differ"
        assert torch.equal(_bits(got[1]), _bits(want[1])), f"K={K}: residual differs"
        assert torch.equal(_bits(got[2]), _bits(want[2])), f"K={K}: normalised row differs"
        # and against the oracle: exact residual, GEMV within 1e-2 on the op's own normalised row
        hidden, residual, nw, ws, scs = case
        _, res_ref = O.rmsnorm(hidden, nw, 1e-6, residual=residual) if rscale == 1.0 else (None, None)
        if res_ref is not None:
            assert torch.equal(_bits(got[1]), _bits(res_ref))
        for o, w, s in zip(got[0], ws, scs):
            ref = O.matmul_ref(got[2], O.fp8_dequant_per_tensor(w, s))
            assert O.max_rel_err(o, ref) < 1e-2


def test_static_entry_refuses_rows_beyond_its_limit(dev):
    from mi355x_qlinear import capi
    K = 20480                                           # the allocating entry takes the two-kernel route here
    case = _case(K, [64], 4, dev)
    want = _run("mi_norm_gemv_scaled", dev, *case)
    assert torch.isfinite(want[0][0].float()).all()
    with pytest.raises(RuntimeError, match="fixed capacity"):
        _run("mi_norm_gemv_static", dev, *case)


def test_static_entry_refuses_a_second_stream(dev):
    """All calls on one GPU share the static counters, so calls that overlap on two streams would
    race.  The first call after a set-up claims the array for its stream; a call on another stream
    is refused (nothing launched, outputs untouched) until the set-up releases the claim."""
    from mi355x_qlinear import capi
    assert capi.lib().mi_static_scratch_setup() == 0
    case = _case(1024, [136], 5, dev)
    want = _run("mi_norm_gemv_scaled", dev, *case)
    side = torch.cuda.Stream()
    got = _run("mi_norm_gemv_static", dev, *case)              # claims the array for the current stream
    assert torch.equal(_bits(got[0][0]), _bits(want[0][0]))
    with torch.cuda.stream(side):
        with pytest.raises(RuntimeError, match="claimed by another stream"):
            _run("mi_norm_gemv_static", dev, *case)
    again = _run("mi_norm_gemv_static", dev, *case)            # the owner keeps working
    assert torch.equal(_bits(again[0][0]), _bits(want[0][0]))
    torch.cuda.synchronize()
    assert capi.lib().mi_static_scratch_setup() == 0           # hand-over: nothing in flight
    with torch.cuda.stream(side):
        moved = _run("mi_norm_gemv_static", dev, *case)
    assert torch.equal(_bits(moved[0][0]), _bits(want[0][0]))
    assert torch.equal(_bits(moved[1]), _bits(want[1])) and torch.equal(_bits(moved[2]), _bits(want[2]))
    torch.cuda.synchronize()
    assert capi.lib().mi_static_scratch_setup() == 0           # leave it unclaimed for whoever comes next
