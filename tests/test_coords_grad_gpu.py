"""GPU parity of the optional coordinate gradient (eighth operator argument) against the CPU oracle.

The reference's fused operator returns no gradient for coords (ops/triton.py:464); its eager operator gets
one by differentiating through grid_sample (ops/torch.py:14-15). The oracle's dcoords is pinned against that
library path in tests/test_oracle.py. Error measure and bars as for the other gradients:
rel = max|x - ref| / max|ref|, 1e-3 for fp32 storage, 2e-2 for bf16/fp16.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import oracle_bwd
from ops import _native
from ops.triton import deform_sdpa_triton
from workloads import WORKLOADS, gen_inputs

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def rel(a, b):
    a = a.detach().double().cpu().numpy() if torch.is_tensor(a) else np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


CASES = [
    # seed B V H Himg Wimg D   P   lo     hi
    (31, 1, 2, 2, 3, 5, 16, 3, -0.25, 1.25),
    (32, 2, 3, 2, 6, 4, 32, 23, -0.1, 1.1),
    (33, 1, 4, 3, 7, 9, 32, 32, 0.0, 1.0),
    (34, 1, 2, 2, 5, 6, 64, 17, -0.5, 1.5),
    (35, 2, 2, 1, 4, 7, 128, 40, 0.0, 1.0),
    (36, 1, 2, 1, 3, 3, 256, 9, -0.1, 1.1),
    (37, 1, 3, 2, 1, 11, 32, 5, -0.2, 1.2),      # single-row image: no y gradient
    (38, 1, 2, 1, 21, 22, 32, 4, -0.1, 1.1),     # fp32: the planes fit in LDS only without the gradient's block
    (39, 1, 2, 2, 20, 22, 64, 16, -0.15, 1.15),  # fp32: dq by the slab kernel, two samples per lane and view
    (40, 1, 2, 1, 19, 19, 64, 32, -0.1, 1.1),    # ... 32 samples per view: the two blocks of a row in one lane
    (41, 1, 2, 1, 24, 24, 64, 16, -0.1, 1.1),    # large enough for the slab kernels at 16-bit storage too
]


@pytest.mark.parametrize("path", ["auto", "gather"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{c[0]}" for c in CASES])
def test_coords_gradient_vs_oracle(case, dtype, path):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    say(f"[case] coords grad seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype} path={path}")
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v, do = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(4))
    c = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
    f = lambda t: t.float().numpy()
    dq_r, dk_r, dv_r, dc_r = oracle_bwd(f(q), f(k), f(v), f(c), f(do), Wimg, Himg, 0.3, with_coords=True)
    dev = "cuda:0"
    qg, kg, vg, cg = (t.to(dev).requires_grad_(True) for t in (q, k, v, c))
    prev = _native.set_path({"auto": _native.PATH_AUTO, "gather": _native.PATH_GATHER}[path])
    try:
        out = deform_sdpa_triton(qg, kg, vg, cg, Wimg, Himg, 0.3, True)
        out.backward(do.to(dev))
        torch.cuda.synchronize()
    finally:
        _native.set_path(prev)
    assert cg.grad is not None and cg.grad.shape == c.shape and cg.grad.dtype == torch.float32
    assert rel(cg.grad, dc_r) < TOL[dtype]
    assert rel(qg.grad, dq_r) < TOL[dtype]
    assert rel(kg.grad, dk_r) < TOL[dtype]
    assert rel(vg.grad, dv_r) < TOL[dtype]


def test_default_call_keeps_the_reference_contract():
    """Seven arguments: coords gets no gradient even when it requires one (ops/triton.py:464);
    eight with False: the same."""
    say("[case] coords grad off")
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 2, 2, 12, 16, generator=g).cuda().requires_grad_(True) for _ in range(3))
    c = torch.rand(1, 2, 12, 2, 3, 2, generator=g).cuda().requires_grad_(True)
    for extra in ((), (False,)):
        c.grad = None
        deform_sdpa_triton(q, k, v, c, 4, 3, 0.5, *extra).sum().backward()
        torch.cuda.synchronize()
        assert c.grad is None and q.grad is not None


def test_coords_gradient_skipped_when_coords_do_not_require_grad():
    say("[case] coords grad requested, coords without requires_grad")
    g = torch.Generator().manual_seed(6)
    q, k, v = (torch.randn(1, 2, 2, 12, 16, generator=g).cuda().requires_grad_(True) for _ in range(3))
    c = torch.rand(1, 2, 12, 2, 3, 2, generator=g).cuda()
    deform_sdpa_triton(q, k, v, c, 4, 3, 0.5, True).sum().backward()
    torch.cuda.synchronize()
    assert c.grad is None and q.grad is not None


@pytest.mark.parametrize("name,batch", [("C2", 0), ("C2", 1), ("C3", 0), ("C4", 1), ("C5", 1)],
                         ids=["C2-b0", "C2-b1", "C3-b0", "C4-b1", "C5-b1"])
def test_coords_gradient_named_workloads(name, batch):
    """Full-size workload; the oracle runs on one batch item (all its heads: the gradient sums over them),
    the first or the last one."""
    wl = WORKLOADS[name]
    say(f"[case] coords grad workload {name} batch item {batch}")
    q, k, v, c, do = gen_inputs(wl)
    dev = "cuda:0"
    qg, kg, vg, cg = (t.to(dev).requires_grad_(True) for t in (q, k, v, c))
    out = deform_sdpa_triton(qg, kg, vg, cg, wl.W_IMG, wl.H_IMG, wl.sm_scale, True)
    out.backward(do.to(dev))
    torch.cuda.synchronize()
    f = lambda t: t[batch:batch + 1].float().numpy()
    *_, dc_r = oracle_bwd(f(q), f(k), f(v), f(c), f(do), wl.W_IMG, wl.H_IMG, wl.sm_scale, with_coords=True)
    assert rel(cg.grad[batch:batch + 1], dc_r) < TOL[wl.torch_dtype()]
    # the whole tensor: finite, and zero exactly where a sample has no tap inside the image
    assert torch.isfinite(cg.grad).all()
    if wl.coords == "border":
        x, y = c[..., 0] * (wl.W_IMG - 1), c[..., 1] * (wl.H_IMG - 1)
        far = (x < -1) | (x > wl.W_IMG) | (y < -1) | (y > wl.H_IMG)
        assert far.any()
        assert (cg.grad.cpu()[far] == 0).all()


def test_dcoords_without_the_workspace_flag_matches_with_it():
    """C ABI: dcoords given but DSDPA_FLAG_COORDS_GRAD not set (workspace sized without it): the gather dq kernel
    computes the gradient; with the flag the staged kernel does. Same numbers to float-atomic noise."""
    say("[case] coords grad through the C ABI, with and without the workspace flag")
    lib = _native.load()
    g = torch.Generator().manual_seed(41)
    B, V, H, Himg, Wimg, D, P = 1, 3, 2, 6, 7, 32, 11
    L = Himg * Wimg
    q, k, v, do = (torch.randn(B, V, H, L, D, generator=g).cuda() for _ in range(4))
    c = (torch.rand(B, V, L, V, P, 2, generator=g) * 1.2 - 0.1).cuda()
    out, lse = torch.empty_like(q), torch.empty(B, V, H, L, device="cuda")
    fws = torch.empty(max(lib.dsdpa_fwd_workspace_bytes(0, B, V, H, Himg, Wimg, D, P), 1), dtype=torch.uint8,
                      device="cuda")
    _native.check(lib.dsdpa_fwd_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out.data_ptr(),
                                    lse.data_ptr(), fws.data_ptr(), B, V, H, Himg, Wimg, D, P, 0.3, None, None))
    res = {}
    for flags in (0, _native.FLAG_COORDS_GRAD):
        nbytes = lib.dsdpa_bwd_workspace_bytes(0, B, V, H, Himg, Wimg, D, P, flags)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        dq, dk, dv, dc = (torch.full_like(t, float("nan")) for t in (q, k, v, c))
        _native.check(lib.dsdpa_bwd_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out.data_ptr(),
                                        lse.data_ptr(), do.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                        dc.data_ptr(), ws.data_ptr(), B, V, H, Himg, Wimg, D, P, 0.3, None, flags, None))
        torch.cuda.synchronize()
        res[flags] = (nbytes, dq.cpu(), dc.cpu())
    assert res[_native.FLAG_COORDS_GRAD][0] > res[0][0]
    assert rel(res[0][1], res[_native.FLAG_COORDS_GRAD][1].numpy()) < 1e-5
    assert rel(res[0][2], res[_native.FLAG_COORDS_GRAD][2].numpy()) < 1e-5
