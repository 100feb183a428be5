"""Deterministic backward (torch.use_deterministic_algorithms / DSDPA_FLAG_DETERMINISTIC): parity with the
oracle at the usual bars and bitwise identical gradients from run to run.

The reference has no such switch: its backward adds into dk/dv with float atomics (ops/triton.py:345-360).
"""
import sys

import numpy as np
import pytest
import torch

from oracle import oracle_bwd
from ops.triton import deform_sdpa_triton
from workloads import WORKLOADS, gen_inputs
from parity_util import oracle_on_slices, slice_bh

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def rel(a, b):
    a = a.detach().double().cpu().numpy()
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture
def deterministic():
    prev = torch.are_deterministic_algorithms_enabled()
    torch.use_deterministic_algorithms(True)
    yield
    torch.use_deterministic_algorithms(prev)


def grads(q, k, v, c, do, W, Himg, scale):
    qg, kg, vg = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    deform_sdpa_triton(qg, kg, vg, c, W, Himg, scale).backward(do)
    torch.cuda.synchronize()
    return qg.grad, kg.grad, vg.grad


CASES = [
    # seed B V H Himg Wimg D   P   lo     hi
    (41, 1, 2, 2, 3, 5, 16, 3, -0.25, 1.25),
    (42, 2, 3, 2, 6, 4, 32, 23, -0.1, 1.1),
    (43, 1, 4, 3, 7, 9, 32, 32, 0.0, 1.0),
    (44, 1, 2, 2, 5, 6, 64, 17, -0.5, 1.5),
    (45, 1, 2, 1, 1, 1, 16, 1, 0.0, 1.0),        # 1x1 image: every colour pass but one is empty of pixels
    (46, 1, 3, 2, 1, 11, 128, 5, -0.2, 1.2),
    (47, 1, 2, 1, 40, 40, 16, 4, 0.45, 0.55),    # clustered: a few very long cell lists
    (48, 1, 2, 2, 20, 20, 64, 16, -0.1, 1.1),    # fp32: dq by the slab kernel (no pairs handed over on this path)
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[f"d{c[0]}" for c in CASES])
def test_deterministic_backward_vs_oracle_and_bitwise_repeatable(case, dtype, deterministic):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    say(f"[case] deterministic seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v, do = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(4))
    c = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
    f = lambda t: t.float().numpy()
    ref = oracle_bwd(f(q), f(k), f(v), f(c), f(do), Wimg, Himg, 0.3)
    dev = [t.cuda() for t in (q, k, v, c, do)]
    first = grads(*dev, Wimg, Himg, 0.3)
    for got, want in zip(first, ref):
        assert rel(got, want) < TOL[dtype]
    for _ in range(3):
        again = grads(*dev, Wimg, Himg, 0.3)
        for a, b in zip(first, again):
            assert torch.equal(a, b)


def test_deterministic_backward_c2_bitwise_repeatable(deterministic):
    """Full-size C2 (5.97 M query*samples, 747 k list entries): five runs, identical bits; and the same
    values as the default backward to within the gradient bar."""
    wl = WORKLOADS["C2"]
    say("[case] deterministic C2")
    q, k, v, c, do = gen_inputs(wl, device="cuda:0")
    first = grads(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    for _ in range(4):
        again = grads(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale)
        for a, b in zip(first, again):
            assert torch.equal(a, b)
    torch.use_deterministic_algorithms(False)
    plain = grads(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    for a, b in zip(first, plain):
        assert rel(a, b.double().cpu().numpy()) < 1e-3


def test_deterministic_backward_c5_full_size(deterministic):
    """Full-size C5 (clustered coordinates: cell lists of up to several thousand samples, the case the list
    ordering exists for): the oracle's bars on two (batch, head) slices, and identical bits on a rerun."""
    wl = WORKLOADS["C5"]
    say("[case] deterministic C5")
    q, k, v, c, do = gen_inputs(wl)
    dev = [t.to("cuda:0") for t in (q, k, v, c, do)]
    first = grads(*dev, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    again = grads(*dev, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    for a, b in zip(first, again):
        assert torch.equal(a, b)
    slices = [(0, 1), (wl.B - 1, wl.H - 1)]
    ref = oracle_on_slices(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale, slices, forward=False)
    for (b, h), (_, rdq, rdk, rdv) in ref.items():
        for got, want in zip(first, (rdq, rdk, rdv)):
            assert rel(slice_bh(got, b, h), want) < TOL[torch.bfloat16], (b, h)


def test_deterministic_with_coords_gradient_is_refused(deterministic):
    say("[case] deterministic + coords grad")
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, 2, 2, 12, 16, generator=g).cuda().requires_grad_(True) for _ in range(3))
    c = torch.rand(1, 2, 12, 2, 3, 2, generator=g).cuda().requires_grad_(True)
    out = deform_sdpa_triton(q, k, v, c, 4, 3, 0.5, True)
    with pytest.raises(RuntimeError):
        out.sum().backward()
