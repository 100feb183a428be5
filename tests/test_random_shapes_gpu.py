"""GPU parity on seeded random shapes: every combination of head width, storage type, odd sample counts,
non-square images and out-of-image coordinates that a fixed list of cases would miss. Same error measure and
bars as tests/test_parity_gpu.py (rel = max|x - ref| / max|ref|; 1e-4 fp32 forward, 1e-3 fp32 gradients,
2e-2 for 16-bit storage), forward and backward through the operator, against the CPU oracle."""
import random
import sys

import numpy as np
import pytest
import torch

from oracle import oracle_bwd, oracle_fwd
from ops.triton import deform_sdpa_triton

pytestmark = pytest.mark.gpu

TOL_FWD = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}
TOL_BWD = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def rel(a, b):
    a = a.detach().double().cpu().numpy()
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def draw_cases(n, seed):
    rng = random.Random(seed)
    cases = []
    for i in range(n):
        D = rng.choice([16, 32, 64, 128, 256])
        Himg, Wimg = rng.randint(1, 13), rng.randint(1, 13)
        cases.append(dict(
            seed=1000 + i, B=rng.randint(1, 2), V=rng.randint(1, 4), H=rng.randint(1, 3), Himg=Himg, Wimg=Wimg, D=D,
            P=rng.choice([1, 2, 3, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 47, 64, 70]),
            lo=rng.choice([0.0, -0.2, -0.6]), hi=rng.choice([1.0, 1.2, 1.6]),
            dtype=rng.choice([torch.float32, torch.float32, torch.bfloat16, torch.float16]),
            scale=rng.choice([0.1, 0.3, 1.0 / D ** 0.5])))
    return cases


CASES = draw_cases(40, seed=2024)


@pytest.mark.parametrize("case", CASES, ids=[f"r{c['seed']}" for c in CASES])
def test_random_shape(case):
    c = case
    print("[case] random shape", {k: (str(v) if k == "dtype" else v) for k, v in c.items()}, flush=True)
    sys.stdout.flush()
    g = torch.Generator().manual_seed(c["seed"])
    L = c["Himg"] * c["Wimg"]
    q, k, v, do = (torch.randn(c["B"], c["V"], c["H"], L, c["D"], generator=g).to(c["dtype"]) for _ in range(4))
    coords = torch.rand(c["B"], c["V"], L, c["V"], c["P"], 2, generator=g) * (c["hi"] - c["lo"]) + c["lo"]
    f = lambda t: t.float().numpy()
    out_r, _ = oracle_fwd(f(q), f(k), f(v), f(coords), c["Wimg"], c["Himg"], c["scale"])
    dq_r, dk_r, dv_r = oracle_bwd(f(q), f(k), f(v), f(coords), f(do), c["Wimg"], c["Himg"], c["scale"])
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = deform_sdpa_triton(qg, kg, vg, coords.cuda(), c["Wimg"], c["Himg"], c["scale"])
    out.backward(do.cuda())
    torch.cuda.synchronize()
    assert rel(out, out_r) < TOL_FWD[c["dtype"]]
    assert rel(vg.grad, dv_r) < TOL_BWD[c["dtype"]]
    if c["V"] * c["P"] == 1:
        # one sample per row: its probability is 1 whatever the logit, so dq and dk are exactly zero and a
        # relative measure has no scale; the kernels leave rounding noise of dout.v~ - dout.out there
        noise = 1e-5 if c["dtype"] == torch.float32 else 2e-2
        assert np.abs(dq_r).max() < 1e-6 and np.abs(dk_r).max() < 1e-6
        assert qg.grad.abs().max().item() < noise and kg.grad.abs().max().item() < noise
    else:
        assert rel(qg.grad, dq_r) < TOL_BWD[c["dtype"]]
        assert rel(kg.grad, dk_r) < TOL_BWD[c["dtype"]]
