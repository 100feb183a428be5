"""GPU tests of the sweep harness, non-default streams and small sample counts."""
import math
import os
import sys

import numpy as np
import pytest
import torch

from oracle import oracle_bwd, oracle_fwd
from ops.triton import deform_sdpa_triton

pytestmark = pytest.mark.gpu


def rel(a, b):
    a = a.detach().double().cpu().numpy()
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def test_sweep_harness_check_lines(tmp_path, capsys):
    """The S x P sweep (the reference's benchmark.py:30-100 loop) on a tiny grid: every [Check] must be ok."""
    print("[case] sweep harness", flush=True)
    import sweep
    rows = sweep.main(["--b", "1", "--h", "2", "--d", "32", "--iw", "6", "--quick", "--warmup", "1", "--rep", "2",
                       "--save-path", str(tmp_path)])
    out = capsys.readouterr().out
    checks = [l for l in out.splitlines() if l.startswith("[Check]")]
    assert len(checks) == 3
    for line in checks:
        assert "False" not in line, line
    assert len(rows) == 2 * 3 * 3 * 2
    assert all(ms > 0 for (_, _, _, _, ms, _) in rows)
    assert os.path.exists(os.path.join(str(tmp_path), "logs.txt"))
    # the per-line tables the reference's perf_report run leaves (benchmark.py:106)
    for mode in ("fwd", "bwd"):
        for P in (2, 6, 12):
            path = os.path.join(str(tmp_path), f"coord-attn-B1-H2-D32-{mode}-W6-P{P}.csv")
            lines = open(path).read().splitlines()
            assert lines[0].startswith("S_views,") and len(lines) == 1 + 3
            assert all(float(x) > 0 for l in lines[1:] for x in l.split(","))


@pytest.mark.parametrize("P", [1, 2, 5, 12, 33, 64, 100])
def test_sample_counts(P):
    """P from 1 (fewer samples than slots) over 33 (ragged pair/chunk edges) to 100 (two 64-sample chunks)."""
    print(f"[case] sample count P={P}", flush=True)
    g = torch.Generator().manual_seed(100 + P)
    B, V, H, Himg, Wimg, D = 1, 3, 2, 5, 4, 32
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g) for _ in range(3))
    c = torch.rand(B, V, L, V, P, 2, generator=g) * 1.2 - 0.1
    do = torch.randn(B, V, H, L, D, generator=g)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = deform_sdpa_triton(qg, kg, vg, c.cuda(), Wimg, Himg, 0.2)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    ro, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), Wimg, Himg, 0.2)
    rdq, rdk, rdv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.2)
    assert rel(out, ro) < 1e-4
    assert rel(qg.grad, rdq) < 1e-3 and rel(kg.grad, rdk) < 1e-3 and rel(vg.grad, rdv) < 1e-3


def test_non_default_stream_and_back_to_back_calls():
    """Work is enqueued on torch's current stream; two calls in a row share no hidden state."""
    print("[case] side stream", flush=True)
    g = torch.Generator().manual_seed(7)
    B, V, H, Himg, Wimg, D, P = 1, 2, 2, 6, 7, 64, 9
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g) for _ in range(3))
    c = torch.rand(B, V, L, V, P, 2, generator=g)
    do = torch.randn(B, V, H, L, D, generator=g)
    ro, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), Wimg, Himg, 0.125)
    rdq, rdk, rdv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.125)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        cg, dog = c.cuda(), do.cuda()
        for _ in range(2):
            qg.grad = kg.grad = vg.grad = None
            out = deform_sdpa_triton(qg, kg, vg, cg, Wimg, Himg, 0.125)
            out.backward(dog)
    side.synchronize()
    assert rel(out, ro) < 1e-4
    assert rel(qg.grad, rdq) < 1e-3 and rel(kg.grad, rdk) < 1e-3 and rel(vg.grad, rdv) < 1e-3


def test_large_image_uses_global_binning_path():
    """A 96x128 image with 2 views has too many cells for the LDS-aggregated binning (V*NC counters do not
    fit in LDS), so the backward takes the global-atomic counting passes; planes are too big for LDS too."""
    print("[case] large image, global binning", flush=True)
    g = torch.Generator().manual_seed(41)
    B, V, H, Himg, Wimg, D, P = 1, 2, 1, 96, 128, 16, 3
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g) for _ in range(3))
    c = torch.rand(B, V, L, V, P, 2, generator=g) * 1.06 - 0.03
    do = torch.randn(B, V, H, L, D, generator=g)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = deform_sdpa_triton(qg, kg, vg, c.cuda(), Wimg, Himg, 0.25)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    ro, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), Wimg, Himg, 0.25)
    rdq, rdk, rdv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.25)
    assert rel(out, ro) < 1e-4
    assert rel(qg.grad, rdq) < 1e-3 and rel(kg.grad, rdk) < 1e-3 and rel(vg.grad, rdv) < 1e-3
