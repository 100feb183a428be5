"""The package's eager operator (ops.torch.deform_sdpa_torch) against the C oracle, on CPU."""
import numpy as np
import pytest
import torch

from oracle import oracle_bwd, oracle_fwd
from ops.torch import deform_sdpa_torch


def rel(a, b):
    a = a.detach().double().numpy() if torch.is_tensor(a) else np.asarray(a, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


@pytest.mark.parametrize("case", [(0, 1, 2, 2, 3, 5, 16, 3, -0.25, 1.25), (1, 2, 3, 2, 6, 4, 32, 7, 0.0, 1.0)])
def test_eager_operator_matches_oracle(case):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).requires_grad_(True) for _ in range(3))
    c = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
    do = torch.randn(B, V, H, L, D, generator=g)
    out = deform_sdpa_torch(q, k, v, c, Wimg, Himg, 0.4)
    out.backward(do)
    n = lambda t: t.detach().numpy()
    ro, _ = oracle_fwd(n(q), n(k), n(v), n(c), Wimg, Himg, 0.4)
    rdq, rdk, rdv = oracle_bwd(n(q), n(k), n(v), n(c), n(do), Wimg, Himg, 0.4)
    assert out.shape == q.shape and out.dtype == q.dtype
    assert rel(out, ro) < 1e-5
    assert rel(q.grad, rdq) < 1e-4 and rel(k.grad, rdk) < 1e-4 and rel(v.grad, rdv) < 1e-4


def test_eager_operator_keeps_storage_dtype():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 1, 6, 16, generator=g).bfloat16() for _ in range(3))
    c = torch.rand(1, 2, 6, 2, 4, 2, generator=g)
    out = deform_sdpa_torch(q, k, v, c, 3, 2, 0.25)
    assert out.dtype == torch.bfloat16
    ro, _ = oracle_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), c.numpy(), 3, 2, 0.25)
    assert rel(out.float(), ro) < 2e-2
