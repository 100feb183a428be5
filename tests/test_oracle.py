"""Pins the CPU oracle (oracle/dsdpa_oracle.c) without running the reference.

The reference holds no golden vectors (its only check is a live A/B,
benchmark.py:116-149), so the oracle is pinned by
  * hand-worked tap tables (x/y order, row*W+col, per-tap zero padding),
  * the ATen library routine grid_sample + softmax (oracle/torch_eager.py),
  * an independent float64 brute force that realises zero padding with a
    zero-bordered image instead of bounds tests,
  * closed forms and invariants a dropped term / swapped index would break,
  * for the backward: autograd through the library routine, central finite
    differences of the oracle's own forward, and homogeneity identities.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle_bwd, oracle_fwd, oracle_taps
from oracle.torch_eager import deform_sdpa_eager, eager_fwd_bwd


def make_case(seed, B, V, H, Himg, Wimg, D, P, lo=0.0, hi=1.0):
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q = torch.randn(B, V, H, L, D, generator=g)
    k = torch.randn(B, V, H, L, D, generator=g)
    v = torch.randn(B, V, H, L, D, generator=g)
    coords = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
    dout = torch.randn(B, V, H, L, D, generator=g)
    return q, k, v, coords, dout


def rel(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


# ---------------------------------------------------------------- taps, by hand
def test_taps_known_answers_nonsquare():
    W, Himg = 4, 3      # x_pix = x*3, y_pix = y*2
    # exact pixel centre (col 1, row 1) -> pixel 1*4+1 = 5 carries all the weight
    pix, w = oracle_taps(1 / 3, 0.5, W, Himg)
    assert pix[0] == 5 and w[0] == pytest.approx(1.0, abs=1e-6)
    assert sum(w[1:]) == pytest.approx(0.0, abs=1e-6)
    # x = 0.5 -> x_pix 1.5 ; y = 0.25 -> y_pix 0.5: cols 1,2 rows 0,1, all weights 1/4
    pix, w = oracle_taps(0.5, 0.25, W, Himg)
    assert pix == [0 * 4 + 1, 0 * 4 + 2, 1 * 4 + 1, 1 * 4 + 2]
    assert w == pytest.approx([0.25] * 4, abs=1e-6)
    # x/y order: x = 0.9 (col 2.7), y = 0.1 (row 0.2)
    pix, w = oracle_taps(0.9, 0.1, W, Himg)
    assert pix == [2, 3, 6, 7]
    assert w == pytest.approx([0.3 * 0.8, 0.7 * 0.8, 0.3 * 0.2, 0.7 * 0.2], abs=1e-5)


def test_taps_out_of_bounds_per_tap():
    W, Himg = 4, 3
    # x_pix = -0.25: left taps outside, right taps (col 0) keep weight 0.75
    pix, w = oracle_taps(-0.25 / 3, 0.0, W, Himg)
    assert pix[0] == -1 and pix[2] == -1
    assert pix[1] == 0 and w[1] == pytest.approx(0.75, abs=1e-5)
    # x_pix = 3.5 (beyond last col 3): left tap col 3 weight 0.5, right tap outside
    pix, w = oracle_taps(3.5 / 3, 0.0, W, Himg)
    assert pix[0] == 3 and w[0] == pytest.approx(0.5, abs=1e-5) and pix[1] == -1
    # y beyond bottom: y_pix = 2.25 -> top taps row 2 weight .75, bottom taps outside
    pix, w = oracle_taps(0.0, 2.25 / 2, W, Himg)
    assert pix[0] == 2 * 4 and w[0] == pytest.approx(0.75, abs=1e-5)
    assert pix[2] == -1 and pix[3] == -1
    # far outside: nothing left
    pix, _ = oracle_taps(5.0, -3.0, W, Himg)
    assert pix == [-1, -1, -1, -1]
    pix, _ = oracle_taps(float("nan"), 0.5, W, Himg)
    assert pix == [-1, -1, -1, -1]


# ------------------------------------------------- library routine (grid_sample)
CASES = [
    # seed B V H Himg Wimg D  P   lo    hi
    (0, 1, 2, 2, 3, 4, 16, 3, -0.3, 1.3),
    (1, 2, 3, 2, 5, 3, 32, 4, 0.0, 1.0),
    (2, 1, 4, 3, 6, 7, 16, 5, -0.1, 1.1),
    (3, 2, 2, 1, 4, 4, 64, 8, 0.0, 1.0),
    (4, 1, 1, 2, 2, 9, 16, 2, -1.5, 2.5),
]


@pytest.mark.parametrize("case", CASES)
def test_fwd_matches_library_routine(case):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    q, k, v, c, _ = make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi)
    ref = deform_sdpa_eager(q.double(), k.double(), v.double(), c.double(), Wimg, Himg, 0.37,
                            dtype=torch.float64)
    out, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), Wimg, Himg, 0.37)
    # coordinates are float32 in the oracle and float64 in this run of the library: 1e-5
    assert rel(out, ref.numpy()) < 1e-5


@pytest.mark.parametrize("case", CASES)
def test_bwd_matches_library_autograd(case):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    q, k, v, c, do = make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi)
    _, dq_r, dk_r, dv_r = eager_fwd_bwd(q, k, v, c, do, Wimg, Himg, 0.37, dtype=torch.float64)
    dq, dk, dv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.37)
    assert rel(dq, dq_r.numpy()) < 1e-5
    assert rel(dk, dk_r.numpy()) < 1e-5
    assert rel(dv, dv_r.numpy()) < 1e-5


# ------------------------------------------- independent brute force (float64)
def brute_force(q, k, v, c, Wimg, Himg, scale):
    """Zero padding by a 2-pixel zero border; dense per-query pixel weights."""
    B, V, H, L, D = q.shape
    P = c.shape[-2]
    out = np.zeros((B, V, H, L, D))
    lse = np.zeros((B, V, H, L))
    pad = 2
    Wp, Hp = Wimg + 2 * pad, Himg + 2 * pad
    for b in range(B):
        for h in range(H):
            kp = np.zeros((V, Hp, Wp, D))
            vp = np.zeros((V, Hp, Wp, D))
            kp[:, pad:pad + Himg, pad:pad + Wimg] = k[b, :, h].reshape(V, Himg, Wimg, D)
            vp[:, pad:pad + Himg, pad:pad + Wimg] = v[b, :, h].reshape(V, Himg, Wimg, D)
            for s1 in range(V):
                for l in range(L):
                    ks, vs = [], []
                    for s2 in range(V):
                        for p in range(P):
                            x = float(c[b, s1, l, s2, p, 0]) * (Wimg - 1) + pad
                            y = float(c[b, s1, l, s2, p, 1]) * (Himg - 1) + pad
                            x = min(max(x, 0.0), Wp - 1.001)   # far outside -> inside the zero border
                            y = min(max(y, 0.0), Hp - 1.001)
                            x0, y0 = int(math.floor(x)), int(math.floor(y))
                            fx, fy = x - x0, y - y0
                            kk = ((1 - fx) * (1 - fy) * kp[s2, y0, x0] + fx * (1 - fy) * kp[s2, y0, x0 + 1]
                                  + (1 - fx) * fy * kp[s2, y0 + 1, x0] + fx * fy * kp[s2, y0 + 1, x0 + 1])
                            vv = ((1 - fx) * (1 - fy) * vp[s2, y0, x0] + fx * (1 - fy) * vp[s2, y0, x0 + 1]
                                  + (1 - fx) * fy * vp[s2, y0 + 1, x0] + fx * fy * vp[s2, y0 + 1, x0 + 1])
                            ks.append(kk)
                            vs.append(vv)
                    ks, vs = np.stack(ks), np.stack(vs)
                    s = ks @ q[b, s1, h, l] * scale
                    w = np.exp(s - s.max())
                    lse[b, s1, h, l] = (s.max() + math.log(w.sum())) / math.log(2.0)
                    out[b, s1, h, l] = (w / w.sum()) @ vs
    return out, lse


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-0.3, 1.3)])
def test_fwd_matches_brute_force(lo, hi):
    q, k, v, c, _ = make_case(11, 1, 2, 2, 3, 4, 16, 3, lo, hi)
    # coords within the 2-pixel border so the clamp above never bites
    ref, lse_ref = brute_force(q.double().numpy(), k.double().numpy(), v.double().numpy(),
                               c.double().numpy(), 4, 3, 0.7)
    out, lse = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 4, 3, 0.7)
    assert rel(out, ref) < 1e-5
    assert np.abs(lse - lse_ref).max() < 1e-4


# ----------------------------------------------------------------- closed forms
def test_pixel_centre_coords_reduce_to_plain_sdpa():
    """Coords on pixel centres make sampling a pure gather -> textbook attention."""
    B, V, H, Himg, Wimg, D, P = 1, 3, 2, 3, 5, 16, 4
    L = Himg * Wimg
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(B, V, H, L, D, generator=g) for _ in range(3))
    col = torch.randint(0, Wimg, (B, V, L, V, P), generator=g)
    row = torch.randint(0, Himg, (B, V, L, V, P), generator=g)
    coords = torch.stack([col / (Wimg - 1), row / (Himg - 1)], dim=-1).float()
    out, lse = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), coords.numpy(), Wimg, Himg, 0.3)
    pix = row * Wimg + col                                   # (B, s1, L, s2, P)
    for s1 in range(V):
        for h in range(H):
            for l in range(0, L, 4):
                keys = torch.cat([k[0, s2, h][pix[0, s1, l, s2]] for s2 in range(V)])   # (V*P, D)
                vals = torch.cat([v[0, s2, h][pix[0, s1, l, s2]] for s2 in range(V)])
                ref = F.scaled_dot_product_attention(q[0, s1, h, l][None, None], keys[None], vals[None],
                                                     scale=0.3)[0, 0]
                assert rel(out[0, s1, h, l], ref.numpy()) < 2e-5
                lref = torch.logsumexp(keys @ q[0, s1, h, l] * 0.3, 0) / math.log(2.0)
                assert abs(lse[0, s1, h, l] - lref.item()) < 1e-4


def test_constant_v_zero_scale_all_oob_and_permutation():
    q, k, v, c, _ = make_case(6, 1, 2, 2, 4, 3, 16, 5)
    vc = torch.full_like(v, 2.5)
    out, _ = oracle_fwd(q.numpy(), k.numpy(), vc.numpy(), c.numpy(), 3, 4, 0.9)
    assert np.abs(out - 2.5).max() < 1e-5                     # convex combination of a constant
    # sm_scale = 0: uniform softmax -> mean of the sampled values; lse = log2(N)
    out0, lse0 = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 3, 4, 0.0)
    outk0, _ = oracle_fwd(q.numpy(), np.zeros_like(k.numpy()), v.numpy(), c.numpy(), 3, 4, 0.9)
    assert rel(out0, outk0) < 1e-6
    assert np.abs(lse0 - math.log2(2 * 5)).max() < 1e-5
    # everything far outside: k~ = v~ = 0 -> out = 0 and the row still has N unit terms
    far = c + 7.0
    outf, lsef = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), far.numpy(), 3, 4, 0.9)
    assert np.abs(outf).max() == 0.0
    assert np.abs(lsef - math.log2(2 * 5)).max() < 1e-5
    dq, dk, dv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), far.numpy(), q.numpy(), 3, 4, 0.9)
    assert np.abs(dq).max() == 0.0 and np.abs(dk).max() == 0.0 and np.abs(dv).max() == 0.0
    # permuting the P samples inside each view leaves out unchanged
    perm = torch.randperm(5, generator=torch.Generator().manual_seed(1))
    outp, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c[:, :, :, :, perm].contiguous().numpy(), 3, 4, 0.9)
    ref, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 3, 4, 0.9)
    assert rel(outp, ref) < 1e-6


def test_view_order_and_head_sharing():
    """Swapping two key views together with their coords is a no-op; heads share coords."""
    q, k, v, c, _ = make_case(7, 1, 3, 2, 3, 3, 16, 2)
    ref, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 3, 3, 0.5)
    # swap key/value views 0 and 2 and the s2 axis of coords -> same output
    idx = [2, 1, 0]
    out, _ = oracle_fwd(q.numpy(), k[:, idx].contiguous().numpy(), v[:, idx].contiguous().numpy(),
                        c[:, :, :, idx].contiguous().numpy(), 3, 3, 0.5)
    assert rel(out, ref) < 1e-6
    # swapping only k/v views (not coords) must change the result: views are not interchangeable
    out2, _ = oracle_fwd(q.numpy(), k[:, idx].contiguous().numpy(), v[:, idx].contiguous().numpy(),
                         c.numpy(), 3, 3, 0.5)
    assert rel(out2, ref) > 1e-3
    # heads are independent and share coords: head 1 alone == slice of the joint run
    out_h1, _ = oracle_fwd(q[:, :, 1:].contiguous().numpy(), k[:, :, 1:].contiguous().numpy(),
                           v[:, :, 1:].contiguous().numpy(), c.numpy(), 3, 3, 0.5)
    assert rel(out_h1, ref[:, :, 1:]) < 1e-7


# -------------------------------------------------------------------- backward
def test_bwd_finite_differences():
    q, k, v, c, do = make_case(8, 1, 2, 1, 2, 3, 16, 2, -0.2, 1.2)
    qn, kn, vn, cn, don = (t.numpy().copy() for t in (q, k, v, c, do))
    dq, dk, dv = oracle_bwd(qn, kn, vn, cn, don, 3, 2, 0.6)

    def loss(qq, kk, vv):
        out, _ = oracle_fwd(qq, kk, vv, cn, 3, 2, 0.6)
        return float((out.astype(np.float64) * don).sum())

    rng = np.random.default_rng(0)
    eps = 1e-2   # forward returns float32; central differences of a smooth function
    for name, arr, grad in (("q", qn, dq), ("k", kn, dk), ("v", vn, dv)):
        for _ in range(12):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            old = arr[idx]
            arr[idx] = old + eps
            lp = loss(qn, kn, vn)
            arr[idx] = old - eps
            lm = loss(qn, kn, vn)
            arr[idx] = old
            fd = (lp - lm) / (2 * eps)
            assert abs(fd - grad[idx]) < 2e-3 * max(1.0, abs(fd)), (name, idx, fd, grad[idx])


@pytest.mark.parametrize("case", CASES)
def test_coords_gradient_matches_library_autograd(case):
    """The gradient of the normalised coordinates, summed over the heads that share them, against
    autograd through grid_sample (float64), out-of-bounds taps included."""
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    q, k, v, c, do = make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi)
    *_, dc_r = eager_fwd_bwd(q, k, v, c, do, Wimg, Himg, 0.37, dtype=torch.float64, with_coords=True)
    *_, dc = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.37,
                        with_coords=True)
    assert dc.shape == tuple(c.shape)
    assert np.abs(dc_r.numpy()).max() > 0
    assert rel(dc, dc_r.numpy()) < 1e-5


def test_coords_gradient_closed_form_linear_image():
    """V = a*col + b*row per channel (a plane), sm_scale = 0: every p_n = 1/N and the bilinear sample of a
    plane is exact, so dL/dx = (W-1)/N * sum_h dout_h.a_h and dL/dy = (Himg-1)/N * sum_h dout_h.b_h for
    every in-bounds sample, whatever the coordinates."""
    B, V, H, Himg, Wimg, D, P = 1, 2, 3, 4, 5, 16, 3
    g = torch.Generator().manual_seed(77)
    L, N = Himg * Wimg, V * P
    a = torch.randn(V, H, D, generator=g)
    b = torch.randn(V, H, D, generator=g)
    col = torch.arange(L) % Wimg
    row = torch.arange(L) // Wimg
    v = (a[:, :, None, :] * col[None, None, :, None] + b[:, :, None, :] * row[None, None, :, None])[None]
    q = torch.randn(B, V, H, L, D, generator=g)
    k = torch.randn(B, V, H, L, D, generator=g)
    do = torch.randn(B, V, H, L, D, generator=g)
    c = torch.rand(B, V, L, V, P, 2, generator=g) * 0.98 + 0.01
    *_, dc = oracle_bwd(q.numpy(), k.numpy(), v.contiguous().numpy(), c.numpy(), do.numpy(), Wimg, Himg, 0.0,
                        with_coords=True)
    # expect[b, s1, l, s2, :, 0] = (W-1)/N * sum_h dout[b,s1,h,l,:] . a[s2,h,:]
    ex = torch.einsum("bshld,thd->bslt", do.double(), a.double()) * (Wimg - 1) / N
    ey = torch.einsum("bshld,thd->bslt", do.double(), b.double()) * (Himg - 1) / N
    assert np.abs(dc[..., 0] - ex[..., None].numpy()).max() < 1e-4 * float(ex.abs().max())
    assert np.abs(dc[..., 1] - ey[..., None].numpy()).max() < 1e-4 * float(ey.abs().max())


def test_coords_gradient_finite_differences():
    """Central differences of the oracle's own forward in single coordinates (steps that stay inside
    the bilinear cell, where the forward is smooth)."""
    q, k, v, c, do = make_case(12, 1, 2, 2, 3, 4, 16, 2, 0.05, 0.95)
    Wimg, Himg = 4, 3
    qn, kn, vn, cn, don = (t.numpy().copy() for t in (q, k, v, c, do))
    *_, dc = oracle_bwd(qn, kn, vn, cn, don, Wimg, Himg, 0.6, with_coords=True)

    def loss(cc):
        out, _ = oracle_fwd(qn, kn, vn, cc, Wimg, Himg, 0.6)
        return float((out.astype(np.float64) * don).sum())

    rng = np.random.default_rng(1)
    eps, checked = 2e-3, 0
    for _ in range(60):
        idx = tuple(rng.integers(0, s) for s in cn.shape)
        size = (Wimg if idx[-1] == 0 else Himg) - 1
        pix = float(cn[idx]) * size
        if min(pix - math.floor(pix), math.ceil(pix) - pix) < 3 * eps * size:
            continue                                    # too close to a cell border
        old = cn[idx]
        cn[idx] = old + eps
        lp = loss(cn)
        cn[idx] = old - eps
        lm = loss(cn)
        cn[idx] = old
        fd = (lp - lm) / (float(np.float32(old + eps)) - float(np.float32(old - eps)))
        assert abs(fd - dc[idx]) < 5e-3 * max(1.0, abs(fd)), (idx, fd, dc[idx])
        checked += 1
    assert checked >= 20


def test_bwd_homogeneity_identities():
    """Logits are bilinear in (q, K) and out is linear in V:
    <q,dq> = <K,dK> and <V,dV> = <dout,out>."""
    q, k, v, c, do = make_case(9, 2, 3, 2, 4, 5, 32, 4, -0.1, 1.1)
    out, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 5, 4, 0.4)
    dq, dk, dv = oracle_bwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), do.numpy(), 5, 4, 0.4)
    a = float((q.numpy().astype(np.float64) * dq).sum())
    b = float((k.numpy().astype(np.float64) * dk).sum())
    assert abs(a - b) < 1e-4 * max(abs(a), 1.0)
    e = float((v.numpy().astype(np.float64) * dv).sum())
    f = float((do.numpy().astype(np.float64) * out).sum())
    assert abs(e - f) < 1e-4 * max(abs(f), 1.0)


def test_library_routine_gradcheck_tiny():
    """The library path itself is differentiable where we use it (float64 gradcheck)."""
    q, k, v, c, _ = make_case(10, 1, 2, 1, 2, 2, 4, 2, 0.05, 0.95)
    q, k, v = (t.double().requires_grad_(True) for t in (q, k, v))
    fn = lambda a, b, d: deform_sdpa_eager(a, b, d, c.double(), 2, 2, 0.5, dtype=torch.float64)
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-5)
