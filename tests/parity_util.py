"""Helpers shared by the GPU parity tests: the error measure and oracle runs on (batch, head) slices.

Batches and heads are independent and the coordinates are shared by the heads, so a (batch, head) slice of
the operator's result must equal the oracle run on that slice of the inputs. The C oracle's backward runs
one thread per (batch, head); slices are therefore run side by side from a thread pool (ctypes releases the
interpreter lock during the call).
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import torch

from oracle import oracle_bwd, oracle_fwd


def rel(a, b):
    """max|a - b| / max|b| per tensor."""
    a = a.detach().double().cpu().numpy() if torch.is_tensor(a) else np.asarray(a, dtype=np.float64)
    b = b.detach().double().cpu().numpy() if torch.is_tensor(b) else np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def slice_bh(t, b, h):
    return t[b:b + 1, :, h:h + 1].contiguous()


def oracle_on_slices(q, k, v, coords, dout, W, Himg, scale, slices, forward=True):
    """{(b, h): (out or None, dq, dk, dv)} from the C oracle, the slices computed in parallel."""
    f = lambda t: t.float().numpy()

    def one(bh):
        b, h = bh
        args = (f(slice_bh(q, b, h)), f(slice_bh(k, b, h)), f(slice_bh(v, b, h)), f(coords[b:b + 1].contiguous()))
        out = oracle_fwd(*args, W, Himg, scale)[0] if forward else None
        dq, dk, dv = oracle_bwd(*args, f(slice_bh(dout, b, h)), W, Himg, scale)
        return out, dq, dk, dv

    with ThreadPoolExecutor(max_workers=max(1, min(16, len(slices)))) as pool:
        return dict(zip(slices, pool.map(one, slices)))


def spread_slices(B, H, n=4):
    """n (batch, head) pairs (all of them when n >= B*H) whose batch and head indices are spread over the shape: the
    first and the last batch item and head are always among them."""
    if n >= B * H:
        return [(b, h) for b in range(B) for h in range(H)]
    cand = [(0, 1 % H), (B - 1, 0), (0, H - 1), (B - 1, H // 2)]
    # further pairs: heads taken round with a stride coprime to H, batch items alternating
    step = next(s for s in (3, 5, 7, 1) if H % s or s == 1)
    cand += [((i + 1) % B, (2 + i * step) % H) for i in range(B * H)]
    out = []
    for c in cand:
        if c not in out:
            out.append(c)
        if len(out) == n:
            break
    return out
