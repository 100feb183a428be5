"""Writes the golden fixtures under tests/golden/ (run once, in the authoring container).

The reference stores no vectors of its own (its only check is the live A/B in
benchmark.py:116-149), so these are produced with the ATen library routine in
float64 (oracle/torch_eager.py: grid_sample bilinear/zeros/align_corners=True +
softmax, gradients by PyTorch autograd) on small seeded inputs that are
non-square, include out-of-image coordinates, and have sample counts that are
not multiples of the kernels' 64-sample chunks. The reference source is not
imported or executed.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle.torch_eager import eager_fwd_bwd  # noqa: E402

CASES = {
    #  name            seed B  V  H  Himg Wimg D   P   lo    hi   scale
    "tiny_nonsquare": (101, 1, 2, 2, 3, 5, 16, 3, -0.25, 1.25, 0.7),
    "mid_oob":        (102, 2, 3, 2, 6, 4, 32, 23, -0.1, 1.1, 0.25),
    "wide_head":      (103, 1, 2, 1, 4, 7, 128, 40, 0.0, 1.0, 0.09),
}


def main():
    for name, (seed, B, V, H, Himg, Wimg, D, P, lo, hi, scale) in CASES.items():
        g = torch.Generator().manual_seed(seed)
        L = Himg * Wimg
        q, k, v = (torch.randn(B, V, H, L, D, generator=g) for _ in range(3))
        coords = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
        dout = torch.randn(B, V, H, L, D, generator=g)
        out, dq, dk, dv = eager_fwd_bwd(q, k, v, coords, dout, Wimg, Himg, scale, dtype=torch.float64)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            q=q.numpy(), k=k.numpy(), v=v.numpy(), coords=coords.numpy(), dout=dout.numpy(),
            out=out.numpy().astype(np.float32), dq=dq.numpy().astype(np.float32),
            dk=dk.numpy().astype(np.float32), dv=dv.numpy().astype(np.float32),
            WIDTH=Wimg, HEIGHT=Himg, sm_scale=np.float32(scale))
        print(name, "written", out.shape)


if __name__ == "__main__":
    main()
