"""Synthetic workloads for the deformable multi-view SDPA operator.

The five named shapes and their input distributions; the counterpart of the
reference harness' ``gen_inputs`` (``benchmark.py:108-114``: q/k/v ~ N(0,1),
coords ~ U[0,1)), extended with the out-of-bounds and clustered-coordinate
distributions the larger shapes call for. Inputs are always drawn on the CPU
from a seeded generator so that a CPU checker and the GPU see identical bits.
"""
import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    B: int
    V: int          # N_VIEWS
    H: int          # N_HEADS
    D: int          # HEAD_DIM
    W_IMG: int
    H_IMG: int
    P: int          # N_SAMPLES per (query, view)
    sm_scale: float
    dtype: str      # "fp32" | "bf16" | "fp16"
    coords: str     # "unit" | "border" | "clustered" | "coherent"
    seed: int

    @property
    def L(self):
        return self.W_IMG * self.H_IMG

    @property
    def rows(self):
        return self.B * self.V * self.H * self.L

    @property
    def query_samples(self):
        """Unit of work: (query row, sample) pairs = B*V*H*L * V*P."""
        return self.rows * self.V * self.P

    @property
    def esize(self):
        return 4 if self.dtype == "fp32" else 2

    def algorithmic_bytes(self, which):
        """Compulsory HBM bytes: q,k,v,out (+ dout,dq,dk,dv and q,k,v,out again) + coords.

        fwd = 4*N*e + C, bwd = 8*N*e + C, fwd+bwd = 12*N*e + 2*C with
        N = B*V*H*L*D elements and C = coords bytes; the per-row log-sum-exp
        side buffer (<1 %) is left out.
        """
        n = self.rows * self.D * self.esize
        c = self.B * self.V * self.L * self.V * self.P * 2 * 4
        return {"fwd": 4 * n + c, "bwd": 8 * n + c, "fwd+bwd": 12 * n + 2 * c}[which]

    def torch_dtype(self):
        return {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[self.dtype]


WORKLOADS = {
    # README example (README.md:26-43)
    "C1": Workload("C1", 2, 8, 16, 32, 14, 14, 32, 0.5, "fp32", "unit", 0),
    # benchmark-shaped (benchmark.py:16-19 with --h 8)
    "C2": Workload("C2", 2, 6, 8, 32, 18, 18, 32, 1.0 / math.sqrt(32), "fp32", "unit", 1),
    # larger maps, coords U[-0.1, 1.1): exercises per-tap zero padding
    "C3": Workload("C3", 1, 6, 8, 64, 32, 32, 16, 0.125, "fp32", "border", 2),
    # bf16 storage, fp32 accumulate
    "C4": Workload("C4", 2, 6, 8, 64, 48, 48, 32, 0.125, "bf16", "unit", 3),
    # backward contention stress: clustered coords
    "C5": Workload("C5", 2, 4, 8, 128, 64, 64, 64, 1.0 / math.sqrt(128), "bf16", "clustered", 4),
}


# Not one of the five named shapes: C5's shape with coordinates as deformable attention produces them, every query
# looking around its own pixel in the other views (reference point = the query's position, scaled to the middle
# 60 % of the image and shifted a little per (batch, query view, key view), samples N(0, 0.03^2) around it), so
# that neighbouring queries look at neighbouring places. C5 itself draws every query's centre at random.
EXTRA_WORKLOADS = {
    "C5c": Workload("C5c", 2, 4, 8, 128, 64, 64, 64, 1.0 / math.sqrt(128), "bf16", "coherent", 5),
}


def find_workload(name):
    return WORKLOADS.get(name) or EXTRA_WORKLOADS[name]


def gen_coords(kind, B, V, L, P, gen, W_IMG=None, H_IMG=None):
    """coords (B, V, L, V, P, 2) fp32; last axis is (x, y) normalised to [0, 1]."""
    shape = (B, V, L, V, P, 2)
    if kind == "unit":
        return torch.rand(shape, generator=gen, dtype=torch.float32)
    if kind == "border":
        return torch.rand(shape, generator=gen, dtype=torch.float32) * 1.2 - 0.1
    if kind == "clustered":
        mu = torch.rand((B, V, L, V, 1, 2), generator=gen, dtype=torch.float32) * 0.2 + 0.4
        eps = torch.randn(shape, generator=gen, dtype=torch.float32) * 0.03
        return (mu + eps).clamp_(0.0, 1.0)
    if kind == "coherent":
        ys, xs = torch.meshgrid(torch.arange(H_IMG), torch.arange(W_IMG), indexing="ij")
        base = torch.stack([xs.reshape(-1) / max(W_IMG - 1, 1), ys.reshape(-1) / max(H_IMG - 1, 1)], -1).float()
        mu = base.view(1, 1, L, 1, 1, 2) * 0.6 + 0.2 + 0.02 * torch.randn((B, V, 1, V, 1, 2), generator=gen, dtype=torch.float32)
        eps = torch.randn(shape, generator=gen, dtype=torch.float32) * 0.03
        return (mu + eps).clamp_(0.0, 1.0)
    raise ValueError(kind)


def gen_inputs(wl, device="cpu", with_dout=True):
    """q, k, v, coords[, dout] for a workload: drawn on CPU in that order, then moved."""
    gen = torch.Generator().manual_seed(wl.seed)
    shape = (wl.B, wl.V, wl.H, wl.L, wl.D)
    q = torch.randn(shape, generator=gen, dtype=torch.float32)
    k = torch.randn(shape, generator=gen, dtype=torch.float32)
    v = torch.randn(shape, generator=gen, dtype=torch.float32)
    coords = gen_coords(wl.coords, wl.B, wl.V, wl.L, wl.P, gen, wl.W_IMG, wl.H_IMG)
    outs = [q, k, v]
    if with_dout:
        outs.append(torch.randn(shape, generator=gen, dtype=torch.float32))
    dt = wl.torch_dtype()
    outs = [t.to(dt) for t in outs]
    outs.insert(3, coords)
    return tuple(t.to(device) for t in outs)


def oob_fractions(wl):
    """Fraction of bilinear taps that fall outside the image, and of samples with all four taps outside,
    for a workload's coordinates (per-tap zero padding: an outside tap contributes nothing)."""
    gen = torch.Generator().manual_seed(wl.seed)
    shape = (wl.B, wl.V, wl.H, wl.L, wl.D)
    for _ in range(3):                      # q, k, v come first in the draw order
        torch.randn(shape, generator=gen, dtype=torch.float32)
    c = gen_coords(wl.coords, wl.B, wl.V, wl.L, wl.P, gen, wl.W_IMG, wl.H_IMG)
    x0 = torch.floor(c[..., 0] * (wl.W_IMG - 1)).to(torch.int64)
    y0 = torch.floor(c[..., 1] * (wl.H_IMG - 1)).to(torch.int64)
    inside = []
    for dy in (0, 1):
        for dx in (0, 1):
            inside.append((x0 + dx >= 0) & (x0 + dx < wl.W_IMG) & (y0 + dy >= 0) & (y0 + dy < wl.H_IMG))
    inside = torch.stack(inside)
    return {"taps_outside": 1.0 - inside.float().mean().item(),
            "samples_fully_outside": (~inside.any(dim=0)).float().mean().item()}
