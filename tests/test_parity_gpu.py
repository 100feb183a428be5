"""GPU parity: the HIP kernels (through the operator and the C ABI) against the CPU oracle.

Error measure, everywhere: rel = max|x - ref| / max|ref| per tensor.
Bars: fp32 forward 1e-4, fp32 gradients 1e-3 (atomic ordering is not
deterministic), 16-bit storage 2e-2 (bf16 and fp16; the oracle is fed the
rounded inputs up-cast to fp32, which is what ops/torch.py:8,9,20 does).
"""
import glob
import math
import os
import sys

import numpy as np
import pytest
import torch

from oracle import oracle_bwd, oracle_fwd
from ops import _native
from ops.triton import deform_sdpa_triton
from workloads import WORKLOADS, find_workload, gen_inputs
from parity_util import oracle_on_slices, rel, slice_bh, spread_slices

pytestmark = pytest.mark.gpu

TOL_FWD = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}
TOL_BWD = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}
PATHS = {"gather": _native.PATH_GATHER, "lds": _native.PATH_LDS, "auto": _native.PATH_AUTO}



def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_op(q, k, v, coords, dout, W, Himg, scale):
    dev = "cuda:0"
    qg, kg, vg = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    out = deform_sdpa_triton(qg, kg, vg, coords.to(dev), W, Himg, scale)
    out.backward(dout.to(dev))
    torch.cuda.synchronize()
    return out.detach(), qg.grad, kg.grad, vg.grad


def oracle_all(q, k, v, coords, dout, W, Himg, scale):
    f = lambda t: t.float().numpy()
    out, lse = oracle_fwd(f(q), f(k), f(v), f(coords), W, Himg, scale)
    dq, dk, dv = oracle_bwd(f(q), f(k), f(v), f(coords), f(dout), W, Himg, scale)
    return out, lse, dq, dk, dv


def make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi, dtype):
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(3))
    coords = torch.rand(B, V, L, V, P, 2, generator=g) * (hi - lo) + lo
    dout = torch.randn(B, V, H, L, D, generator=g).to(dtype)
    return q, k, v, coords, dout


SMALL = [
    # seed B  V  H  Himg Wimg D    P   lo    hi
    (1, 1, 2, 2, 3, 5, 16, 3, -0.25, 1.25),     # tiny, non-square, N=6 < one chunk
    (2, 2, 3, 2, 6, 4, 32, 23, -0.1, 1.1),      # N=69: one full chunk + ragged tail
    (3, 1, 4, 3, 7, 9, 32, 32, 0.0, 1.0),       # N=128, L=63 not a multiple of the row tile
    (4, 1, 2, 2, 5, 6, 64, 17, -0.5, 1.5),      # heavy out-of-image
    (5, 2, 2, 1, 4, 7, 128, 40, 0.0, 1.0),
    (6, 1, 2, 1, 3, 3, 256, 9, -0.1, 1.1),
    (7, 1, 1, 1, 1, 1, 16, 1, 0.0, 1.0),        # degenerate 1x1 image, one sample
    (8, 1, 3, 2, 1, 11, 32, 5, -0.2, 1.2),      # single-row image
    (9, 1, 3, 2, 11, 1, 32, 5, -0.2, 1.2),      # single-column image
    (10, 1, 2, 2, 4, 5, 32, 129, -0.1, 1.1),    # many samples per view: three 64-sample pieces of the tap table
    (11, 1, 1, 2, 6, 6, 64, 200, 0.0, 1.0),     # one view, 200 samples
    (12, 1, 9, 1, 4, 3, 32, 2, -0.1, 1.1),      # many views, two samples each: the gather kernels are chosen
]


@pytest.mark.parametrize("path", sorted(PATHS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("case", SMALL, ids=[f"s{c[0]}" for c in SMALL])
def test_small_cases_vs_oracle(case, dtype, path):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    say(f"[case] small seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype} path={path}")
    q, k, v, c, do = make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi, dtype)
    scale = 1.0 / math.sqrt(D)
    prev = _native.set_path(PATHS[path])
    try:
        out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    finally:
        _native.set_path(prev)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert out.dtype == dtype and dq.dtype == dtype and dk.dtype == dtype and dv.dtype == dtype
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_staged_forward_two_row_blocks(dtype):
    """Many planes, few samples per view: the staged forward then gives a workgroup two blocks of query rows per
    staged plane (512 workgroups of one block would be two rounds on 256 CUs; 8 samples per view make the staging
    weigh). Rows per (batch, head) = 1944 is no multiple of the 256 rows of a workgroup: the last one is part full."""
    B, V, H, Himg, Wimg, D, P = 2, 6, 16, 18, 18, 32, 8
    say(f"[case] two row blocks B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    q, k, v, c, do = make_case(71, B, V, H, Himg, Wimg, D, P, -0.05, 1.05, dtype)
    scale = 1.0 / math.sqrt(D)
    out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


# fp32 storage, 16 or 32 samples per view, planes too large for LDS but small enough for two 16-column slabs of the
# whole image: the forward and the dq kernel walk the planes slab by slab through LDS (fwd_slab_kernel,
# bwd_dq_slab_kernel), every tap read from there.
SLABS = [
    # seed B  V  H  Himg Wimg D    P   lo     hi
    (81, 1, 2, 2, 20, 20, 64, 16, -0.1, 1.1),   # width a multiple of 4: two padding columns per image row; 800 query rows: 4 full workgroups and a part
    (82, 2, 3, 1, 23, 19, 64, 16, -0.3, 1.3),   # odd width, runs of 16 pixels cut by the row end, heavy out-of-image
    (83, 1, 2, 2, 17, 17, 128, 16, 0.0, 1.0),   # eight slabs per plane
    (84, 1, 1, 3, 20, 32, 32, 16, -0.05, 1.05), # two slabs per plane, one view
    (85, 1, 2, 1, 32, 32, 64, 16, -0.1, 1.1),   # the largest image the kernel takes (64 runs)
    (86, 1, 1, 2, 21, 48, 64, 16, -0.1, 1.1),   # three runs per image row, 63 runs
    (87, 1, 2, 1, 40, 16, 64, 16, 0.0, 1.0),    # one run per image row, tall image
    (88, 1, 2, 1, 16, 17, 128, 16, -0.2, 1.2),  # second run of a row holds one pixel
    (89, 1, 2, 2, 20, 20, 64, 32, -0.1, 1.1),   # 32 samples per view: two blocks of 16 per query row in one lane
    (90, 2, 1, 1, 25, 30, 32, 32, -0.2, 1.2),
    (91, 1, 3, 1, 18, 18, 128, 32, 0.0, 1.0),
    (92, 1, 2, 1, 30, 31, 64, 32, -0.1, 1.1),
]


@pytest.mark.parametrize("case", SLABS, ids=[f"b{c[0]}" for c in SLABS])
def test_slab_forward_vs_oracle(case):
    seed, B, V, H, Himg, Wimg, D, P, lo, hi = case
    dtype = torch.float32
    say(f"[case] slabs seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    q, k, v, c, do = make_case(seed, B, V, H, Himg, Wimg, D, P, lo, hi, dtype)
    c[0, 0, 1, 0, 3, 0] = float("nan")                     # a sample without taps
    c[0, V - 1, 5, 0, 7] = torch.tensor([1.0, 1.0])        # exactly on the last pixel: x1, y1 outside with weight 0
    c[0, 0, 6, V - 1, 2] = torch.tensor([-0.5, 0.5])       # far outside
    scale = 1.0 / math.sqrt(D)
    out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    prev = _native.set_path(_native.PATH_GATHER)           # the same forward by the gather kernel
    try:
        with torch.no_grad():
            og = deform_sdpa_triton(q.cuda(), k.cuda(), v.cuda(), c.cuda(), Wimg, Himg, scale)
    finally:
        _native.set_path(prev)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert torch.isfinite(out).all()
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(out, og.cpu().numpy()) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]                   # (dq by the slab kernel, dk/dv from the pairs it hands over)
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


# Clustered coordinates with at least 64 samples per view: the gather kernels then cut chunks per key view and
# work on the pixels of the window a chunk's samples fall into (fp32: multiply-adds; 16-bit storage: the 4x4x4
# block matrix instruction), or gather tap by tap where the window is too large or the image too narrow.
WINDOWS = [
    # seed B  V  H  Himg Wimg D    P    sigma  centres lo, hi
    (31, 1, 2, 2, 24, 20, 32, 64, 0.04, 0.3, 0.7),
    (32, 1, 3, 1, 16, 40, 128, 100, 0.03, 0.0, 1.0),       # clusters on the border: windows cut by the image edge
    (33, 2, 2, 2, 30, 30, 64, 70, 0.02, -0.05, 1.05),      # centres outside the image: samples with no tap inside
    (34, 1, 2, 1, 40, 3, 16, 64, 0.05, 0.2, 0.8),          # image narrower than one unit of a window row
    (35, 1, 1, 2, 12, 12, 256, 130, 0.3, 0.5, 0.5),        # wide spread: windows too large, every chunk gathers
    (36, 1, 2, 2, 33, 29, 64, 64, 0.004, 0.1, 0.9),        # very tight clusters: windows of one or two units
    (37, 1, 4, 1, 48, 48, 256, 64, 0.03, 0.3, 0.7),        # q and dout rows of a (batch, head) beyond 4 MB: dk/dv lists
                                                           # per group of query views (fp32: four groups, 16-bit: two)
]


# path: GATHER = forward in window mode, backward by the per-tap atomic kernel; AUTO = where the planes do not fit in
# LDS (w32, w33, w35, w36 and the fp32 case of w31), forward and dq in window mode, dq handing (p, ds) to the
# cell-binned dk/dv kernel (four-entry trips for 16-bit storage at D >= 128), else the staged kernels.
@pytest.mark.parametrize("path", [_native.PATH_GATHER, _native.PATH_AUTO], ids=["gather", "auto"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("case", WINDOWS, ids=[f"w{c[0]}" for c in WINDOWS])
def test_clustered_windows_vs_oracle(case, dtype, path):
    seed, B, V, H, Himg, Wimg, D, P, sigma, lo, hi = case
    say(f"[case] windows seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} sigma={sigma} {dtype} path={path}")
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(3))
    mu = torch.rand(B, V, L, V, 1, 2, generator=g) * (hi - lo) + lo
    c = mu + sigma * torch.randn(B, V, L, V, P, 2, generator=g)
    c[0, 0, 1, 0, 3, 0] = float("nan")                     # one NaN coordinate inside a cluster
    do = torch.randn(B, V, H, L, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    prev = _native.set_path(path)
    try:
        out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    finally:
        _native.set_path(prev)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_dense_box_forward_mixed_tiles_and_untouched_pixels(dtype):
    """16-bit storage, at least 64 samples per view, planes too large for LDS: tiles of 16 queries whose taps fall
    into a small box of the key view are worked on as dense products over the box (matrix instructions), the other
    tiles by the gather kernel. Here (1) every other tile of 16 queries has its samples spread over the whole image
    (no box), so that both kernels write parts of one output; (2) the clustered queries look at two spots with a
    gap between them: the box spans the gap, whose pixels no tap touches -- and V holds NaN and infinity there,
    which must not reach the output (the reference reads touched pixels only, ops/torch.py:14-15)."""
    say(f"[case] dense box forward, mixed tiles, NaN in untouched pixels {dtype}")
    g = torch.Generator().manual_seed(81)
    B, V, H, Himg, Wimg, D, P = 1, 2, 2, 24, 24, 64, 64
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(3))
    spot = torch.where(torch.rand(B, V, L, V, P, 1, generator=g) < 0.5, 0.3, 0.7)          # one of the two spots per sample
    c = spot + 0.012 * torch.randn(B, V, L, V, P, 2, generator=g)
    wide = ((torch.arange(L) // 16) % 2 == 1).view(1, 1, L, 1, 1, 1)                       # every other tile of 16 queries
    c = torch.where(wide, torch.rand(B, V, L, V, P, 2, generator=g), c)
    # the image centre lies between the spots: 0.5 * 23 = 11.5 -> pixels (11..12, 11..12); the spots' taps stay
    # within +-0.06 * 23 = 1.4 pixels of 6.9 and 16.1
    tight = c[:, :, ~wide.view(-1)]
    assert ((tight - 0.3).abs().amax(-1).clamp(max=1) < 0.07).logical_or((tight - 0.7).abs().amax(-1) < 0.07).all()
    v_bad = v.clone()
    for (yy, xx, val) in ((11, 11, float("nan")), (12, 12, float("inf")), (11, 12, float("-inf"))):
        v_bad[:, :, :, yy * Wimg + xx, :] = val
    do = torch.randn(B, V, H, L, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    # queries of the spread tiles may well touch the centre pixels: compare the clustered rows only for v_bad, and
    # everything for the clean v
    out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype] and rel(dk, rdk) < TOL_BWD[dtype] and rel(dv, rdv) < TOL_BWD[dtype]
    with torch.no_grad():
        out_bad = deform_sdpa_triton(q.cuda(), k.cuda(), v_bad.cuda(), c.cuda(), Wimg, Himg, scale)
    torch.cuda.synchronize()
    rows = ~wide.view(-1)
    assert torch.isfinite(out_bad[:, :, :, rows.cuda()].float()).all()
    assert rel(out_bad[:, :, :, rows.cuda()], ro[:, :, :, rows.numpy()]) < TOL_FWD[dtype]


GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_golden_fixtures(path):
    z = np.load(path)
    say(f"[case] golden {os.path.basename(path)}")
    W, Himg, scale = int(z["WIDTH"]), int(z["HEIGHT"]), float(z["sm_scale"])
    t = lambda n: torch.from_numpy(z[n])
    out, dq, dk, dv = run_op(t("q"), t("k"), t("v"), t("coords"), t("dout"), W, Himg, scale)
    assert rel(out, z["out"]) < 1e-4
    assert rel(dq, z["dq"]) < 1e-3
    assert rel(dk, z["dk"]) < 1e-3
    assert rel(dv, z["dv"]) < 1e-3


def test_lse_through_c_abi():
    """Direct C-ABI forward call: out and the base-2 log-sum-exp side buffer."""
    say("[case] c-abi forward lse")
    q, k, v, c, _ = make_case(21, 2, 3, 2, 6, 4, 32, 23, -0.1, 1.1, torch.float32)
    lib = _native.load()
    dev = "cuda:0"
    qg, kg, vg, cg = (t.to(dev).contiguous() for t in (q, k, v, c))
    out = torch.empty_like(qg)
    lse = torch.empty(q.shape[:4], device=dev, dtype=torch.float32)
    ws = torch.empty(lib.dsdpa_fwd_workspace_bytes(_native.DSDPA_F32, 2, 3, 2, 6, 4, 32, 23), device=dev,
                     dtype=torch.uint8)
    assert ws.numel() > 0
    rc = lib.dsdpa_fwd_f32(qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), cg.data_ptr(), out.data_ptr(),
                           lse.data_ptr(), ws.data_ptr(), 2, 3, 2, 6, 4, 32, 23, 0.2, None,
                           torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    ro, rl = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), c.numpy(), 4, 6, 0.2)
    assert rel(out, ro) < 1e-4
    assert np.abs(lse.cpu().numpy() - rl).max() < 1e-4


def test_closed_forms_on_gpu():
    say("[case] closed forms")
    q, k, v, c, do = make_case(22, 1, 2, 2, 4, 3, 32, 5, 0.0, 1.0, torch.float32)
    dev = "cuda:0"
    # constant V -> out is that constant
    out = deform_sdpa_triton(q.to(dev), k.to(dev), torch.full_like(v, 2.5).to(dev), c.to(dev), 3, 4, 0.9)
    assert (out - 2.5).abs().max().item() < 1e-5
    # everything far outside: out = 0, all gradients 0
    out, dq, dk, dv = run_op(q, k, v, c + 7.0, do, 3, 4, 0.9)
    assert out.abs().max().item() == 0.0
    assert dq.abs().max().item() == 0.0 and dk.abs().max().item() == 0.0 and dv.abs().max().item() == 0.0
    # NaN coordinates drop their samples instead of poisoning the row
    cn = c.clone()
    cn[0, 0, 0, 0, 0, 0] = float("nan")
    out = deform_sdpa_triton(q.to(dev), k.to(dev), v.to(dev), cn.to(dev), 3, 4, 0.9)
    ro, _ = oracle_fwd(q.numpy(), k.numpy(), v.numpy(), cn.numpy(), 3, 4, 0.9)
    assert torch.isfinite(out).all()
    assert rel(out, ro) < 1e-4


def test_reentrant_backward_and_noncontiguous_inputs():
    """retain_graph re-entry (benchmark.py:79) and strided q/k/v/dout."""
    say("[case] re-entrant backward")
    q, k, v, c, do = make_case(23, 1, 2, 2, 4, 5, 32, 6, 0.0, 1.0, torch.float32)
    dev = "cuda:0"
    base = torch.randn(1, 2, 2, 20, 64, generator=torch.Generator().manual_seed(1)).to(dev)
    qg = base[..., ::2].detach().requires_grad_(True)          # non-contiguous view
    kg, vg = k.to(dev).requires_grad_(True), v.to(dev).requires_grad_(True)
    out = deform_sdpa_triton(qg, kg, vg, c.to(dev), 5, 4, 0.3)
    dog = do.to(dev)
    out.backward(dog, retain_graph=True)
    g1 = (qg.grad.clone(), kg.grad.clone(), vg.grad.clone())
    qg.grad = kg.grad = vg.grad = None
    out.backward(dog.transpose(-1, -2).contiguous().transpose(-1, -2), retain_graph=True)
    ro, _, rdq, rdk, rdv = oracle_all(qg.detach().cpu(), k, v, c, do, 5, 4, 0.3)
    assert rel(out, ro) < 1e-4
    for got, again, ref in zip((qg.grad, kg.grad, vg.grad), g1, (rdq, rdk, rdv)):
        assert rel(got, ref) < 1e-3 and rel(again, ref) < 1e-3


# ------------------------------------------------------------------ strided q, k, v
# The reference's forward takes the strides of q, k, v (ops/triton.py:396-405). Here q, k, v with a contiguous
# head dimension are read in place: the two layouts a model produces without a copy -- a projection output
# (B, V, L, H, D) permuted to (B, V, H, L, D), and the three slices of a fused (B, V, L, 3, H, D) projection.
STRIDED = [
    # seed B  V  H  Himg Wimg D    P   layout
    (61, 2, 3, 2, 6, 4, 32, 23, "permuted"),      # planes in LDS
    (62, 1, 2, 3, 5, 7, 64, 9, "fused-qkv"),
    (63, 1, 2, 2, 40, 40, 64, 6, "permuted"),     # planes too large for LDS: gather kernels
    (64, 1, 2, 2, 24, 20, 32, 64, "fused-qkv"),   # 64 samples per view: chunks per view, window mode
    (65, 1, 2, 2, 20, 22, 64, 16, "permuted"),    # fp32: the slab kernels (planes staged into LDS from strided rows)
    (66, 1, 2, 2, 19, 21, 64, 32, "fused-qkv"),
]


def _strided_inputs(seed, B, V, H, L, D, layout, dtype):
    g = torch.Generator().manual_seed(seed)
    if layout == "permuted":
        base = [torch.randn(B, V, L, H, D, generator=g).to(dtype).cuda() for _ in range(3)]
        return [t.permute(0, 1, 3, 2, 4) for t in base]
    qkv = torch.randn(B, V, L, 3, H, D, generator=g).to(dtype).cuda()
    return [qkv[:, :, :, i].permute(0, 1, 3, 2, 4) for i in range(3)]


@pytest.mark.parametrize("path", sorted(PATHS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("case", STRIDED, ids=[f"t{c[0]}" for c in STRIDED])
def test_strided_inputs_read_in_place(case, dtype, path):
    seed, B, V, H, Himg, Wimg, D, P, layout = case
    say(f"[case] strided seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {layout} {dtype} path={path}")
    L = Himg * Wimg
    q, k, v = _strided_inputs(seed, B, V, H, L, D, layout, dtype)
    assert not q.is_contiguous() and q.stride(-1) == 1
    g = torch.Generator().manual_seed(seed + 100)
    c = (torch.rand(B, V, L, V, P, 2, generator=g) * 1.2 - 0.1).cuda()
    if P >= 64:
        c = (0.5 + 0.05 * torch.randn(B, V, L, V, P, 2, generator=g)).cuda()
    do = torch.randn(B, V, H, L, D, generator=g).to(dtype).cuda()
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
    scale = 1.0 / math.sqrt(D)
    prev = _native.set_path(PATHS[path])
    try:
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        out = deform_sdpa_triton(qg, kg, vg, c, Wimg, Himg, scale)
        torch.cuda.synchronize()
        fwd_extra = torch.cuda.max_memory_allocated() - before
        out.backward(do)
        torch.cuda.synchronize()
    finally:
        _native.set_path(prev)
    # no copy of q, k, v was made: the forward allocated out, lse and its workspace, nothing tensor-sized beyond
    lib = _native.load()
    code = _native.DSDPA_F32 if dtype == torch.float32 else _native.DSDPA_BF16
    ws = lib.dsdpa_fwd_workspace_bytes(code, B, V, H, Himg, Wimg, D, P)
    tensor_bytes = q.numel() * q.element_size()
    assert fwd_extra < tensor_bytes + q.numel() // D * 4 + ws + tensor_bytes // 2 + 4096, (fwd_extra, tensor_bytes, ws)
    assert out.is_contiguous() and qg.grad.shape == q.shape
    ro, _, rdq, rdk, rdv = oracle_all(q.cpu(), k.cpu(), v.cpu(), c.cpu(), do.cpu(), Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(qg.grad, rdq) < TOL_BWD[dtype]
    assert rel(kg.grad, rdk) < TOL_BWD[dtype]
    assert rel(vg.grad, rdv) < TOL_BWD[dtype]


def test_unreadable_layouts_are_copied():
    """A head dimension that is not contiguous, or rows that are not 16-byte aligned, cannot be read in place: the
    operator copies (the reference would read them through its strides; same results)."""
    say("[case] strided layouts that need a copy")
    g = torch.Generator().manual_seed(65)
    B, V, H, Himg, Wimg, D, P = 1, 2, 2, 4, 5, 32, 6
    L = Himg * Wimg
    wide = torch.randn(B, V, H, L, 2 * D, generator=g).cuda()
    q = wide[..., ::2]                                      # head dimension strided
    k = torch.randn(B, V, H, L, D + 2, generator=g).cuda()[..., 2:]     # rows start 8 bytes off a 16-byte boundary
    v = torch.randn(B, V, H, L, D, generator=g).cuda()
    c = torch.rand(B, V, L, V, P, 2, generator=g).cuda()
    do = torch.randn(B, V, H, L, D, generator=g).cuda()
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
    out = deform_sdpa_triton(qg, kg, vg, c, Wimg, Himg, 0.3)
    out.backward(do)
    torch.cuda.synchronize()
    ro, _, rdq, rdk, rdv = oracle_all(q.cpu(), k.cpu(), v.cpu(), c.cpu(), do.cpu(), Wimg, Himg, 0.3)
    assert rel(out, ro) < 1e-4 and rel(qg.grad, rdq) < 1e-3 and rel(kg.grad, rdk) < 1e-3 and rel(vg.grad, rdv) < 1e-3


# ------------------------------------------------------------------ the five named workloads
@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5", "C5c"])
def test_named_workloads_full_size(name):
    """Full-size run of each workload (the reference checks out, dq, dk, dv on the whole tensors,
    benchmark.py:116-149).

    * forward: the oracle over the WHOLE tensor (every batch, view, head and pixel);
    * backward: the oracle over the WHOLE tensors for C1-C3 (every (batch, head) slice), on eight of the sixteen
      (batch, head) slices for C4 and C5, batch and head indices spread (a slice of the full result must equal the
      oracle run on the slice: batches and heads are independent, coords are shared by the heads);
    * every (batch, head), sliced or not: the identities <q,dq> = <K,dK> (the logits are bilinear in q and K)
      and <V,dV> = <dout,out>, taken PER (batch, head) -- with `out` pinned everywhere by the full forward,
      a gradient plane that landed in another head's or batch item's place breaks them."""
    wl = find_workload(name)               # (C5c: C5's shape with every query looking around its own pixel)
    say(f"[case] workload {name} {wl}")
    q, k, v, c, do = gen_inputs(wl)
    dt = wl.torch_dtype()
    out, dq, dk, dv = run_op(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    assert torch.isfinite(out).all() and torch.isfinite(dq).all()
    assert torch.isfinite(dk).all() and torch.isfinite(dv).all()
    # forward over the whole tensor
    f = lambda t: t.float().numpy()
    ro, _ = oracle_fwd(f(q), f(k), f(v), f(c), wl.W_IMG, wl.H_IMG, wl.sm_scale)
    assert rel(out, ro) < TOL_FWD[dt]
    ro_t = torch.from_numpy(ro)
    for b in range(wl.B):                      # ... and per (batch, head): no plane may hide behind the global maximum
        for h in range(wl.H):
            assert rel(out[b, :, h], ro_t[b, :, h]) < TOL_FWD[dt], (b, h)
    # identities per (batch, head) (fp64 sums on the GPU)
    dims = (1, 3, 4)
    qd, kd, vd, dod = (t.to("cuda").double() for t in (q, k, v, do))
    a = (qd * dq.double()).sum(dims)
    bb = (kd * dk.double()).sum(dims)
    e = (vd * dv.double()).sum(dims)
    ff = (dod * out.double()).sum(dims)
    norm_qk = (qd.pow(2).sum(dims).sqrt() * dq.double().pow(2).sum(dims).sqrt())
    norm_v = (dod.pow(2).sum(dims).sqrt() * out.double().pow(2).sum(dims).sqrt())
    tol_id = 1e-3 if dt == torch.float32 else 3e-2
    assert ((a - bb).abs() < tol_id * norm_qk).all(), (a, bb)
    assert ((e - ff).abs() < tol_id * norm_v).all(), (e, ff)
    # backward on slices
    slices = spread_slices(wl.B, wl.H, wl.B * wl.H if name in ("C1", "C2", "C3") else 8)
    say(f"        oracle backward on slices {slices}")
    ref = oracle_on_slices(q, k, v, c, do, wl.W_IMG, wl.H_IMG, wl.sm_scale, slices, forward=False)
    for (bb_, hh), (_, rdq, rdk, rdv) in ref.items():
        assert rel(slice_bh(dq, bb_, hh), rdq) < TOL_BWD[dt], (bb_, hh)
        assert rel(slice_bh(dk, bb_, hh), rdk) < TOL_BWD[dt], (bb_, hh)
        assert rel(slice_bh(dv, bb_, hh), rdv) < TOL_BWD[dt], (bb_, hh)


def test_backward_recomputes_where_one_pair_exceeds_the_hand_over_buffer():
    """6 views of 90x90 with 64 samples: the (p, ds) pairs of ONE (batch, head) are 149 MB, more than the buffer
    the dq kernel may fill, so nothing is handed over and the cell kernel recomputes p and ds on a shape that
    otherwise takes the gather kernels (window mode in the forward and dq)."""
    B, V, H, Himg, Wimg, D, P = 1, 6, 1, 90, 90, 16, 64
    dtype = torch.float32
    lib = _native.load()
    # (the workspace holds no pair buffer: lists, counters and per-row pairs only)
    ws = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, B, V, H, Himg, Wimg, D, P, 0)
    assert ws < 12 * B * V * Himg * Wimg * V * P + (64 << 20)
    say(f"[case] no hand-over B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    g = torch.Generator().manual_seed(97)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(3))
    mu = torch.rand(B, V, L, V, 1, 2, generator=g) * 0.8 + 0.1
    c = mu + 0.03 * torch.randn(B, V, L, V, P, 2, generator=g)
    do = torch.randn(B, V, H, L, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


@pytest.mark.parametrize("spread, seed, D, dtype", [
    ("uniform", 101, 128, torch.bfloat16), ("clustered", 102, 128, torch.bfloat16), ("tight", 103, 128, torch.bfloat16),
    ("clustered", 104, 128, torch.float16), ("clustered", 105, 256, torch.float16), ("uniform", 106, 256, torch.bfloat16)],
    ids=["uniform", "clustered", "tight", "clustered-fp16", "clustered-d256-fp16", "uniform-d256"])
def test_backward_merges_entries_of_one_query_in_long_lists(spread, seed, D, dtype):
    """D = 128 in bf16 with the pairs handed over: the dk/dv kernel merges neighbouring list entries of one query
    and keeps the merged ones in a ring. 20x20 images (too large for the staged kernels) with 64 samples from 4 views
    give lists of some 230 entries
    per cell -- several 64-entry blocks, so the ring wraps. `uniform`: hardly any entry merges (the two blocks
    merged before the first trip fill the ring to its last place); `clustered`: sigma of one pixel, about half of
    them merge; `tight`: sigma of a tenth of a pixel, runs longer than the four entries that merge into one.
    D = 256: trips of eight merged entries instead of sixteen."""
    B, V, H, Himg, Wimg, P = 1, 4, 2 if D == 128 else 1, 20, 20, 64
    say(f"[case] merged entries {spread} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype) for _ in range(3))
    if spread == "uniform":
        c = torch.rand(B, V, L, V, P, 2, generator=g)
    else:
        mu = torch.rand(B, V, L, V, 1, 2, generator=g) * 0.8 + 0.1
        c = mu + (1.0 / 20 if spread == "clustered" else 0.1 / 20) * torch.randn(B, V, L, V, P, 2, generator=g)
    do = torch.randn(B, V, H, L, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    out, dq, dk, dv = run_op(q, k, v, c, do, Wimg, Himg, scale)
    ro, _, rdq, rdk, rdv = oracle_all(q, k, v, c, do, Wimg, Himg, scale)
    assert rel(out, ro) < TOL_FWD[dtype]
    assert rel(dq, rdq) < TOL_BWD[dtype]
    assert rel(dk, rdk) < TOL_BWD[dtype]
    assert rel(dv, rdv) < TOL_BWD[dtype]


@pytest.mark.parametrize("name", ["C2", "C4", "C5"])
def test_peak_memory_is_linear_in_tensor_size(name):
    """No sampled-tensor materialisation, no softmax matrix either: the fwd+bwd peak beyond the inputs and dout is
    out, dq, dk, dv (4 tensors), for 16-bit storage the fp32 dk/dv accumulators (the reference's dk32/dv32,
    ops/triton.py:428-429: 4 more), scratch proportional to the COORDINATES, which all heads share (20 bytes of tap
    table and 12 of cell ordering per 8-byte coordinate pair on the staged shapes, 12 of cell ordering on the
    others) -- and at most 128 MiB in which the dq kernel leaves (p, ds) of one group of (batch, head) pairs for the
    dk/dv kernel, whatever the shape. Nothing scales with samples x head width (the eager path needs 2*QS*D*4
    bytes: 1.5 GB at C2, 69 GB at C5), nor with samples x rows (8 bytes per query*sample would be 0.54 GB at C5)."""
    wl = WORKLOADS[name]
    say(f"[case] peak memory {name}")
    q, k, v, c, do = gen_inputs(wl, device="cuda")
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    out = deform_sdpa_triton(q, k, v, c, wl.W_IMG, wl.H_IMG, wl.sm_scale)
    out.backward(do)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - base
    tensor_bytes = q.numel() * q.element_size()
    coords_bytes = c.numel() * c.element_size()
    acc_bytes = 0 if q.dtype == torch.float32 else 2 * q.numel() * 4
    staged = name == "C2"
    # (the fifth tensor's worth is room for the per-row and per-cell side buffers: lse, delta, counters, work list)
    bound = 5 * tensor_bytes + acc_bytes + (4 if staged else 2) * coords_bytes + (0 if staged else 128 << 20)
    assert extra <= bound, (extra, bound, tensor_bytes, coords_bytes)
    if name == "C5":
        assert extra - 3 * tensor_bytes <= 620_000_000      # beyond dq, dk, dv: out, lse and the workspace
