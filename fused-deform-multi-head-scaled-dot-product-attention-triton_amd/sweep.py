"""Latency / peak-memory sweep and correctness check of the fused operator against the eager one.

The counterpart of the reference harness (``benchmark.py:12-149``) without ``triton.testing``: same CLI
(``--b --h --d --iw --sm-scale``), same sweep (``S_views`` x ``P_samples`` in {2,4,..,12}, forward and
backward, providers "fused" and "torch"), same ``[Check]`` lines (``allclose(atol=rtol=1e-2)`` on out/dq/dk/dv
plus max-abs errors, run at the largest ``S_views`` of each line) and ``[Mem]`` lines. Functions are defined
before use, and timing uses HIP events on the current stream (median of ``--rep`` runs after ``--warmup``).

    python sweep.py --b 2 --h 8 --d 32 --iw 18            # full sweep, prints a table per mode
    python sweep.py --quick                               # S, P in {2, 6, 12} only
    python sweep.py --views 24 --samples 16 --path lds    # one point, on a named kernel path

Besides the printed tables it leaves, in ``--save-path`` (default ``./results``), ``logs.txt`` with the ``[Mem]``
lines and one latency CSV (and one peak-memory CSV) per mode and ``P_samples`` -- the files the reference's
``perf_report`` run writes (``benchmark.py:106``).
"""
import argparse
import os
import statistics
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

from ops import _native                                         # noqa: E402
from ops.torch import deform_sdpa_torch as ref_deform_sdpa      # noqa: E402
from ops.triton import deform_sdpa_triton as fused_deform_sdpa  # noqa: E402


def gen_inputs(batch, S_views, N_HEADS, W_IMG, H_IMG, HEAD_DIM, P_samples, device, dtype=torch.float32, seed=0):
    """q, k, v ~ N(0,1) (requires_grad), coords ~ U[0,1) -- the reference's ``gen_inputs`` with a seed."""
    g = torch.Generator().manual_seed(seed)
    L = W_IMG * H_IMG
    q, k, v = (torch.randn(batch, S_views, N_HEADS, L, HEAD_DIM, generator=g).to(dtype).to(device).requires_grad_(True)
               for _ in range(3))
    coords = torch.rand(batch, S_views, L, S_views, P_samples, 2, generator=g).to(device)
    return q, k, v, coords


def check_correctness(q, k, v, coords, W_IMG, H_IMG, sm_scale, atol=1e-2, rtol=1e-2):
    """Fused vs eager on the same inputs: forward, then dq/dk/dv with a shared dout."""
    dout = torch.randn_like(q)
    res = {}
    grads = {}
    for name, fn in (("ref", ref_deform_sdpa), ("fused", fused_deform_sdpa)):
        qq, kk, vv = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
        out = fn(qq, kk, vv, coords.detach().clone(), W_IMG, H_IMG, sm_scale)
        out.backward(dout)
        grads[name] = (out.detach(), qq.grad, kk.grad, vv.grad)
    for label, a, b in zip(("out", "dq", "dk", "dv"), grads["ref"], grads["fused"]):
        res[label + "_ok"] = torch.allclose(a.float(), b.float(), atol=atol, rtol=rtol)
        res[label + "_max"] = (a.float() - b.float()).abs().max().item()
    return res


def time_ms(fn, warmup, rep):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(rep):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return statistics.median(times)


def bench_point(provider, mode, q, k, v, coords, W_IMG, H_IMG, sm_scale, warmup, rep):
    op = fused_deform_sdpa if provider == "fused" else ref_deform_sdpa
    if mode == "fwd":
        def fn():
            with torch.no_grad():
                return op(q, k, v, coords, W_IMG, H_IMG, sm_scale)
    else:
        out = op(q, k, v, coords, W_IMG, H_IMG, sm_scale)
        dout = torch.randn_like(out)

        def fn():
            q.grad = k.grad = v.grad = None
            out.backward(dout, retain_graph=True)
    ms = time_ms(fn, warmup, rep)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    fn()
    torch.cuda.synchronize()
    peak_mb = (torch.cuda.max_memory_allocated() - base) / 1e6
    return ms, peak_mb


def write_csv_tables(rows, args, providers, S_LIST, P_LIST):
    """One CSV per (mode, P_samples) line of the sweep, named and shaped like the tables the reference harness
    leaves in its results directory (``benchmark.py:106``, ``perf_report(...).run(save_path=..., print_data=True)``:
    x column ``S_views``, one latency column per provider), so that the published plots can be redrawn; plus the
    peak-memory table of the same points (the reference keeps those figures as ``[Mem]`` lines only)."""
    titles = {"fused": "HIP (coord-fused)", "torch": "Torch (grid_sample)"}
    for mode in ("fwd", "bwd"):
        for P in P_LIST:
            name = f"coord-attn-B{args.b}-H{args.h}-D{args.d}-{mode}-W{args.iw}-P{P}"
            for suffix, col in ((".csv", 4), ("-peak-mb.csv", 5)):
                with open(os.path.join(args.save_path, name + suffix), "w") as f:
                    f.write("S_views," + ",".join(titles[p] for p in providers) + "\n")
                    for S in S_LIST:
                        vals = {r[3]: r[col] for r in rows if r[:3] == (mode, P, S)}
                        f.write(f"{S:.1f}," + ",".join(f"{vals[p]:.6f}" for p in providers) + "\n")


def main(argv=None):
    ap = argparse.ArgumentParser(description="Sweep of deformable multi-view SDPA: fused HIP kernels vs eager PyTorch.")
    ap.add_argument("--b", type=int, default=2, help="Batch size.")
    ap.add_argument("--h", type=int, default=32, help="Number of attention heads.")
    ap.add_argument("--d", type=int, default=32, help="Dimension of each attention head.")
    ap.add_argument("--iw", type=int, default=18, help="Width of the image (height is set to be the same).")
    ap.add_argument("--sm-scale", type=float, default=0.5)
    ap.add_argument("--dtype", default="fp32", choices=["fp32", "bf16", "fp16"])
    ap.add_argument("--quick", action="store_true", help="S, P in {2, 6, 12} only")
    ap.add_argument("--views", default=None, help="comma-separated S_views instead of the sweep's")
    ap.add_argument("--samples", default=None, help="comma-separated P_samples instead of the sweep's")
    ap.add_argument("--path", default="auto", choices=["auto", "lds", "gather"],
                    help="kernel path of the fused provider: chosen by shape, K/V planes staged in LDS, or taps "
                         "gathered through L1/L2")
    ap.add_argument("--no-torch", action="store_true", help="skip timing the eager provider")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--rep", type=int, default=20)
    ap.add_argument("--save-path", default="./results")
    args = ap.parse_args(argv)

    dtype = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[args.dtype]
    S_LIST = [2, 6, 12] if args.quick else [2, 4, 6, 8, 10, 12]
    P_LIST = [2, 6, 12] if args.quick else [2, 4, 6, 8, 10, 12]
    if args.views:
        S_LIST = [int(x) for x in args.views.split(",")]
    if args.samples:
        P_LIST = [int(x) for x in args.samples.split(",")]
    prev_path = _native.set_path({"auto": _native.PATH_AUTO, "lds": _native.PATH_LDS, "gather": _native.PATH_GATHER}[args.path])
    providers = ["fused"] if args.no_torch else ["fused", "torch"]
    dev = torch.device("cuda", torch.cuda.current_device())
    os.makedirs(args.save_path, exist_ok=True)
    log = open(os.path.join(args.save_path, "logs.txt"), "w")
    rows = []
    for mode in ("fwd", "bwd"):
        for P in P_LIST:
            for S in S_LIST:
                q, k, v, coords = gen_inputs(args.b, S, args.h, args.iw, args.iw, args.d, P, dev, dtype)
                if S == max(S_LIST) and mode == "fwd":
                    chk = check_correctness(q, k, v, coords, args.iw, args.iw, args.sm_scale)
                    print(f"[Check] B={args.b}, heads={args.h}, S={S}, W={args.iw}, H={args.iw}, P={P}, D={args.d} | "
                          + " ".join(f"{n}:{chk[n + '_ok']}({chk[n + '_max']:.2e})" for n in ("out", "dq", "dk", "dv")),
                          flush=True)
                for provider in providers:
                    ms, peak = bench_point(provider, mode, q, k, v, coords, args.iw, args.iw, args.sm_scale,
                                           args.warmup, args.rep)
                    rows.append((mode, P, S, provider, ms, peak))
                    print(f"[Mem] provider={provider:6s} mode={mode:3s} | B={args.b} heads={args.h} S={S} W={args.iw} "
                          f"H={args.iw} P={P} D={args.d} | peak={peak:.1f} MB", file=log, flush=True)
                del q, k, v, coords
    log.close()
    _native.set_path(prev_path)
    write_csv_tables(rows, args, providers, S_LIST, P_LIST)
    for mode in ("fwd", "bwd"):
        print(f"\nlatency (ms), mode={mode}, B={args.b} H={args.h} D={args.d} W={args.iw} dtype={args.dtype}")
        print("  P   S " + " ".join(f"{p:>12s}" for p in providers) + "   peak MB " + " ".join(f"{p:>10s}" for p in providers))
        for P in P_LIST:
            for S in S_LIST:
                ms = {r[3]: r[4] for r in rows if r[:3] == (mode, P, S)}
                pk = {r[3]: r[5] for r in rows if r[:3] == (mode, P, S)}
                print(f"{P:3d} {S:3d} " + " ".join(f"{ms[p]:12.4f}" for p in providers) + "           "
                      + " ".join(f"{pk[p]:10.1f}" for p in providers))
    return rows


if __name__ == "__main__":
    main()
