#!/usr/bin/env python3
"""Benchmark of the fused deformable multi-view SDPA operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C5] [--only] [--no-cpu]

A "step" is one forward + backward pass of the public operator
(`deform_sdpa_triton`, autograd) over one batch of the workload, inputs already
resident in HBM. Prints ONE JSON line on stdout:

  metric/value   M query.samples/s of fwd+bwd (query.samples = B*V*H*L * V*P)
  roofline       the dominant (longest) kernel against the 8 TB/s HBM roofline on its
                 own algorithmic (compulsory) bytes; its average duration is measured
                 here with HIP events recorded by the library around that kernel
                 on the launch stream, during the timed steps
  cpu_baseline   the same workload through the host-CPU PyTorch path
                 (grid_sample + softmax, oracle/torch_eager.py), same run

The headline workload is C5, the largest of the five named shapes. The other four
are measured in the same run (a shorter leg each; --only skips them) and reported
as flat, short keys inside "config": c1_ms (fwd+bwd step), c1_gqs (G query.samples/s),
c1_frac (fwd+bwd compulsory bytes / step time / 8 TB/s), c1_kfrac (the same for the
workload's longest kernel on that kernel's own bytes and duration); cg_ms is the headline
workload's step with the optional gradient of the coordinates switched on.
Per-workload details go to stderr and, with --details FILE, as JSON into that file.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "fused-deform-multi-head-scaled-dot-product-attention-triton_amd")
for _p in (ROOT, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0     # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs per workload), each
# counter scaled by its reading for a plain 256 MiB copy in the same run. The figures, the scale factors and
# the commands are in profiles/hbm_traffic_*.md; profiles/traffic.json holds the bytes per launch by workload
# and kernel, and is rewritten whenever the counters are collected again.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


KERNEL_SAMPLE_EVERY = 10     # one step in ten of the timed region carries the per-kernel events
KERNEL_SLOTS = ("fwd", "bwd_dkdv", "bwd_dq", "bwd_bin", "desc_table")     # the library timer's slots 0..4


def load_traffic(workload, which):
    """Measured HBM bytes per launch of a kernel of a workload, or None when it was not measured."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    v = table.get(workload, {}).get(which)
    return int(v) if v is not None else None


def measure_gpu(wl, steps, warmup, extras=True):
    import torch
    from ops import _native
    from ops.triton import deform_sdpa_triton
    from workloads import gen_inputs

    dev = torch.device("cuda:0")
    q, k, v, coords, dout = gen_inputs(wl, device=dev)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    W, Hh, scale = wl.W_IMG, wl.H_IMG, wl.sm_scale

    def step():
        q.grad = k.grad = v.grad = None
        out = deform_sdpa_triton(q, k, v, coords, W, Hh, scale)
        out.backward(dout)

    def collect(timed_steps):
        # per kernel: "ms" = busy time per step (the binning's three launches added up, the two table
        # fills of a step added up), "launches_per_step"
        res = {}
        for which, name in enumerate(KERNEL_SLOTS):
            ms, n = _native.timer_collect(which)
            res[name] = {"ms": ms / max(timed_steps, 1), "launches_per_step": n / max(timed_steps, 1)}
        return res

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # The timed region: exactly `steps` steps. Every KERNEL_SAMPLE_EVERY-th of them runs with the library's
    # kernel timer on (HIP events attached to the kernel dispatches on the launch streams): a timed launch
    # costs a few microseconds of GPU idle time, which sampling keeps below 1 % of the region.
    timed_steps = 0
    t0 = time.perf_counter()
    for i in range(steps):
        sample = i % KERNEL_SAMPLE_EVERY == 0
        if sample:
            _native.timer_enable(True)
            timed_steps += 1
        step()
        if sample:
            _native.timer_enable(False)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kern = collect(timed_steps)
    ms_step = (t1 - t0) * 1e3 / steps
    res = {"ms_per_step": ms_step, "kernels": kern}
    if not extras:
        return res

    # forward alone (no autograd graph), timed separately
    with torch.no_grad():
        for _ in range(max(2, warmup // 2)):
            deform_sdpa_triton(q, k, v, coords, W, Hh, scale)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            deform_sdpa_triton(q, k, v, coords, W, Hh, scale)
        torch.cuda.synchronize()
        res["fwd_only_ms"] = (time.perf_counter() - t0) * 1e3 / steps

    # the main kernels one after the other on one stream (in the timed region above the backward's dq and
    # dk/dv sides share the GPU where both leave room, which stretches both)
    import ops.triton as op_module
    op_module.SINGLE_STREAM = True
    try:
        step()
        torch.cuda.synchronize()
        _native.timer_enable(True)
        for _ in range(5):
            step()
        torch.cuda.synchronize()
        _native.timer_enable(False)
    finally:
        op_module.SINGLE_STREAM = False
    res["kernels_single_stream_ms"] = {name: v["ms"] for name, v in collect(5).items()}

    # the same step with the gradient of the coordinates as well (the operator's optional eighth argument; the
    # reference's fused operator has none, its eager one gets it through grid_sample)
    cg = coords.clone().requires_grad_(True)

    def step_cg():
        q.grad = k.grad = v.grad = cg.grad = None
        deform_sdpa_triton(q, k, v, cg, W, Hh, scale, True).backward(dout)

    for _ in range(3):
        step_cg()
    torch.cuda.synchronize()
    n_cg = max(5, steps // 2)
    t0 = time.perf_counter()
    for _ in range(n_cg):
        step_cg()
    torch.cuda.synchronize()
    res["coords_grad_ms_per_step"] = (time.perf_counter() - t0) * 1e3 / n_cg
    cg.grad = None
    del cg

    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    step()
    torch.cuda.synchronize()
    res["peak_extra_bytes"] = int(torch.cuda.max_memory_allocated() - base)
    return res


def measure_cpu(wl, budget_s=25.0):
    """Host-CPU PyTorch path (grid_sample + softmax + autograd) on a bounded sample of the workload.

    Batches and heads are independent and the coordinates are shared by the heads, so the workload is
    B*H equal (batch, head) chunks; the eager path is run chunk by chunk (which also bounds its memory: it
    materialises 2*QS*D*4 bytes of sampled K and V per chunk) for about budget_s seconds, and the rate is
    the query.samples of the chunks done over the time they took."""
    import torch
    from oracle.torch_eager import eager_fwd_bwd
    from workloads import gen_inputs

    q, k, v, coords, dout = gen_inputs(wl)
    threads = torch.get_num_threads()
    chunks = [(b, h) for b in range(wl.B) for h in range(wl.H)]
    qs_chunk = wl.query_samples // len(chunks)

    def run_chunk(b, h):
        sl = lambda t: t[b:b + 1, :, h:h + 1].float()
        eager_fwd_bwd(sl(q), sl(k), sl(v), coords[b:b + 1], sl(dout), wl.W_IMG, wl.H_IMG, wl.sm_scale)

    t0 = time.perf_counter()
    run_chunk(*chunks[-1])                             # warm-up
    warm = time.perf_counter() - t0
    done, t0 = 0, time.perf_counter()
    for (b, h) in chunks:
        run_chunk(b, h)
        done += 1
        if time.perf_counter() - t0 + warm > budget_s:
            break
    dt = time.perf_counter() - t0
    return {
        "value": done * qs_chunk / dt / 1e6,
        "unit": "M query*samples/s (fwd+bwd)",
        "cores": threads,
        "kind": "port",
        "sample": f"{wl.name}: {done} of its {len(chunks)} (batch, head) chunks ({done * qs_chunk} of "
                  f"{wl.query_samples} query*samples), fwd+bwd through ATen grid_sample + softmax + autograd, "
                  f"after 1 warm-up chunk; {dt / done * 1e3:.0f} ms per chunk, os.cpu_count()={os.cpu_count()}",
        "ms_per_step_extrapolated": dt / done * len(chunks) * 1e3,
    }


# Per-kernel algorithmic (compulsory) bytes: every tensor the kernel must read or write, once.
#   fwd      q,k,v read + out written + coords            = 4*N*e + C
#   bwd_dq   q,k,v,out,dout read + dq written + coords    = 6*N*e + C
#   bwd_dkdv q,k,v,dout read + dk,dv written + coords     = 6*N*e + C
# (whole backward, each tensor once: 8*N*e + C; the per-row lse/delta side buffers are left out.) One launch
# processes all B*V*H*L * V*P query.samples of the workload.
def kernel_bytes(w, name):
    n = w.rows * w.D * w.esize
    c = w.B * w.V * w.L * w.V * w.P * 8
    return {"fwd": 4 * n + c, "bwd_dq": 6 * n + c, "bwd_dkdv": 6 * n + c}[name]


def kernel_report(w, gk):
    rep = {}
    for name in ("fwd", "bwd_dq", "bwd_dkdv"):
        ms = gk[name]["ms"]
        if gk[name]["launches_per_step"] == 0 or ms <= 0:
            continue
        ach = kernel_bytes(w, name) / (ms * 1e-3) / 1e9
        rep[name] = {"kernel_ms": ms, "algorithmic_bytes": kernel_bytes(w, name), "achieved": ach,
                     "frac": ach / HBM_PEAK_GBS}
    return rep


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C5", help="the headline workload (default: C5, the largest)")
    ap.add_argument("--only", action="store_true", help="measure the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--details", default=None, help="also write the per-workload details as JSON into this file")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run a plain 256 MiB device copy a few times (known HBM traffic, used to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU; run with --gpus 1 "
                 "(the operator shards over (batch, head) with no exchange between the shards)")

    from workloads import WORKLOADS, find_workload, oob_fractions
    wl = find_workload(args.workload)            # (one of the five named shapes, or an extra one such as C5c)
    if args.copy_calibration:
        import torch
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    g = measure_gpu(wl, args.steps, args.warmup)
    qs = wl.query_samples
    value = qs / (g["ms_per_step"] * 1e-3) / 1e6

    rep = kernel_report(wl, g["kernels"])
    dominant = max(rep, key=lambda k: rep[k]["kernel_ms"])
    dom = rep[dominant]
    alone_ms = g["kernels_single_stream_ms"][dominant]
    roofline = {
        "bound": "hbm", "kernel": dominant, "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": dom["frac"], "traffic": load_traffic(wl.name, dominant),
        # A kernel may cover the workload in several launches (the backward of the larger shapes goes group by
        # group of (batch, head) pairs; the forward may be a dense-box launch plus a gather launch for the tiles it
        # declines): bytes, traffic and kernel_ms are then the sums over the launches of one step, so that
        # achieved = bytes per launch / average launch duration all the same.
        "launches_per_step": g["kernels"][dominant]["launches_per_step"],
        "algorithmic_bytes": dom["algorithmic_bytes"], "kernel_ms": dom["kernel_ms"],
        # the same kernel with the backward on one stream (in the timed region the backward's two sides run
        # on two streams and share the CUs where both leave room)
        "kernel_ms_one_stream": alone_ms,
        "frac_one_stream": dom["algorithmic_bytes"] / (alone_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if alone_ms > 0 else None,
    }
    kernels_ms = sum(v["ms"] for v in g["kernels"].values())
    details = {
        "workload": wl.name, "query_samples": qs, **g, "per_kernel": rep,
        "fwd_only_MQS_per_s": qs / (g["fwd_only_ms"] * 1e-3) / 1e6,
        "all_kernels_ms": kernels_ms,
        "fwd_bwd_frac_of_roofline_on_kernel_time":
            wl.algorithmic_bytes("fwd+bwd") / (kernels_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "fwd_bwd_frac_of_roofline_on_step_time":
            wl.algorithmic_bytes("fwd+bwd") / (g["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "coords_outside_image": oob_fractions(wl),
    }
    log("[bench]", json.dumps(details))

    # the other named workloads, a shorter leg each: flat keys (nested objects do not survive every reader)
    all_details = {wl.name: details}
    others = {}
    if not args.only:
        for name, w in WORKLOADS.items():
            if name == wl.name:
                continue
            n_steps = 100 if w.query_samples < 2e7 else 40    # these steps take 0.4 - 6 ms
            gg = measure_gpu(w, n_steps, 10, extras=False)
            r = kernel_report(w, gg["kernels"])
            dk = max(r, key=lambda k: r[k]["kernel_ms"])
            d = {"workload": name, "query_samples": w.query_samples, **gg, "per_kernel": r,
                 "MQS_per_s": w.query_samples / (gg["ms_per_step"] * 1e-3) / 1e6,
                 "fwd_bwd_frac_of_roofline_on_step_time":
                     w.algorithmic_bytes("fwd+bwd") / (gg["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS}
            log("[bench]", json.dumps(d))
            all_details[name] = d
            key = name.lower()
            others[key + "_ms"] = round(gg["ms_per_step"], 4)
            others[key + "_gqs"] = round(d["MQS_per_s"] / 1e3, 3)
            others[key + "_frac"] = round(d["fwd_bwd_frac_of_roofline_on_step_time"], 5)
            others[key + "_kfrac"] = round(r[dk]["frac"], 5)
            others[key + "_kernel"] = dk
            others[key + "_fwd_ms"] = round(gg["kernels"]["fwd"]["ms"], 4)

    cpu = None
    if not args.no_cpu:
        cpu = measure_cpu(wl)
        log("[bench] cpu baseline", json.dumps(cpu))

    if args.details:
        with open(args.details, "w") as f:
            json.dump({"gpu": all_details, "cpu": cpu}, f, indent=1)

    config = {"workload": f"{wl.name}: B{wl.B} V{wl.V} H{wl.H} D{wl.D} {wl.H_IMG}x{wl.W_IMG} P{wl.P} "
                          f"{wl.dtype} coords={wl.coords}, fwd+bwd through the autograd operator",
              "query_samples_per_step": qs,
              "fwd_only_ms": round(g["fwd_only_ms"], 5),
              "step_frac": round(details["fwd_bwd_frac_of_roofline_on_step_time"], 5),
              "peak_extra_bytes": g["peak_extra_bytes"],
              "cg_ms": round(g["coords_grad_ms_per_step"], 4)}      # fwd+bwd step that also returns d loss / d coords
    for name, v in g["kernels"].items():
        config["k_" + name + "_ms"] = round(v["ms"], 5)
    for name, v in g["kernels_single_stream_ms"].items():
        config["k1_" + name + "_ms"] = round(v, 5)
    config.update(others)
    line = {
        "metric": "fused fwd+bwd M query*samples/s (and % of HBM roofline), 1xMI355X vs host-CPU torch",
        "value": value, "unit": "M query*samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": g["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if wl.dtype == "fp32" else wl.dtype, "data": "synthetic",
        "config": config,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
