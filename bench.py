#!/usr/bin/env python3
"""Benchmark of the fused deformable multi-view SDPA operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--all] [--no-cpu]

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

Per-workload details (forward alone, backward alone, all five shapes with --all)
go to stderr and, with --details FILE, as JSON into that file.
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


# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs), each counter
# scaled by its reading for a plain 256 MiB copy: FETCH x 2.000, WRITE x 1.000. Source and commands:
# profiles/hbm_traffic_C2.md. Only the kernels of the bench workload were measured.
MEASURED_TRAFFIC_BYTES = {
    "C2": {
        "fwd": int((35033.1 * 2.0 + 4009.5) * 1024),
        "bwd_dq": int((38971.0 * 2.0 + 3888.0) * 1024),
        "bwd_dkdv": int((42852.5 * 2.0 + 110976.0) * 1024),
    },
}


KERNEL_SAMPLE_EVERY = 10     # one step in ten of the timed region carries the per-kernel events


def load_traffic(workload, which):
    """Measured HBM bytes per launch of a kernel of a workload, or None when it was not measured."""
    return MEASURED_TRAFFIC_BYTES.get(workload, {}).get(which)


def measure_gpu(wl, steps, warmup):
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

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # The timed region: exactly `steps` steps. Every KERNEL_SAMPLE_EVERY-th of them runs with the library's
    # kernel timer on (HIP events attached to the kernel dispatches on the launch stream): a timed launch
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
    kern = {}
    for which, name in enumerate(("fwd", "bwd_dkdv", "bwd_dq", "bwd_bin", "desc_table")):
        ms, n = _native.timer_collect(which)
        kern[name] = {"ms": ms / max(n, 1), "launches": n, "per_step": n / max(timed_steps, 1)}
    ms_step = (t1 - t0) * 1e3 / steps

    # forward alone (no autograd graph), timed separately
    with torch.no_grad():
        for _ in range(max(2, warmup // 2)):
            deform_sdpa_triton(q, k, v, coords, W, Hh, scale)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            deform_sdpa_triton(q, k, v, coords, W, Hh, scale)
        torch.cuda.synchronize()
        fwd_only_ms = (time.perf_counter() - t0) * 1e3 / steps

    # the three main kernels one after the other on one stream (in the timed region above the backward's
    # dq and dk/dv kernels share the GPU, which stretches both)
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
    alone = {}
    for which, name in enumerate(("fwd", "bwd_dkdv", "bwd_dq", "bwd_bin", "desc_table")):
        ms, n = _native.timer_collect(which)
        alone[name] = ms / max(n, 1)

    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    step()
    torch.cuda.synchronize()
    peak_extra = torch.cuda.max_memory_allocated() - base
    return {
        "ms_per_step": ms_step,
        "fwd_only_ms": fwd_only_ms,
        "kernels": kern,
        "kernels_single_stream_ms": alone,
        "peak_extra_bytes": int(peak_extra),
    }


def measure_cpu(wl, budget_s=25.0):
    """Host-CPU PyTorch path on the same workload; bounded to about budget_s seconds."""
    import torch
    from oracle.torch_eager import eager_fwd_bwd
    from workloads import gen_inputs

    q, k, v, coords, dout = gen_inputs(wl)
    threads = torch.get_num_threads()
    chunked = wl.query_samples * wl.D * 8 > 8e9       # sampled K~+V~ above 8 GB: one (b, h) at a time
    f = lambda: eager_fwd_bwd(q.float(), k.float(), v.float(), coords, dout.float(),
                              wl.W_IMG, wl.H_IMG, wl.sm_scale, chunked=chunked)
    t0 = time.perf_counter()
    f()                                                # warm-up
    warm = time.perf_counter() - t0
    reps = int(max(1, min(5, (budget_s - warm) // max(warm, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(reps):
        f()
    dt = (time.perf_counter() - t0) / reps
    return {
        "value": wl.query_samples / dt / 1e6,
        "unit": "M query*samples/s (fwd+bwd)",
        "cores": threads,
        "kind": "port",
        "sample": f"{wl.name} full workload, fwd+bwd, 1 warm-up + {reps} timed reps, "
                  f"{dt * 1e3:.0f} ms/step, os.cpu_count()={os.cpu_count()}"
                  + (", chunked over (batch, head)" if chunked else ""),
        "ms_per_step": dt * 1e3,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="C2")
    ap.add_argument("--all", action="store_true", help="also report the other workloads on stderr")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--details", default=None, help="also write the per-workload details as JSON into this file")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run a plain 256 MiB device copy a few times (known HBM traffic, used to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU; run with --gpus 1 "
                 "(the operator shards over (batch, head) with no exchange between the shards)")

    from workloads import WORKLOADS, oob_fractions
    wl = WORKLOADS[args.workload]
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

    # Per-kernel algorithmic (compulsory) bytes: every tensor the kernel must read or write, once.
    #   fwd      q,k,v read + out written + coords            = 4*N*e + C
    #   bwd_dq   q,k,v,out,dout read + dq written + coords    = 6*N*e + C
    #   bwd_dkdv q,k,v,dout read + dk,dv written + coords     = 6*N*e + C
    # (whole backward, each tensor once: 8*N*e + C; the per-row lse/delta side buffers are left out.)
    def kernel_bytes(w, name):
        n = w.rows * w.D * w.esize
        c = w.B * w.V * w.L * w.V * w.P * 8
        return {"fwd": 4 * n + c, "bwd_dq": 6 * n + c, "bwd_dkdv": 6 * n + c}[name]

    def kernel_report(w, gk):
        rep = {}
        for name in ("fwd", "bwd_dq", "bwd_dkdv"):
            ms = gk[name]["ms"]
            if gk[name]["launches"] == 0 or ms <= 0:
                continue
            ach = kernel_bytes(w, name) / (ms * 1e-3) / 1e9
            rep[name] = {"kernel_ms": ms, "algorithmic_bytes": kernel_bytes(w, name), "achieved": ach,
                         "frac": ach / HBM_PEAK_GBS}
        return rep

    rep = kernel_report(wl, g["kernels"])
    dominant = max(rep, key=lambda k: rep[k]["kernel_ms"])
    dom = rep[dominant]
    roofline = {
        "bound": "hbm", "kernel": dominant, "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": dom["frac"], "traffic": load_traffic(wl.name, dominant),
        "algorithmic_bytes": dom["algorithmic_bytes"], "kernel_ms": dom["kernel_ms"],
        # the same kernel with the GPU to itself (backward on one stream): it shares the CUs with the dq kernel
        # in the timed region
        "kernel_ms_one_stream": g["kernels_single_stream_ms"][dominant],
        "frac_one_stream": dom["algorithmic_bytes"] / (g["kernels_single_stream_ms"][dominant] * 1e-3) / 1e9
                           / HBM_PEAK_GBS if g["kernels_single_stream_ms"][dominant] > 0 else None,
    }
    # per step: every timed item once, except the table fill (once in the forward, once in the backward)
    kernels_ms = sum(v["ms"] * v["per_step"] for v in g["kernels"].values())
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

    all_details = {wl.name: details}
    if args.all:
        for name, w in WORKLOADS.items():
            if name == wl.name:
                continue
            gg = measure_gpu(w, max(5, args.steps // 5), max(2, args.warmup // 2))
            d = {"workload": name, "query_samples": w.query_samples, **gg,
                 "MQS_per_s": w.query_samples / (gg["ms_per_step"] * 1e-3) / 1e6,
                 "per_kernel": kernel_report(w, gg["kernels"]),
                 "fwd_bwd_frac_of_roofline_on_step_time":
                     w.algorithmic_bytes("fwd+bwd") / (gg["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 "coords_outside_image": oob_fractions(w)}
            log("[bench]", json.dumps(d))
            all_details[name] = d

    cpu = None
    if not args.no_cpu:
        cpu = measure_cpu(wl)
        log("[bench] cpu baseline", json.dumps(cpu))

    if args.details:
        with open(args.details, "w") as f:
            json.dump({"gpu": all_details, "cpu": cpu}, f, indent=1)

    line = {
        "metric": "fused fwd+bwd M query*samples/s (and % of HBM roofline), 1xMI355X vs host-CPU torch",
        "value": value, "unit": "M query*samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": g["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if wl.dtype == "fp32" else wl.dtype, "data": "synthetic",
        "config": {"workload": f"{wl.name}: B{wl.B} V{wl.V} H{wl.H} D{wl.D} {wl.H_IMG}x{wl.W_IMG} P{wl.P} "
                               f"{wl.dtype} coords={wl.coords}, fwd+bwd through the autograd operator",
                   "query_samples_per_step": qs,
                   "fwd_only_ms": g["fwd_only_ms"],
                   "kernel_ms": {k: round(v["ms"], 5) for k, v in g["kernels"].items()},
                   "kernel_ms_one_stream": {k: round(v, 5) for k, v in g["kernels_single_stream_ms"].items()},
                   "fwd_bwd_frac_of_hbm_roofline_on_step_time": details["fwd_bwd_frac_of_roofline_on_step_time"],
                   "peak_extra_bytes": g["peak_extra_bytes"]},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
