"""Builds libdsdpa.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python build.py            # writes lib/libdsdpa.so next to this file

hipcc cross-compiles without a GPU. Packed-FP32 instruction selection is
switched off for the device pass (the host pass prints a harmless "not a
recognized feature" note for that flag).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRCS = [os.path.join(HERE, "csrc", n) for n in ("dsdpa_api.hip", "dsdpa_sort.hip", "dsdpa_f32.hip", "dsdpa_bf16.hip", "dsdpa_f16.hip")]
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libdsdpa.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-munsafe-fp-atomics",                       # hardware float atomics (global_atomic_add_f32 / ds_add_f32)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form",          # MFMA accumulators in VGPRs: no copies to and from AGPRs around the loops
    "-Wall", "-Wno-unused-function",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    return proc.returncode, out


def build_library(verbose=True, extra_flags=()):
    """Compile the translation units in parallel (one per storage type, the C ABI, the list sort) and link."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".o") for s in SRCS]
    cmds = [[hipcc, *HIPCC_FLAGS, *extra_flags, "-c", s, "-o", o] for s, o in zip(SRCS, objs)]
    if verbose:
        for c in cmds:
            print(" ".join(c), flush=True)
    with ThreadPoolExecutor(max_workers=len(cmds)) as pool:
        results = list(pool.map(_run, cmds))
    for (rc, out), c in zip(results, cmds):
        if out.strip() and verbose:
            print(out)
        if rc != 0:
            raise RuntimeError("hipcc failed: " + " ".join(c) + "\n" + out)
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(link), flush=True)
    rc, out = _run(link)
    if rc != 0:
        raise RuntimeError("link failed:\n" + out)
    return LIB


if __name__ == "__main__":
    build_library(extra_flags=sys.argv[1:])
