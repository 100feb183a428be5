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
SRC = os.path.join(HERE, "csrc", "dsdpa_api.hip")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libdsdpa.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-munsafe-fp-atomics",                       # hardware float atomics (global_atomic_add_f32 / ds_add_f32)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build_library(verbose=True, extra_flags=()):
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, SRC, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip() and verbose:
        print(out)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return LIB


if __name__ == "__main__":
    build_library(extra_flags=sys.argv[1:])
