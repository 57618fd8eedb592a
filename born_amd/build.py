"""Builds born_amd/lib/libborn_rocm.so (the C-ABI library) with hipcc for gfx950.

Usage: python -m born_amd.build            (also called by __graft_entry__.build())
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libborn_rocm.so")
SOURCES = ["api.hip", "basic_kernels.hip", "topk_row.hip", "nucleus_row.hip", "sample_wide.hip", "spec_kernels.hip", "linear.hip", "tensor_ops.hip",
           "division.cpp"]          # .cpp: host code only

# -ffp-contract=off and correctly rounded fp32 division: every floating-point step of the
# fixed-point pipeline must be a single IEEE rounding, identical on host and device.
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
HOST_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-Wall"]


def hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
        if src.endswith(".cpp"):
            cmd = [hipcc()] + HOST_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        else:
            cmd = [hipcc()] + FLAGS + os.environ.get("BORN_EXTRA_HIPCC_FLAGS", "").split() + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(f"--- {src} failed:\n{out}", file=sys.stderr)
        elif verbose and out.strip():
            print(f"--- {src}:\n{out}")
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
