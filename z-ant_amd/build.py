"""Builds libzant_hip.so (the product) for gfx950 with hipcc.  Cross-compiles without a GPU.

Usage: python z-ant_amd/build.py            (from the repository root)
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libzant_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # never let the compiler form packed-f32 VALU ops; rounding of a*b+c stays two-step everywhere
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
    "-Wall", "-Wno-unused-function",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


HOST_TEST = os.path.join(HERE, "host", "test_host_mirror")


OBJ = os.path.join(HERE, "_obj")  # per-source objects (not tracked); every build recompiles all of them


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        jobs.append((obj, [HIPCC] + FLAGS + ["-c", src, "-o", obj]))

    def run(job):
        if verbose:
            print(" ".join(job[1]), flush=True)
        subprocess.check_call(job[1])
        return job[0]

    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:  # one translation unit per core
        objs = list(pool.map(run, jobs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # the C++ host mirror of the reference's operator interface: plain g++ over the C ABI (no HIP headers)
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
           os.path.join(HERE, "host", "test_host_mirror.cpp"), "-o", HOST_TEST, "-L", HERE, "-lzant_hip",
           "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
