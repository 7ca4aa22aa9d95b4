"""Builds libzant_hip.so (the product) for gfx950 with hipcc.  Cross-compiles without a GPU.

Usage: python z-ant_amd/build.py            (from the repository root)
"""
import glob
import os
import re
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


# sources whose kernels hide LDS reads from the compiler (checked for spills at build time, see build())
NO_SPILL_SOURCES = {"qconv_ps_i8.hip", "qblock_i8.hip", "qconv_i8.hip", "conv_f32.hip", "gemm_f32.hip"}

# kernels whose hand-written stores take their bases from scalar registers: a scalar spill reloaded (v_readlane) right
# in front of such a store would need wait states the compiler cannot count through inline asm
NO_SGPR_SPILL_KERNELS = ("conv_f32_c1k3_pool_mfma_kernel",)

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
        if os.path.basename(job[1][-3]) not in NO_SPILL_SOURCES:
            subprocess.check_call(job[1])
            return job[0]
        # These sources issue LDS reads the compiler does not see and wait for them by hand.  A register that is in
        # flight between such a read and its wait must not be copied: a spill to scratch taken in that window saves
        # garbage.  So a kernel of these files that spills fails the build.
        res = subprocess.run(job[1] + ["-Rpass-analysis=kernel-resource-usage"], stderr=subprocess.PIPE, text=True)
        if res.returncode:
            sys.stderr.write(res.stderr)
            raise subprocess.CalledProcessError(res.returncode, job[1])
        name, bad = None, []
        for line in res.stderr.splitlines():
            m = re.search(r"remark: Function Name: (\S+)", line)
            if m:
                name = m.group(1)
            m = re.search(r"remark:\s+(VGPRs Spill): (\d+)", line)
            if m and name and int(m.group(2)) > 0 and "_kernel" in name:
                bad.append(f"{name}: {m.group(1)} = {m.group(2)}")
            m = re.search(r"remark:\s+(SGPRs Spill): (\d+)", line)
            if m and name and int(m.group(2)) > 0 and any(k in name for k in NO_SGPR_SPILL_KERNELS):
                bad.append(f"{name}: {m.group(1)} = {m.group(2)}")
        if bad:
            raise RuntimeError("kernels with hand-scheduled LDS reads or stores must not spill:\n  " + "\n  ".join(bad))
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
