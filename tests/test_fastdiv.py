"""The multiply-high division the kernels decode indices with, checked on the CPU against plain integer division."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_fixed_divisor_division_is_exact_below_2_pow_31(tmp_path):
    exe = str(tmp_path / "fastdiv_check")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "z-ant_amd", "csrc"),
                           os.path.join(ROOT, "tests", "fastdiv_check.cpp"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout
    assert " bad 0" in out.stdout
