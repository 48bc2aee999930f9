"""Every operand request of the GEMM kernels stays inside its operand.

The kernels take the address arithmetic of their LDS-direct loads from ``primus_amd/csrc/mx_gemm_addr.h``;
``tests/gemm_bounds_check.cpp`` includes the same header, built here for the host with g++, and walks every request
of a tile (all threads, load rounds and K slots, the look-ahead slots past the contraction range included, tiles
starting at any row) under the hardware's range-check rule (both offsets of a request are checked against
num_records, dword by dword; ``tests/test_gpu_range_check.py`` pins that rule on the device).  No GPU is involved
here: an out-of-bounds read is shown by arithmetic, not by a fault.
"""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def test_every_accepted_request_is_inside_the_operand(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no host compiler")
    exe = str(tmp_path / "gemm_bounds_check")
    subprocess.run([gxx, "-O2", "-std=c++17", "-Wall", "-Werror", os.path.join(HERE, "gemm_bounds_check.cpp"), "-o", exe], check=True)
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert " 0 failures" in res.stdout, res.stdout
