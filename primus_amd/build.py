"""Builds the HIP extension (libmxlinear.so) for gfx950 with hipcc.

The library is a plain C-ABI shared object (see include/mxlinear.h); it is
built in-tree so that it travels with the source tree to machines that have a
GPU but no compiler step in their test run.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmxlinear.so")
SOURCES = ["mx_quantize.hip", "mx_gemm.hip", "mx_activation.hip", "mx_norm.hip", "mx_pad.hip", "mx_blockwise.hip", "mx_calibrate.hip", "mx_shuffle.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 arithmetic is kept off on purpose (target feature of the device pass)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the MX linear path needs the ROCm compiler to build")


def build(verbose: bool = False) -> str:
    """Compile every HIP source into primus_amd/lib/libmxlinear.so; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building libmxlinear.so")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
