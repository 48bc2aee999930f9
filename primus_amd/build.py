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
SOURCES = ["mx_quantize.hip", "mx_gemm.hip", "mx_gemm_bf16.hip", "mx_activation.hip", "mx_norm.hip", "mx_pad.hip", "mx_blockwise.hip", "mx_calibrate.hip", "mx_shuffle.hip"]

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
    """Compile every HIP source (one hipcc process per file, side by side) and link primus_amd/lib/libmxlinear.so;
    returns its path."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = hipcc_path()
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]

    def compile_one(src: str):
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *compile_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        return obj, subprocess.run(cmd, capture_output=True, text=True)

    workers = max(1, min(len(SOURCES), os.cpu_count() or 1, 8))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        results = list(pool.map(compile_one, SOURCES))
    for obj, res in results:
        if res.returncode != 0:
            sys.stderr.write(res.stdout + res.stderr)
            raise RuntimeError("hipcc failed compiling %s" % os.path.basename(obj))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[obj for obj, _ in results], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed linking libmxlinear.so")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
