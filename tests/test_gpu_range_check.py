"""The hardware rule behind the GEMM kernels' memory safety, pinned on the device.

The kernels request whole 256-row tiles through raw buffer descriptors that end with the operand and rely on the
range check to drop whatever lies past it.  Part of a request's offset travels in the per-lane register, part in the
scalar offset; this test shows that gfx950 checks their SUM against num_records, dword by dword, that a dropped dword
arrives as zero in LDS, and that a scalar offset beyond num_records does not wrap around.  Every case stays inside
one 64 KiB buffer, so no outcome could touch foreign memory.  ``tests/test_gemm_bounds.py`` then walks every request
of the kernels under exactly this rule on the host.
"""
import ctypes

import numpy as np
import pytest
import torch

from primus_amd import _lib

pytestmark = pytest.mark.gpu


def test_range_check_covers_per_lane_and_scalar_offset(gpu):
    lib = _lib.load()
    words = 16384
    buf = (torch.arange(words, dtype=torch.int32, device=gpu) + 1)          # word i holds i + 1: never zero
    cases = [
        # (voff, soff, records), what is expected to arrive
        (16, 0, 64, "in"), (64, 0, 64, "out"), (56, 0, 64, "half"),
        (16, 32, 64, "in"), (40, 32, 64, "out"),            # 40 + 32 >= 64: the scalar offset counts
        (16, 64, 64, "out"), (16, 128, 64, "out"),          # scalar offset at / beyond num_records: no wrap-around
        (0, 4096, 64, "out"), (16, 4096, 4096, "out"), (16, 4096, 8192, "in"),
        (4088, 4096, 8192, "half"), (4096, 4096, 8192, "out"), (16, 8192, 8192, "out"), (16, 32768, 8192, "out"),
        (0, 0, 0, "out"), (0, 16, 0xFFFFFFFF, "in"),
        (16, 32, 52, "first"), (16, 32, 51, "out"), (16, 32, 48, "out"),      # a dword needs all four of its bytes
    ]
    arr = np.array([c[:3] for c in cases], dtype=np.uint32)
    dc = torch.from_numpy(arr.view(np.int32).copy()).to(gpu)
    out = torch.full((len(cases) * 4,), -1, dtype=torch.int32, device=gpu)
    top = int(max(int(c[0]) + int(c[1]) for c in cases))
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.mxl_calibrate_range_check(ctypes.c_void_p(buf.data_ptr()), words * 4, ctypes.c_void_p(dc.data_ptr()), len(cases),
                                       ctypes.c_void_p(out.data_ptr()), top, st)
    assert rc == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint32).reshape(len(cases), 4)
    for (voff, soff, rec, kind), g in zip(cases, got):
        w0 = (voff + soff) // 4 + 1
        want = {"in": [w0, w0 + 1, w0 + 2, w0 + 3], "out": [0, 0, 0, 0], "half": [w0, w0 + 1, 0, 0], "first": [w0, 0, 0, 0]}[kind]
        assert list(g) == want, (voff, soff, rec, kind, list(g))
    # the entry point refuses cases that could leave the buffer
    assert lib.mxl_calibrate_range_check(ctypes.c_void_p(buf.data_ptr()), 4096, ctypes.c_void_p(dc.data_ptr()), len(cases),
                                         ctypes.c_void_p(out.data_ptr()), top, st) == -1
