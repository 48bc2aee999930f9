"""The allocation-free RMSNorm backward (static device scratch) against the entry point that takes a workspace:
two calls in a row through the C ABI, the second on a smaller input; results must be bit-identical."""

import ctypes

import pytest
import torch

from primus_amd import _lib

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    dev = torch.device("cuda:0")
    x = torch.randn(rows, k, generator=g).bfloat16().to(dev)
    dy = torch.randn(rows, k, generator=g).bfloat16().to(dev)
    w = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(dev)
    rstd = torch.empty(rows, dtype=torch.float32, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.mxl_rmsnorm_fwd(_ptr(x), _ptr(w), ctypes.c_float(1e-5), rows, k, None, _ptr(rstd), st) == 0
    nbytes = lib.mxl_rmsnorm_bwd_workspace_bytes(rows, k)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    dx_a, dw_a = torch.empty_like(x), torch.empty_like(w)
    dx_b, dw_b = torch.full_like(x, 7.0), torch.full_like(w, 7.0)
    assert lib.mxl_rmsnorm_bwd(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx_a), _ptr(dw_a), _ptr(ws), nbytes, st) == 0
    rc = lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx_b), _ptr(dw_b), st)
    torch.cuda.synchronize()
    return rc, (dx_a, dw_a), (dx_b, dw_b), nbytes


def test_noalloc_matches_workspace_entry_point_twice():
    lib = _lib.load()
    limit = lib.mxl_rmsnorm_bwd_noalloc_max_bytes()
    assert limit == 8 << 20
    # first a problem that fills most of the static array, then a smaller one (the array keeps the first call's sums)
    for rows, k, seed in ((900, 2048, 1), (37, 512, 2), (0, 256, 3)):
        rc, (dx_a, dw_a), (dx_b, dw_b), nbytes = _both(lib, rows, k, seed)
        assert nbytes <= limit and rc == 0, (rows, k, rc)
        assert torch.equal(dx_a.view(torch.int16), dx_b.view(torch.int16)), (rows, k)
        assert torch.equal(dw_a.view(torch.int16), dw_b.view(torch.int16)), (rows, k)


def test_noalloc_refuses_what_does_not_fit():
    lib = _lib.load()
    assert lib.mxl_rmsnorm_bwd_workspace_bytes(4096, 4096) > lib.mxl_rmsnorm_bwd_noalloc_max_bytes()
    rc, _, (dx_b, dw_b), _ = _both(lib, 4096, 4096, 4)
    assert rc == -4                                            # MXL_ESCRATCH, and nothing was written
    assert bool((dx_b == 7.0).all()) and bool((dw_b == 7.0).all())
    assert b"scratch" in lib.mxl_error_string(rc)
    assert lib.mxl_rmsnorm_bwd_noalloc(None, None, None, None, 4, 100, None, None, None) == -1   # k % 8
