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
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(st) == 0
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


def _inputs(rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    dev = torch.device("cuda:0")
    x = torch.randn(rows, k, generator=g).bfloat16().to(dev)
    dy = torch.randn(rows, k, generator=g).bfloat16().to(dev)
    w = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(dev)
    rstd = torch.empty(rows, dtype=torch.float32, device=dev)
    return x, dy, w, rstd


def test_noalloc_serves_one_stream_per_device_and_rebinds():
    """All calls on a GPU share the static array: a call on a stream other than the bound one is refused
    (MXL_ESTREAM, nothing launched) until the caller rebinds the entry point."""
    lib = _lib.load()
    rows, k = 64, 512
    x, dy, w, rstd = _inputs(rows, k, 11)
    main = torch.cuda.current_stream()
    st = ctypes.c_void_p(main.cuda_stream)
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(st) == 0
    assert lib.mxl_rmsnorm_fwd(_ptr(x), _ptr(w), ctypes.c_float(1e-5), rows, k, None, _ptr(rstd), st) == 0
    dx0, dw0 = torch.empty_like(x), torch.empty_like(w)
    assert lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx0), _ptr(dw0), st) == 0
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    st2 = ctypes.c_void_p(side.cuda_stream)
    dx1, dw1 = torch.full_like(x, 7.0), torch.full_like(w, 7.0)
    rc = lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx1), _ptr(dw1), st2)
    torch.cuda.synchronize()
    assert rc == -5 and b"stream" in lib.mxl_error_string(rc)
    assert bool((dx1 == 7.0).all()) and bool((dw1 == 7.0).all())
    # rebinding (the first stream's work is finished: synchronised above) moves the entry point to the side stream
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(st2) == 0
    assert lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx1), _ptr(dw1), st2) == 0
    assert lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx0), _ptr(dw0), st) == -5
    torch.cuda.synchronize()
    assert torch.equal(dx0.view(torch.int16), dx1.view(torch.int16)) and torch.equal(dw0.view(torch.int16), dw1.view(torch.int16))
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(st) == 0     # leave it on the main stream for whoever comes next


def test_noalloc_under_graph_capture_replays_bit_identically():
    """The entry point's reason to exist: a captured backward (bound to the capturing stream beforehand) replays on
    new inputs, with eager work between the replays, and every replay equals the workspace entry point."""
    lib = _lib.load()
    rows, k = 200, 1024
    x, dy, w, rstd = _inputs(rows, k, 21)
    dev = x.device
    dx_g, dw_g = torch.empty_like(x), torch.empty_like(w)
    cap = torch.cuda.Stream()
    cst = ctypes.c_void_p(cap.cuda_stream)
    cap.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(cst) == 0          # set-up belongs in front of the capture
    with torch.cuda.graph(graph, stream=cap):
        assert lib.mxl_rmsnorm_fwd(_ptr(x), _ptr(w), ctypes.c_float(1e-5), rows, k, None, _ptr(rstd), cst) == 0
        assert lib.mxl_rmsnorm_bwd_noalloc(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), rows, k, _ptr(dx_g), _ptr(dw_g), cst) == 0
    nbytes = lib.mxl_rmsnorm_bwd_workspace_bytes(rows, k)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for seed in (22, 23, 24):
        nx, ndy, nw, _ = _inputs(rows, k, seed)
        x.copy_(nx), dy.copy_(ndy), w.copy_(nw)
        dx_g.fill_(3.0), dw_g.fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        dx_e, dw_e, rstd_e = torch.empty_like(x), torch.empty_like(w), torch.empty_like(rstd)
        assert lib.mxl_rmsnorm_fwd(_ptr(x), _ptr(w), ctypes.c_float(1e-5), rows, k, None, _ptr(rstd_e), st) == 0
        assert lib.mxl_rmsnorm_bwd(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd_e), rows, k, _ptr(dx_e), _ptr(dw_e), _ptr(ws), nbytes, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(dx_g.view(torch.int16), dx_e.view(torch.int16)), seed
        assert torch.equal(dw_g.view(torch.int16), dw_e.view(torch.int16)), seed
    assert lib.mxl_rmsnorm_bwd_noalloc_bind(st) == 0
