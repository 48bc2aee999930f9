"""The unquantised bf16 grouped GEMM (``ops.grouped_gemm``; reference call site
primus/backends/megatron/core/extensions/primus_turbo.py:2210-2216) against a per-expert fp32 matmul of the same bf16
inputs: forward, dgrad and wgrad, ``trans_b`` both ways, ragged and empty experts, main_grad accumulation, and a
graph capture replayed with new routing (the counts never leave the device).

Tolerance: the kernel accumulates in fp32 and rounds once to bf16, so against the fp32 reference the error is one
bf16 rounding of the result (2^-8 relative) plus the accumulation-order error, (k + 64) * 2^-23 * sum |a_i b_i|.
On small-integer operands every partial sum is exact and the comparison is bit for bit."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref(a, b, lens, trans_b):
    outs, off = [], 0
    for g, n in enumerate(lens):
        rows = a[off:off + n].float()
        w = b[g].float()
        outs.append(rows @ (w.t() if trans_b else w))
        off += n
    return torch.cat(outs, 0)


def _close(got, want, absdot, k):
    bound = 2.0 ** -8 * want.abs() + (k + 64) * 2.0 ** -23 * absdot + 1e-30
    bad = (got.float() - want).abs() > bound
    assert not bool(bad.any()), (int(bad.sum()), float(((got.float() - want).abs() / bound).max()))


CASES = [
    # lens, n, k
    ([100, 0, 37, 300], 320, 256),
    ([1, 129, 0, 0, 128, 255], 288, 96),          # n not a multiple of the 256-wide tile, nor of 128
    ([700], 512, 160),
    ([0, 0, 5], 32, 32),
    ([513, 256, 31], 2880, 64),
]


@pytest.mark.parametrize("lens,n,k", CASES)
@pytest.mark.parametrize("trans_b", [True, False])
def test_forward_and_gradients_match_fp32_matmul(gpu, lens, n, k, trans_b):
    import primus_amd.pytorch as turbo

    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(m * 7 + n + k)
    a = torch.randn(m, k, generator=gen).bfloat16().to(gpu).requires_grad_()
    b = (torch.randn(*((G, n, k) if trans_b else (G, k, n)), generator=gen) * 0.1).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(m, n, generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = turbo.ops.grouped_gemm(a, b, gl, trans_b=trans_b)
    y.backward(dy)
    assert y.dtype == torch.bfloat16 and y.shape == (m, n) and a.grad.shape == a.shape and b.grad.shape == b.shape
    ad, bd = a.detach(), b.detach()
    _close(y, _ref(ad, bd, lens, trans_b), _ref(ad.abs(), bd.abs(), lens, trans_b), k)
    _close(a.grad, _ref(dy, bd, lens, not trans_b), _ref(dy.abs(), bd.abs(), lens, not trans_b), n)
    off = 0
    for g, ln in enumerate(lens):
        x_g, d_g = ad[off:off + ln].float(), dy[off:off + ln].float()
        want = d_g.t() @ x_g if trans_b else x_g.t() @ d_g
        absd = d_g.abs().t() @ x_g.abs() if trans_b else x_g.abs().t() @ d_g.abs()
        _close(b.grad[g], want, absd, ln)
        if ln == 0:
            assert not bool(b.grad[g].any())
        off += ln


def test_exact_on_small_integers_and_rows_beyond_the_counts(gpu):
    """Integer operands: every product and partial sum is exact, so the result equals the fp32 matmul bit for bit;
    rows of ``a`` that the counts do not cover leave their output rows untouched."""
    from primus_amd.pytorch import kernels as K

    lens, n, k = [300, 0, 129, 200], 512, 1024
    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(5)
    a = torch.randint(-3, 4, (m + 50, k), generator=gen).bfloat16().to(gpu)
    b = torch.randint(-3, 4, (G, n, k), generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = K.grouped_gemm_bf16_impl(a, b, gl)
    want = _ref(a[:m], b, lens, True).bfloat16()
    assert torch.equal(y[:m], want)
    bt = b.transpose(1, 2).contiguous()
    assert torch.equal(K.grouped_gemm_bf16_impl(a, bt, gl, b_kn=True)[:m], want)
    dw = K.grouped_gemm_bf16_wgrad_impl(y[:m].contiguous() * 0 + a[:m, :n].contiguous(), a[:m].contiguous(), gl)
    off = 0
    for g, ln in enumerate(lens):
        p, q = a[off:off + ln, :n].float(), a[off:off + ln].float()
        assert torch.equal(dw[g], (p.t() @ q).bfloat16()), g
        off += ln


def test_wgrad_accumulates_into_main_grad(gpu):
    import primus_amd.pytorch as turbo

    lens, n, k = [64, 0, 200], 256, 128
    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(9)
    a = torch.randint(-2, 3, (m, k), generator=gen).bfloat16().to(gpu).requires_grad_()
    b = torch.randint(-2, 3, (G, n, k), generator=gen).bfloat16().to(gpu).requires_grad_()
    dy = torch.randint(-2, 3, (m, n), generator=gen).bfloat16().to(gpu)
    before = torch.randint(-100, 100, (G, n, k), generator=gen).float().to(gpu)
    b.main_grad = before.clone()
    b.grad_added_to_main_grad = False
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    turbo.ops.grouped_gemm(a, b, gl, trans_b=True, fuse_bgrad_accum_pattern="megatron").backward(dy)
    assert b.grad_added_to_main_grad
    off = 0
    for g, ln in enumerate(lens):
        want = before[g] + dy[off:off + ln].float().t() @ a.detach()[off:off + ln].float()
        assert torch.equal(b.main_grad[g], want), g
        off += ln


def test_replays_under_a_graph_with_new_routing(gpu):
    import primus_amd.pytorch as turbo

    G, n, k, rows = 4, 384, 256, 700
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(rows, k, generator=gen).bfloat16().to(gpu).requires_grad_()
    w = (torch.randn(G, n, k, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(rows, n, generator=gen).bfloat16().to(gpu)
    lens = torch.tensor([100, 0, 343, 257], dtype=torch.int64, device=gpu)

    def step():
        y = turbo.ops.grouped_gemm(x, w, lens)
        dx, dw = torch.autograd.grad(y, [x, w], dy)
        return y, dx, dw

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for new_lens, seed in (([0, 0, 0, 700], 2), ([175, 175, 175, 175], 3), ([699, 1, 0, 0], 4)):
        g2 = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            x.copy_(torch.randn(rows, k, generator=g2).bfloat16())
            lens.copy_(torch.tensor(new_lens, dtype=torch.int64))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for u, v in zip(got, want):
            assert torch.equal(u.view(torch.int16), v.view(torch.int16)), (new_lens, seed)


def test_shapes_the_kernel_does_not_take_are_refused(gpu):
    import primus_amd.pytorch as turbo

    gl = torch.tensor([4], dtype=torch.int64, device=gpu)
    a = torch.zeros(4, 40, dtype=torch.bfloat16, device=gpu)          # contraction not a multiple of 32
    b = torch.zeros(1, 16, 40, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        turbo.ops.grouped_gemm(a, b, gl)


TILE_CASES = [
    ([100, 0, 37, 300], 320, 256),
    ([1, 129, 0, 0, 128, 255, 257], 288, 96),
    ([1500, 3, 700], 544, 160),
    ([0, 0, 5], 32, 32),
    ([513, 256, 31], 2880, 64),
]


@pytest.mark.parametrize("lens,n,k", TILE_CASES)
def test_both_tile_heights_give_the_same_bits_and_match_fp32(gpu, lens, n, k):
    """The 256-row tiles (4-stage ring, one workgroup per CU) and the 128-row tiles (2 stages, two per CU) add every
    output element's products in the same order: forward, dgrad, wgrad and the accumulating wgrad are bit-identical,
    and each matches the fp32 matmul per expert."""
    from primus_amd.pytorch import kernels as K

    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(m + 3 * n + k)
    a = torch.randn(m, k, generator=gen).bfloat16().to(gpu)
    b = (torch.randn(G, n, k, generator=gen) * 0.1).bfloat16().to(gpu)
    dy = torch.randn(m, n, generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    outs = {}
    for tile in (128, 256):
        y = K.grouped_gemm_bf16_impl(a, b, gl, tile=tile)
        dx = K.grouped_gemm_bf16_impl(dy, b, gl, b_kn=True, tile=tile)
        dw = K.grouped_gemm_bf16_wgrad_impl(dy, a, gl, tile=tile)
        acc = torch.full((G, n, k), 0.5, dtype=torch.float32, device=gpu)
        K.grouped_gemm_bf16_wgrad_impl(dy, a, gl, accum_into=acc, tile=tile)
        outs[tile] = (y, dx, dw, acc)
    for u, v in zip(outs[128], outs[256]):
        assert torch.equal(u.view(torch.int16 if u.dtype == torch.bfloat16 else torch.int32),
                           v.view(torch.int16 if v.dtype == torch.bfloat16 else torch.int32))
    y, dx, dw, acc = outs[256]
    _close(y, _ref(a, b, lens, True), _ref(a.abs(), b.abs(), lens, True), k)
    _close(dx, _ref(dy, b, lens, False), _ref(dy.abs(), b.abs(), lens, False), n)
    off = 0
    for g, ln in enumerate(lens):
        x_g, d_g = a[off:off + ln].float(), dy[off:off + ln].float()
        _close(dw[g], d_g.t() @ x_g, d_g.abs().t() @ x_g.abs(), ln)
        assert torch.allclose(acc[g], 0.5 + d_g.t() @ x_g, rtol=1e-5, atol=1e-3 * max(1, ln) ** 0.5)
        off += ln


def test_tile_flags_are_validated(gpu):
    from primus_amd.pytorch import kernels as K

    a = torch.zeros(64, 64, dtype=torch.bfloat16, device=gpu)
    b = torch.zeros(1, 64, 64, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        K.grouped_gemm_bf16_impl(a, b, None, tile=64)


@pytest.mark.parametrize("tile", [128, 256])
def test_many_rounds_of_tiles_are_exact_on_integers(gpu, tile):
    """More tiles than persistent workgroups (several rounds per workgroup, ragged and empty groups in between):
    integer operands make every partial sum exact, so forward, dgrad and wgrad equal the fp32 matmul bit for bit."""
    from primus_amd.pytorch import kernels as K

    lens = [3000, 0, 517, 4100, 1, 2600, 255, 9527]
    n, k = 2048, 256
    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(77)
    a = torch.randint(-3, 4, (m, k), generator=gen).bfloat16().to(gpu)
    b = torch.randint(-2, 3, (G, n, k), generator=gen).bfloat16().to(gpu)
    dy = torch.randint(-2, 3, (m, n), generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = K.grouped_gemm_bf16_impl(a, b, gl, tile=tile)
    dx = K.grouped_gemm_bf16_impl(dy, b, gl, b_kn=True, tile=tile)
    dw = K.grouped_gemm_bf16_wgrad_impl(dy, a, gl, tile=tile)
    assert torch.equal(y, _ref(a, b, lens, True).bfloat16())
    assert torch.equal(dx, _ref(dy, b, lens, False).bfloat16())
    off = 0
    for g, ln in enumerate(lens):
        want = (dy[off:off + ln].float().t() @ a[off:off + ln].float()).bfloat16()
        assert torch.equal(dw[g], want), g
        off += ln
