"""RMSNorm kernels and the normalisation fused into the MX quantiser, on the GPU.

Bars: rstd and the normalised output equal the oracle bit for bit (the kernel's summation order is part
of its definition); the fused normalisation + quantisation equals quantising the normalised tensor byte
for byte; gradients are floating point: dx within one bf16 ulp of the float64 closed form plus 1e-5 of
the magnitude of the two terms that cancel, dw (a sum over all rows rounded to bf16) within 2^-7 relative
plus 1e-4 of the sum of magnitudes."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


def _inputs(seed, rows, k, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, k, generator=g) * spread * torch.logspace(-1, 1, rows)[:, None]).bfloat16()
    w = (1 + 0.2 * torch.randn(k, generator=g)).bfloat16()
    dy = torch.randn(rows, k, generator=g).bfloat16()
    return x, w, dy


SHAPES = [(1, 8), (37, 32), (300, 160), (64, 4096), (5, 2056), (1030, 1024), (3, 16384), (2, 8192)]


@pytest.mark.parametrize("rows,k", SHAPES)
@pytest.mark.parametrize("eps", [1e-5, 0.0])
def test_forward_equals_the_oracle(gpu, rows, k, eps):
    from primus_amd.pytorch import kernels as K

    x, w, _ = _inputs(rows + k, rows, k)
    if rows > 2 and eps > 0:
        x[1] = 0          # an all-zero row: rstd = 1 / sqrt(eps), y = 0
    y, rstd = K.rmsnorm_fwd_impl(x.to(gpu), w.to(gpu), eps)
    want_bits, want_rstd = o.rmsnorm_ref(x, w, eps)
    assert np.array_equal(rstd.cpu().numpy().view(np.uint32), want_rstd.view(np.uint32))
    assert np.array_equal(_bits(y), want_bits)
    none, rstd2 = K.rmsnorm_fwd_impl(x.to(gpu), w.to(gpu), eps, want_y=False)
    assert none is None and torch.equal(rstd, rstd2)


@pytest.mark.parametrize("rows,k", SHAPES + [(2500, 512)])
def test_backward_vs_oracle(gpu, rows, k):
    from primus_amd.pytorch import kernels as K

    x, w, dy = _inputs(3 * rows + k, rows, k)
    eps = 1e-5
    _, rstd = K.rmsnorm_fwd_impl(x.to(gpu), w.to(gpu), eps, want_y=False)
    dx, dw = K.rmsnorm_bwd_impl(dy.to(gpu), x.to(gpu), w.to(gpu), rstd)
    want_dx, want_dw = o.rmsnorm_bwd_ref(dy, x, w, eps)
    xf, df, wf = x.double().numpy(), dy.double().numpy(), w.double().numpy()
    r = 1.0 / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + eps)
    g = df * wf
    mag = (np.abs(g) + np.abs(xf * r) * np.abs((g * xf * r).mean(axis=1, keepdims=True))) * r
    got = o.bf16_bits_to_f32(_bits(dx)).astype(np.float64)
    assert np.all(np.abs(got - want_dx) <= np.abs(want_dx) * 2.0 ** -7 + 1e-5 * mag + 1e-30)
    got_w = o.bf16_bits_to_f32(_bits(dw)).astype(np.float64)
    mag_w = (np.abs(df) * np.abs(xf * r)).sum(axis=0)
    assert np.all(np.abs(got_w - want_dw) <= np.abs(want_dw) * 2.0 ** -7 + 1e-4 * mag_w + 1e-30)
    # run to run identical (fixed summation order, no atomics)
    dx2, dw2 = K.rmsnorm_bwd_impl(dy.to(gpu), x.to(gpu), w.to(gpu), rstd)
    assert _same(dx, dx2) and _same(dw, dw2)


def test_no_rows(gpu):
    from primus_amd.pytorch import kernels as K

    x = torch.empty(0, 256, dtype=torch.bfloat16, device=gpu)
    w = torch.ones(256, dtype=torch.bfloat16, device=gpu)
    y, rstd = K.rmsnorm_fwd_impl(x, w, 1e-5)
    assert y.shape == (0, 256) and rstd.shape == (0,)
    dx, dw = K.rmsnorm_bwd_impl(x, x, w, rstd)
    assert dx.shape == (0, 256) and torch.count_nonzero(dw.float()) == 0


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("rows,k", [(37, 32), (300, 160), (257, 4096), (1030, 1024), (64, 16384)])
@pytest.mark.parametrize("kchunk", [False, True])
def test_fused_quantiser_equals_the_two_kernels(gpu, fmt, rows, k, kchunk):
    from primus_amd.pytorch import kernels as K

    x, w, _ = _inputs(rows * 3 + k + fmt, rows, k)
    x, w = x.to(gpu), w.to(gpu)
    y, rstd = K.rmsnorm_fwd_impl(x, w, 1e-5)
    for colwise in (True, False):
        want = K.quantize_mx_impl(y, fmt, rowwise=True, colwise=colwise, pad_to=128, kchunk=kchunk)
        got = K.rmsnorm_quantize_impl(x, w, rstd, fmt, colwise=colwise, pad_to=128, kchunk=kchunk)
        for a, b in zip(got, want):
            assert (a is None and b is None) or _same(a, b)
    for mode in (1, 2):
        want = K.quantize_mx_impl(y, fmt, mode, rowwise=True, colwise=True, pad_to=128, kchunk=kchunk)
        got = K.rmsnorm_quantize_impl(x, w, rstd, fmt, mode, colwise=True, pad_to=128, kchunk=kchunk)
        assert all(_same(a, b) for a, b in zip(got, want))


def test_operator_matches_torch(gpu):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.ops.normalization import rmsnorm

    assert rmsnorm is turbo.ops.rmsnorm
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 50, 512, generator=g).bfloat16().to(gpu).requires_grad_()
    w = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(6, 50, 512, generator=g).bfloat16().to(gpu)
    y = rmsnorm(x, w, 1e-5)
    gx, gw = torch.autograd.grad(y, [x, w], dy)
    xd, wd = x.detach().double().requires_grad_(), w.detach().double().requires_grad_()
    yd = torch.nn.functional.rms_norm(xd, [512], wd, 1e-5)
    gxd, gwd = torch.autograd.grad(yd, [xd, wd], dy.double())
    assert y.shape == x.shape and gx.shape == x.shape and gw.shape == w.shape
    assert torch.all((y.double() - yd).abs() <= yd.abs() * 2.0 ** -8 + 1e-30)
    assert (gx.double() - gxd).abs().max() <= 2.0 ** -6 * gxd.abs().max()
    assert (gw.double() - gwd).abs().max() <= 2.0 ** -6 * gwd.abs().max()
    with pytest.raises(ValueError):
        rmsnorm(x.float(), w, 1e-5)
    with pytest.raises(ValueError):
        turbo.kernels.rmsnorm_fwd_impl(x.detach().view(-1, 512)[:, :500], w.detach()[:500].contiguous(), 1e-5)


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("rows,k,n", [(300, 160, 96), (512, 1024, 256), (33, 4096, 128)])
@pytest.mark.parametrize("kchunk", [True, False])
def test_fused_linear_equals_norm_then_linear(gpu, fp4, rows, k, n, kchunk):
    """rmsnorm_gemm == gemm(rmsnorm(x)): output and all three gradients bit for bit."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    if fp4:
        cfg = Float4QuantConfig(format=Format.E2M1_X2, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
        plain, fused = turbo.ops.gemm_fp4, turbo.ops.rmsnorm_gemm_fp4
    else:
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
        plain, fused = turbo.ops.gemm_fp8, turbo.ops.rmsnorm_gemm_fp8
    g = torch.Generator().manual_seed(rows + k + n)
    x = torch.randn(rows, k, generator=g).bfloat16().to(gpu)
    nw = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(gpu)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(rows, n, generator=g).bfloat16().to(gpu)
    outs = []
    try:
        turbo.ops.set_kchunk_layout(kchunk)
        for f in (False, True):
            xx, nn, ww = x.clone().requires_grad_(), nw.clone().requires_grad_(), w.clone().requires_grad_()
            y = fused(xx, nn, 1e-5, ww, config=cfg) if f else plain(turbo.ops.rmsnorm(xx, nn, 1e-5), ww, config=cfg)
            outs.append((y,) + torch.autograd.grad(y, [xx, nn, ww], dy))
    finally:
        turbo.ops.set_kchunk_layout(True)
    for a, b in zip(*outs):
        assert _same(a, b)
    # only the weight needs a gradient: no dgrad, no norm backward
    xx, ww = x.clone(), w.clone().requires_grad_()
    y = fused(xx, nw, 1e-5, ww, config=cfg)
    (gw,) = torch.autograd.grad(y, [ww], dy)
    assert _same(y, outs[0][0]) and _same(gw, outs[0][3])
