"""Pins the oracle's RMSNorm (forward in the kernel's float32 summation order, backward closed form)
against float64 closed forms, torch's rms_norm and autograd (library routines) and invariants that a
dropped eps, a mean taken as a sum, a missing weight or a wrong sign in the backward would break."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o


def _inputs(seed, rows, k, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, k, generator=g) * spread).bfloat16()
    w = (1 + 0.2 * torch.randn(k, generator=g)).bfloat16()
    return x, w


@pytest.mark.parametrize("rows,k,eps", [(5, 32, 1e-5), (7, 4096, 1e-5), (3, 2056, 1e-6), (2, 16384, 1e-5), (4, 8, 0.5)])
def test_rstd_matches_float64(rows, k, eps):
    x, _ = _inputs(rows + k, rows, k)
    got = o.rmsnorm_rstd(x, eps)
    want = 1.0 / np.sqrt((x.double().numpy() ** 2).mean(axis=1) + eps)
    assert got.dtype == np.float32
    np.testing.assert_allclose(got, want, rtol=4e-7)       # a few float32 roundings


def test_rstd_special_rows():
    x = torch.zeros(3, 64).bfloat16()
    x[1] = 2.0
    x[2, 0] = 8.0
    got = o.rmsnorm_rstd(x, 1e-6)
    np.testing.assert_allclose(got, [1e3, 1 / np.sqrt(4 + 1e-6), 1 / np.sqrt(1 + 1e-6)], rtol=1e-6)


@pytest.mark.parametrize("rows,k", [(9, 4096), (5, 160), (3, 8192)])
def test_forward_matches_torch(rows, k):
    x, w = _inputs(rows * k, rows, k)
    bits, rstd = o.rmsnorm_ref(x, w, 1e-5)
    y = o.bf16_bits_to_f32(bits).astype(np.float64)
    want64 = torch.nn.functional.rms_norm(x.double(), [k], w.double(), 1e-5).numpy()
    assert np.all(np.abs(y - want64) <= np.abs(want64) * 2.0 ** -8 + 1e-30)      # half a bf16 ulp: one rounding
    # torch's bf16 routine: same values up to one ulp where the exact result sits next to a rounding boundary
    t = torch.nn.functional.rms_norm(x, [k], w, 1e-5).float().numpy().astype(np.float64)
    assert np.all(np.abs(y - t) <= np.abs(t) * 2.0 ** -7 + 1e-30)
    assert (y != t).mean() < 0.01


def test_forward_invariants():
    x, w = _inputs(3, 6, 512)
    ones = torch.ones(512).bfloat16()
    bits, _ = o.rmsnorm_ref(x, ones, 0.0)
    y = o.bf16_bits_to_f32(bits).astype(np.float64)
    np.testing.assert_allclose(np.sqrt((y ** 2).mean(axis=1)), 1.0, rtol=3e-3)   # unit rms (bf16 rounding of y)
    # scaling the input by a power of two changes nothing when eps = 0
    bits4, _ = o.rmsnorm_ref((x.float() * 4).bfloat16(), ones, 0.0)
    assert np.array_equal(bits, bits4)
    # the weight multiplies column-wise: doubling it doubles y exactly
    a, _ = o.rmsnorm_ref(x, w, 1e-5)
    b, _ = o.rmsnorm_ref(x, (w.float() * 2).bfloat16(), 1e-5)
    assert np.array_equal(o.bf16_bits_to_f32(a) * 2, o.bf16_bits_to_f32(b))
    # a large eps dominates: y ~ x * w / sqrt(eps)
    c, _ = o.rmsnorm_ref(x, w, 1e6)
    np.testing.assert_allclose(o.bf16_bits_to_f32(c), x.float().numpy() * w.float().numpy() / 1e3, rtol=2e-2, atol=1e-6)


@pytest.mark.parametrize("rows,k", [(6, 256), (4, 4096)])
def test_backward_matches_torch_autograd_float64(rows, k):
    x, w = _inputs(rows + 7 * k, rows, k)
    g = torch.Generator().manual_seed(11)
    dy = torch.randn(rows, k, generator=g).bfloat16()
    xd, wd = x.double().requires_grad_(), w.double().requires_grad_()
    y = torch.nn.functional.rms_norm(xd, [k], wd, 1e-5)
    gx, gw = torch.autograd.grad(y, [xd, wd], dy.double())
    dx, dw = o.rmsnorm_bwd_ref(dy, x, w, 1e-5)
    np.testing.assert_allclose(dx, gx.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(dw, gw.numpy(), rtol=1e-9, atol=1e-12)


def test_backward_is_orthogonal_to_the_input_direction():
    """With eps = 0 the output does not change along x, so dx . x = 0 for every row."""
    x, w = _inputs(5, 8, 1024)
    g = torch.Generator().manual_seed(2)
    dy = torch.randn(8, 1024, generator=g).bfloat16()
    dx, _ = o.rmsnorm_bwd_ref(dy, x, w, 0.0)
    dots = (dx * x.double().numpy()).sum(axis=1)
    assert np.all(np.abs(dots) < 1e-9 * np.abs(dx).sum(axis=1) * np.abs(x.double().numpy()).max())
