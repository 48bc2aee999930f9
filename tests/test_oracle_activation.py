"""Pins the oracle's gated activation (swiglu / geglu with router probabilities and row mask)
against library routines (torch float64 silu / gelu and autograd) and against identities that a
wrong sign, a swapped half or a dropped factor would break."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o


def _inputs(seed=0, m=7, f=24):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, 2 * f, generator=g) * 3).bfloat16()
    p = torch.rand(m, generator=g)
    mask = torch.tensor([True, True, False, True, True, False, True][:m])
    return x, p, mask


@pytest.mark.parametrize("activation,fn", [("silu", torch.nn.functional.silu), ("gelu", torch.nn.functional.gelu)])
def test_forward_matches_torch_float64(activation, fn):
    x, p, mask = _inputs()
    xd = x.double()
    f = x.shape[1] // 2
    want = fn(xd[:, :f]) * xd[:, f:] * p.double()[:, None]
    want = torch.where(mask[:, None], want, torch.zeros_like(want))
    got = o.glu_with_probs_ref(x, p.numpy(), mask.numpy(), activation, out_bf16=False)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-14)
    bits = o.glu_with_probs_ref(x, p.numpy(), mask.numpy(), activation)
    assert np.array_equal(bits, o.to_bf16_bits(want.float().bfloat16()))


@pytest.mark.parametrize("activation,fn", [("silu", torch.nn.functional.silu), ("gelu", torch.nn.functional.gelu)])
def test_backward_matches_torch_autograd_float64(activation, fn):
    x, p, mask = _inputs(seed=1)
    g = torch.Generator().manual_seed(5)
    dy = torch.randn(x.shape[0], x.shape[1] // 2, generator=g).bfloat16()
    xd, pd = x.double().requires_grad_(), p.double().requires_grad_()
    f = x.shape[1] // 2
    y = fn(xd[:, :f]) * xd[:, f:] * pd[:, None]
    y = torch.where(mask[:, None], y, torch.zeros_like(y))
    y.backward(dy.double())
    dx, dp = o.glu_with_probs_bwd_ref(dy, x, p.numpy(), mask.numpy(), activation)
    np.testing.assert_allclose(dx, xd.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dp, pd.grad.numpy(), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_identities(activation):
    g = np.linspace(-12, 12, 97)
    a_pos, _ = o._act64(g, activation)
    a_neg, _ = o._act64(-g, activation)
    np.testing.assert_allclose(a_pos - a_neg, g, rtol=0, atol=1e-12)   # act(x) - act(-x) = x
    assert o._act64(np.array([0.0]), activation)[0][0] == 0.0
    big, _ = o._act64(np.array([40.0, -40.0]), activation)
    assert big[0] == pytest.approx(40.0) and abs(big[1]) < 1e-12
    # derivative against a centred difference
    h = 1e-6
    _, da = o._act64(g, activation)
    num = (o._act64(g + h, activation)[0] - o._act64(g - h, activation)[0]) / (2 * h)
    np.testing.assert_allclose(da, num, rtol=1e-6, atol=1e-8)


def test_gate_is_the_first_half_and_probs_scale_rows():
    x = torch.zeros(2, 16).bfloat16()
    x[:, :8] = 2.0      # gate
    x[:, 8:] = 3.0      # linear
    y = o.glu_with_probs_ref(x, np.array([1.0, 0.5]), None, "silu", out_bf16=False)
    silu2 = 2.0 / (1.0 + np.exp(-2.0))
    np.testing.assert_allclose(y[0], silu2 * 3.0)
    np.testing.assert_allclose(y[1], 0.5 * silu2 * 3.0)
    swapped = torch.cat([x[:, 8:], x[:, :8]], dim=1)
    assert not np.allclose(o.glu_with_probs_ref(swapped, np.ones(2), None, "silu", out_bf16=False), y[0])
