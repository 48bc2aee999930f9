"""Pins the oracle's tensor-wise FP8 quantiser: the E5M2 cast against torch.float8_e5m2 (library routine)
over every bf16 value and float32 samples on the rounding boundaries, the quantiser against the reference's
formula (primus_turbo_float8_local.py:194-207) evaluated with torch ops in float32, and the scaled GEMM
against a float64 matmul of the decoded operands."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o


def test_e5m2_cast_every_bf16_value():
    bits = np.arange(65536, dtype=np.uint16)
    f = o.bf16_bits_to_f32(bits)
    fin = np.isfinite(f)
    want = torch.from_numpy(f.copy()).clamp(-57344, 57344).to(torch.float8_e5m2).view(torch.uint8).numpy()
    got = o.cast_e5m2(f)
    assert np.array_equal(got[fin], want[fin])
    nan = np.isnan(f)
    assert np.all((got[nan] & 0x7F) == 0x7F)
    inf = np.isinf(f)
    assert np.all((got[inf] & 0x7F) == 0x7B)          # saturates like any large value


def test_e5m2_cast_on_rounding_boundaries():
    # midpoints between neighbouring E5M2 values and their float32 neighbours: ties go to the even code
    codes = np.arange(0, 0x7B, dtype=np.uint8)
    lo, hi = o.decode_e5m2(codes).astype(np.float64), o.decode_e5m2(codes + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    for v in (mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9))):
        want = torch.from_numpy(v.copy()).to(torch.float8_e5m2).view(torch.uint8).numpy()
        assert np.array_equal(o.cast_e5m2(v), want)
        assert np.array_equal(o.cast_e5m2(-v), want | 0x80)
    assert np.array_equal(o.cast_e5m2(mid) & 1, np.zeros_like(codes))       # even code on every tie


def test_e5m2_decode_matches_torch():
    c = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(c.copy()).view(torch.float8_e5m2).float().numpy()
    got = o.decode_e5m2(c)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


@pytest.mark.parametrize("fmt,dt,fmax", [(o.FMT_E4M3, torch.float8_e4m3fn, 448.0), (o.FMT_E5M2, torch.float8_e5m2, 57344.0)])
@pytest.mark.parametrize("spread", [1e-3, 1.0, 300.0])
def test_quantiser_matches_the_reference_formula(fmt, dt, fmax, spread):
    g = torch.Generator().manual_seed(int(fmax) + int(spread * 10))
    x = (torch.randn(64, 96, generator=g) * spread).bfloat16()
    codes, scale_inv = o.quantize_tensorwise(x, fmt)
    xf = x.float()
    amax = xf.abs().amax()
    scale = fmax / amax.clamp(min=1e-12)                                     # float32, as the reference computes it
    want = (xf * scale).clamp(-fmax, fmax).to(dt).view(torch.uint8).numpy()
    assert np.array_equal(codes, want)
    # torch evaluates scalar / tensor as scalar * reciprocal(tensor): within two float32 ulps of the IEEE divisions
    assert np.isclose(scale_inv, (1.0 / scale).item(), rtol=2.5e-7)
    assert np.isclose(scale_inv, float(amax.double() / fmax), rtol=2.5e-7)
    # the largest element lands on the largest code, and decoding inverts the scaling to FP8 precision
    assert (codes.reshape(-1)[xf.abs().argmax()] & 0x7F) == (0x7E if fmt == o.FMT_E4M3 else 0x7B)
    deq = o.decode_fp8(codes, fmt).astype(np.float64) * float(scale_inv)
    step = 2.0 ** -3 if fmt == o.FMT_E4M3 else 2.0 ** -2
    big = np.abs(xf.numpy()) > float(amax) * 2.0 ** -6                       # normal range of both formats
    assert np.all(np.abs(deq - xf.numpy())[big] <= np.abs(xf.numpy())[big] * step / 2 * 1.01)


def test_quantiser_special_cases():
    z = torch.zeros(4, 32).bfloat16()
    codes, si = o.quantize_tensorwise(z, o.FMT_E4M3)
    assert not codes.any() and np.isclose(si, 1e-12 / 448.0, rtol=1e-6)
    x = torch.ones(4, 32).bfloat16()
    x[1, 1] = float("nan")
    codes, _ = o.quantize_tensorwise(x, o.FMT_E5M2)
    assert np.all(codes == 0x7F)
    x[1, 1] = float("-inf")
    codes, _ = o.quantize_tensorwise(x, o.FMT_E4M3)
    assert np.all(codes == 0x7F)


def test_scaled_gemm_matches_float64():
    rng = np.random.default_rng(3)
    a = rng.integers(0, 256, size=(24, 64)).astype(np.uint8)
    b = rng.integers(0, 256, size=(40, 64)).astype(np.uint8)
    a[(a & 0x7C) == 0x7C] = 0x10        # no E5M2 Inf / NaN
    b[(b & 0x7F) == 0x7F] = 0x10        # no E4M3 NaN
    got = o.tensorwise_gemm_nt_ref(a, 0.37, b, 1.9, o.FMT_E5M2, o.FMT_E4M3, out_bf16=False)
    want = (o.decode_e5m2(a).astype(np.float64) @ o.decode_e4m3(b).astype(np.float64).T) * np.float64(np.float32(0.37) * np.float32(1.9))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
