"""Pins the oracle's 16-point randomised Hadamard transform (transposed copies of the MXFP4 recipe)
against scipy's Hadamard matrix and by the properties that make it usable in a wgrad GEMM."""

import numpy as np
import scipy.linalg

from oracle import mx_oracle as o


def _bits(a):
    return o.f32_to_bf16_bits(np.asarray(a, dtype=np.float32))


def _vals(b):
    return o.bf16_bits_to_f32(b).astype(np.float64)


def test_matches_the_hadamard_matrix():
    H = scipy.linalg.hadamard(16).astype(np.float64)          # Sylvester order
    rng = np.random.default_rng(0)
    # small integers: every partial sum is exact in float32 and the result exact in bf16 after / 4
    x = rng.integers(-3, 4, size=(64, 5)).astype(np.float32) * 4
    for signs in (0, 0xFFFF, 0xA6C9, 0x0001, 0x8000):
        s = np.array([-1.0 if (signs >> i) & 1 else 1.0 for i in range(16)])
        got = _vals(o.hadamard16_rows(_bits(x), signs))
        for g in range(4):
            want = H @ (s[:, None] * x[16 * g : 16 * g + 16].astype(np.float64)) / 4
            assert np.array_equal(got[16 * g : 16 * g + 16], want)
    # general values: equal to the float64 product up to fp32 accumulation and one bf16 rounding
    x = rng.standard_normal((32, 7)).astype(np.float32)
    xb = _bits(x)
    got = _vals(o.hadamard16_rows(xb, 0x1234))
    s = np.array([-1.0 if (0x1234 >> i) & 1 else 1.0 for i in range(16)])
    for g in range(2):
        want = H @ (s[:, None] * _vals(xb)[16 * g : 16 * g + 16]) / 4
        assert np.abs(got[16 * g : 16 * g + 16] - want).max() <= 2.0 ** -8 * np.abs(want).max() + 1e-6


def test_orthogonal_and_involutive():
    rng = np.random.default_rng(1)
    x = rng.integers(-8, 9, size=(48, 6)).astype(np.float32) * 16     # exact through two transforms
    xb = _bits(x)
    twice = o.hadamard16_rows(o.hadamard16_rows(xb, 0), 0)            # H/4 is its own inverse
    assert np.array_equal(_vals(twice), x.astype(np.float64))
    # inner products over the token axis are preserved when both operands use the same signs
    y = rng.integers(-8, 9, size=(48, 6)).astype(np.float32) * 16
    tx, ty = _vals(o.hadamard16_rows(xb, 0xBEEF)), _vals(o.hadamard16_rows(_bits(y), 0xBEEF))
    assert np.array_equal(tx.T @ ty, x.astype(np.float64).T @ y.astype(np.float64))
    # ... and not when they differ
    tz = _vals(o.hadamard16_rows(_bits(y), 0xBEEE))
    assert not np.array_equal(tx.T @ tz, x.astype(np.float64).T @ y.astype(np.float64))


def test_lowers_the_fp4_error_of_heavy_tailed_data():
    """What the transform is for: element-wise heavy tails (Student-t, 3 degrees of freedom) are
    spread over 16 positions before they meet the 4-bit grid; the wgrad contraction of two such
    operands is markedly closer to the exact one (about half the error; asserted with margin)."""
    import torch

    rng = np.random.default_rng(2)
    xt = torch.tensor(rng.standard_t(3, (1024, 32)).astype(np.float32)).bfloat16()
    yt = torch.tensor(rng.standard_t(3, (1024, 16)).astype(np.float32)).bfloat16()
    exact = xt.float().numpy().astype(np.float64).T @ yt.float().numpy().astype(np.float64)

    def wgrad(signs):
        qa, sa = o.quantize_mx_colwise_segmented_fp4(xt, [1024], rht_signs=signs)
        qb, sb = o.quantize_mx_colwise_segmented_fp4(yt, [1024], rht_signs=signs)
        a = o.dequantize_mx(qa, sa, o.FMT_E2M1).astype(np.float64)
        b = o.dequantize_mx(qb, sb, o.FMT_E2M1).astype(np.float64)
        return a @ b.T

    err_plain = np.linalg.norm(wgrad(None) - exact)
    err_rht = np.linalg.norm(wgrad(0xA6C9) - exact)
    assert err_rht < 0.8 * err_plain, (err_rht, err_plain)
