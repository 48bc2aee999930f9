"""The C restatement (oracle/mx_oracle.c) against the Python oracle, bit for bit,
and both against the committed golden fixtures.  CPU only."""

import os

import numpy as np
import pytest
import torch

from oracle import c_oracle as c
from oracle import mx_oracle as o

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module", autouse=True)
def _built():
    c.build()


def _awkward(seed=1):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(200, 96, generator=g) * torch.exp2(torch.randint(-30, 30, (200, 1), generator=g).float())).bfloat16()
    x[3, 5] = float("inf")
    x[9, 40] = float("nan")
    x[20] = 0
    x[21, :32] = 1e-38
    return o.to_bf16_bits(x)


@pytest.mark.parametrize("fmt", [o.FMT_E4M3, o.FMT_E2M1])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_c_equals_python(fmt, mode):
    xb = _awkward()
    a, b = o.quantize_mx_rowwise(xb, fmt, mode), c.quantize_rowwise(xb, fmt, mode)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    lens = [33, 0, 130, 37]
    a, b = o.quantize_mx_colwise_segmented(xb, lens, fmt, mode), c.quantize_colwise_segmented(xb, lens, fmt, mode)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    w = o.to_bf16_bits((torch.randn(2, 64, 96, generator=torch.Generator().manual_seed(2)) * 0.02).bfloat16())
    for u, v in zip(o.quantize_mx_2d(w, fmt, mode), c.quantize_2d(w, fmt, mode)):
        assert np.array_equal(u, v)
    q, s = o.quantize_mx_rowwise(xb, fmt, mode)
    d1, d2 = o.dequantize_mx(q, s, fmt), c.dequantize(q, s, fmt)
    assert np.array_equal(np.isnan(d1), np.isnan(d2))
    assert np.array_equal(np.nan_to_num(d1), np.nan_to_num(d2))


def test_c_gemm_equals_python():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(40, 64, generator=g).bfloat16()
    w = (torch.randn(24, 64, generator=g) * 0.05).bfloat16()
    xq, xs = o.quantize_mx_rowwise(x)
    wq, ws = o.quantize_mx_rowwise(w)
    want = o.bf16_bits_to_f32(o.gemm_nt_ref(xq, xs, wq, ws))
    got = o.bf16_bits_to_f32(c.matmul_nt_bf16(c.dequantize(xq, xs, 0), c.dequantize(wq, ws, 0)))
    # summation order differs (BLAS vs a plain loop): equal within one bf16 ulp
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0**-7 + 1e-6)


def test_golden_exhaustive_bf16():
    z = np.load(os.path.join(GOLD, "exhaustive_bf16.npz"))
    for fmt, fn in ((o.FMT_E4M3, "e4m3"), (o.FMT_E2M1, "e2m1")):
        for mode, mn in ((0, "floor"), (1, "rceil"), (2, "even")):
            for name in ("x", "y"):
                for impl in (o.quantize_mx_rowwise, c.quantize_rowwise):
                    q, s = impl(z[name], fmt, mode)
                    assert np.array_equal(q, z[f"{name}_{fn}_{mn}_q"]), (fn, mn, name, impl)
                    assert np.array_equal(s, z[f"{name}_{fn}_{mn}_s"]), (fn, mn, name, impl)


def test_golden_matrices_and_ragged_gemm():
    z = np.load(os.path.join(GOLD, "matrices.npz"))
    for name in ("normal", "weight", "outlier"):
        xb = z[f"{name}_x"]
        for fmt, fn in ((o.FMT_E4M3, "e4m3"), (o.FMT_E2M1, "e2m1")):
            q, s = c.quantize_rowwise(xb, fmt)
            assert np.array_equal(q, z[f"{name}_{fn}_row_q"]) and np.array_equal(s, z[f"{name}_{fn}_row_s"])
            q, s = c.quantize_colwise_segmented(xb, [64], fmt)
            assert np.array_equal(q, z[f"{name}_{fn}_col_q"]) and np.array_equal(s, z[f"{name}_{fn}_col_s"])
            got = c.quantize_2d(xb, fmt)
            for k, v in zip(("2d_q", "2d_s", "2d_qt", "2d_st"), got):
                assert np.array_equal(v, z[f"{name}_{fn}_{k}"])
    r = np.load(os.path.join(GOLD, "ragged_gemm.npz"))
    y = o.grouped_gemm_nt_ref(r["xq"], r["xs"], r["wq"], r["ws"], r["lens"])
    assert np.array_equal(y, r["y"])
    dx, dw = o.linear_bwd_ref(r["x"], r["w"], r["dy"], group_lens=list(r["lens"]))
    assert np.array_equal(dx, r["dx"]) and np.array_equal(dw, r["dw"])
    assert not r["dw"][0].any()  # empty expert -> zero gradient
