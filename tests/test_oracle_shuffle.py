"""The pre-shuffled MXFP4 layouts of the oracle against the published view / permute formulation evaluated by torch,
inverses, and the scale shapes the reference's own shape function states (primus_turbo_mxfp4_local.py:184-198)."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o


def _shuffle_weight_by_views(x: torch.Tensor) -> torch.Tensor:
    # layout (16, 16) on one-byte elements: BN = 16 rows, BK = 32 bytes, innermost run 16 bytes
    n, k = x.shape
    v = x.view(1, n // 16, 16, k // 32, 2, 16).permute(0, 1, 3, 4, 2, 5).contiguous()
    return v.view(n, k)


def _e8m0_shuffle_by_views(s: torch.Tensor) -> torch.Tensor:
    m, n = s.shape
    padded = torch.zeros(((m + 255) // 256 * 256, (n + 7) // 8 * 8), dtype=s.dtype)
    padded[:m, :n] = s
    sm, sn = padded.shape
    v = padded.view(sm // 32, 2, 16, sn // 8, 2, 4, 1).permute(0, 3, 5, 2, 4, 1, 6).contiguous()
    return v.view(sm, sn)


@pytest.mark.parametrize("rows,row_bytes", [(16, 32), (32, 64), (128, 128), (48, 96), (512, 1440)])
def test_code_shuffle_matches_the_view_formulation(rows, row_bytes):
    rng = np.random.default_rng(rows * 7 + row_bytes)
    x = rng.integers(0, 256, size=(rows, row_bytes), dtype=np.uint8)
    got = o.shuffle_codes_16x16(x)
    want = _shuffle_weight_by_views(torch.from_numpy(x)).numpy()
    assert np.array_equal(got, want)
    assert np.array_equal(o.unshuffle_codes_16x16(got), x)
    # a 16 x 32-byte block becomes 512 consecutive bytes: first the low 16 bytes of its 16 rows, then the high ones
    assert np.array_equal(got.ravel()[:256].reshape(16, 16), x[:16, :16])
    assert np.array_equal(got.ravel()[256:512].reshape(16, 16), x[:16, 16:32])


def test_code_shuffle_rejects_ragged_shapes():
    with pytest.raises(ValueError):
        o.shuffle_codes_16x16(np.zeros((8, 32), dtype=np.uint8))
    with pytest.raises(ValueError):
        o.shuffle_codes_16x16(np.zeros((16, 48), dtype=np.uint8))


@pytest.mark.parametrize("rows,blocks", [(256, 8), (32, 8), (1, 1), (100, 5), (300, 90), (512, 4), (2880, 90)])
def test_scale_shuffle_matches_the_view_formulation(rows, blocks):
    rng = np.random.default_rng(rows * 13 + blocks)
    s = rng.integers(1, 256, size=(rows, blocks), dtype=np.uint8)
    got = o.shuffle_e8m0(s)
    want = _e8m0_shuffle_by_views(torch.from_numpy(s)).numpy()
    assert got.shape == want.shape == o.shuffled_scale_shape(rows, blocks)
    assert np.array_equal(got, want)
    assert np.array_equal(o.unshuffle_e8m0(got, rows, blocks), s)
    # the padding holds zero bytes: every non-zero input byte appears exactly once
    assert int((got != 0).sum()) == rows * blocks


def test_shuffled_scale_shape_is_the_reference_shape_function():
    # rs_M = cdiv(M, 256) * 256, rs_N = cdiv(cdiv(N_pad, 32), 8) * 8
    for m, n_pad in [(128, 256), (4096, 4096), (1000, 2944), (16384, 5760)]:
        blocks = -(-n_pad // 32)
        assert o.shuffled_scale_shape(m, blocks) == (-(-m // 256) * 256, -(-blocks // 8) * 8)
