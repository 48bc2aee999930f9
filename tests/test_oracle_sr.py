"""Pins the oracle's stochastic rounding to E2M1 (gradients of the MXFP4 recipe) by what the
definition of stochastic rounding fixes: exhaustive enumeration of the 2^16 random values for a set
of inputs covering every interval of the value table."""

import numpy as np

from oracle import mx_oracle as o

GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
ALL16 = np.arange(1 << 16, dtype=np.uint32)


def _bf16_values(lo, hi, n, rng):
    v = rng.uniform(lo, hi, size=n).astype(np.float32)
    return o.bf16_bits_to_f32(o.f32_to_bf16_bits(v))


def test_every_draw_is_a_neighbour_and_the_mean_is_the_input():
    rng = np.random.default_rng(7)
    vals = np.concatenate([_bf16_values(0, 6, 200, rng), _bf16_values(0, 0.01, 20, rng), GRID.astype(np.float32),
                           np.array([5.97, 0.499, 1.999, 3.99], dtype=np.float32)])
    for v in vals:
        for s in (1.0, -1.0):
            x = np.float32(s * v)
            codes = o.cast_e2m1_sr(np.full(1 << 16, x, dtype=np.float32), ALL16)
            mags = GRID[codes & 7]
            assert (((codes >> 3) & 1) == (1 if np.signbit(x) else 0)).all()
            lo = GRID[GRID <= abs(v)].max()
            hi = GRID[GRID > abs(v)].min() if abs(v) < 6 else 6.0
            assert set(np.unique(mags)) <= {lo, hi}
            # unbiased to within the 16-bit resolution of the random value
            assert abs(mags.mean() - abs(float(v))) <= (hi - lo) * 2.0 ** -16 + 1e-12
            # monotone in the random value: once a draw rounds up, all larger draws do
            assert (np.diff(mags) >= 0).all()


def test_grid_points_never_move_and_saturation():
    for i, g in enumerate(GRID):
        for s in (1.0, -1.0):
            codes = o.cast_e2m1_sr(np.full(1 << 16, s * g, dtype=np.float32), ALL16)
            assert ((codes & 7) == i).all()
    for v in (6.0, 6.5, 7.9, 100.0):
        assert ((o.cast_e2m1_sr(np.full(1 << 16, v, dtype=np.float32), ALL16) & 7) == 7).all()
        assert (o.cast_e2m1_sr(np.full(16, -v, dtype=np.float32), ALL16[:16]) == 15).all()


def test_zero_random_value_truncates_and_rne_is_one_of_the_two_outcomes():
    rng = np.random.default_rng(3)
    v = _bf16_values(-6, 6, 4096, rng)
    down = o.cast_e2m1_sr(v, np.zeros(v.shape, dtype=np.uint32))
    up = o.cast_e2m1_sr(v, np.full(v.shape, 0xFFFF, dtype=np.uint32))
    lo = np.array([GRID[GRID <= abs(x)].max() for x in v])
    assert np.array_equal(GRID[down & 7], lo)                          # toward zero
    rne = o.cast_e2m1(v)
    assert (((rne & 7) == (down & 7)) | ((rne & 7) == (up & 7))).all()


def test_counter_hash_is_uniform_and_streams_differ():
    n = 1 << 18
    c = np.arange(n, dtype=np.uint64)
    w0 = o.sr_word(c, seed=1234, stream=0)
    w1 = o.sr_word(c, seed=1234, stream=1)
    w2 = o.sr_word(c, seed=1235, stream=0)
    for w in (w0, w1, w2):
        for half in (w & 0xFFFF, w >> 16):
            # 256 buckets of the top byte: chi-square with 255 dof, mean 255, sd ~22.6
            counts = np.bincount((half >> 8).astype(np.int64), minlength=256)
            chi = ((counts - n / 256) ** 2 / (n / 256)).sum()
            assert chi < 255 + 6 * 22.6, chi
            assert abs(half.astype(np.float64).mean() / 65535 - 0.5) < 0.005
        bits = np.unpackbits(w.view(np.uint8))
        assert abs(bits.mean() - 0.5) < 0.002
    assert (w0 != w1).mean() > 0.999 and (w0 != w2).mean() > 0.999
    # neighbouring counters are uncorrelated
    a = (w0[:-1] >> 16).astype(np.float64)
    b = (w0[1:] >> 16).astype(np.float64)
    assert abs(np.corrcoef(a, b)[0, 1]) < 0.01
    # the high counter word matters
    hi = o.sr_word(c + (np.uint64(1) << np.uint64(32)), seed=1234, stream=0)
    assert (hi != w0).mean() > 0.999
    # a bijection has no collisions on distinct 32-bit inputs
    assert len(np.unique(o._sr_mix(np.arange(1 << 20, dtype=np.uint64)))) == 1 << 20


def test_quantise_sr_keeps_scales_and_is_unbiased_over_seeds():
    import torch

    rng = np.random.default_rng(11)
    x = torch.tensor(rng.standard_normal((8, 64)).astype(np.float32)).bfloat16()
    q0, s0 = o.quantize_mx_rowwise(x, o.FMT_E2M1)
    acc = np.zeros((8, 64))
    n = 400
    for seed in range(n):
        q, s = o.quantize_mx_rowwise_sr(x, seed)
        assert np.array_equal(s, s0)
        acc += o.dequantize_mx(q, s, o.FMT_E2M1)
    xf = x.float().numpy().astype(np.float64)
    scale = o.scale_f32(s0).astype(np.float64).repeat(32, axis=1)
    sat = np.abs(xf) > 6 * scale                      # saturated elements are biased by construction
    err = np.abs(acc / n - xf)[~sat]
    # one draw is off by at most one grid step (<= 2 scale units); the mean of n by ~ step / sqrt(n)
    assert (err <= 5 * 2 * scale[~sat] / np.sqrt(n)).all()
    # same seed, same codes; the two copies use different streams
    assert np.array_equal(o.quantize_mx_rowwise_sr(x, 5)[0], o.quantize_mx_rowwise_sr(x, 5)[0])
    assert not np.array_equal(o.quantize_mx_rowwise_sr(x, 5)[0], o.quantize_mx_rowwise_sr(x, 5, stream=1)[0])
    # the transposed copy is the row-wise routine on the padded transpose
    lens = [5, 0, 3]
    qT, sT = o.quantize_mx_colwise_segmented_sr(x, lens, 9)
    q_rne, s_rne = o.quantize_mx_colwise_segmented(x, lens, o.FMT_E2M1)
    assert qT.shape == q_rne.shape and np.array_equal(sT, s_rne)
