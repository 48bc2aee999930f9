"""HIP quantisers (through the C ABI) against the CPU oracle and the golden
fixtures: codes and E8M0 scales must match bit for bit."""

import os

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
FMTS = [(o.FMT_E4M3, "e4m3"), (o.FMT_E2M1, "e2m1")]
MODES = [(0, "floor"), (1, "rceil"), (2, "even")]


def _bf16_dev(bits: np.ndarray, dev):
    return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)


def _np(t):
    return None if t is None else t.view(torch.uint8).cpu().numpy()


def _quant(x, fmt, mode, dev, lens=None, row=True, col=True):
    from primus_amd.pytorch import kernels as K

    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=dev)
    return [_np(t) for t in K.quantize_mx_impl(x, fmt, mode, rowwise=row, colwise=col, group_lens=gl)]


@pytest.mark.parametrize("fmt,fn", FMTS)
@pytest.mark.parametrize("mode,mn", MODES)
def test_exhaustive_bf16_golden(gpu, fmt, fn, mode, mn):
    """All 65536 bf16 bit patterns (NaN, Inf, subnormals, both zeros included)."""
    z = np.load(os.path.join(GOLD, "exhaustive_bf16.npz"))
    for name in ("x", "y"):
        q, s, _, _ = _quant(_bf16_dev(z[name], gpu), fmt, mode, gpu, col=False)
        assert np.array_equal(s, z[f"{name}_{fn}_{mn}_s"]), name
        assert np.array_equal(q, z[f"{name}_{fn}_{mn}_q"]), name


@pytest.mark.parametrize("fmt,fn", FMTS)
def test_golden_matrices(gpu, fmt, fn):
    from primus_amd.pytorch import kernels as K

    z = np.load(os.path.join(GOLD, "matrices.npz"))
    for name in ("normal", "weight", "outlier"):
        x = _bf16_dev(z[f"{name}_x"], gpu)
        q, s, qc, sc = _quant(x, fmt, 0, gpu)
        assert np.array_equal(q, z[f"{name}_{fn}_row_q"]) and np.array_equal(s, z[f"{name}_{fn}_row_s"])
        assert np.array_equal(qc, z[f"{name}_{fn}_col_q"]) and np.array_equal(sc, z[f"{name}_{fn}_col_s"])
        got = [_np(t) for t in K.quantize_mx_weight_2d_impl(x, fmt, 0)]
        for k, v in zip(("2d_q", "2d_s", "2d_qt", "2d_st"), got):
            assert np.array_equal(v, z[f"{name}_{fn}_{k}"]), k


@pytest.mark.parametrize("fmt,fn", FMTS)
@pytest.mark.parametrize("mode,mn", MODES)
@pytest.mark.parametrize("shape", [(300, 192), (1, 32), (129, 2880), (128, 128), (31, 64)])
def test_seeded_vs_oracle(gpu, fmt, fn, mode, mn, shape):
    g = torch.Generator().manual_seed(hash(shape) % 1000)
    m, c = shape
    x = (torch.randn(m, c, generator=g) * torch.exp2(torch.randint(-10, 10, (m, 1), generator=g).float())).bfloat16()
    if m > 20:
        x[5, 7] = 1000.0
        x[17, : min(c, 40)] = 0.0
    xd = x.to(gpu)
    q, s, qc, sc = _quant(xd, fmt, mode, gpu)
    rq, rs = o.quantize_mx_rowwise(x, fmt, mode)
    assert np.array_equal(q, rq) and np.array_equal(s, rs)
    cq, cs = o.quantize_mx_colwise_segmented(x, [m], fmt, mode)
    assert np.array_equal(qc, cq) and np.array_equal(sc, cs)
    # each copy alone gives the same bytes as the dual pass
    q1, s1, _, _ = _quant(xd, fmt, mode, gpu, col=False)
    _, _, qc1, sc1 = _quant(xd, fmt, mode, gpu, row=False)
    assert np.array_equal(q1, rq) and np.array_equal(s1, rs) and np.array_equal(qc1, cq) and np.array_equal(sc1, cs)


@pytest.mark.parametrize("fmt,fn", FMTS)
@pytest.mark.parametrize(
    "lens",
    [[33, 0, 130, 1, 136], [0, 0, 5], [128, 256], [1], [0], [127, 129, 0, 0, 64], [7] * 40],
)
def test_ragged_segments_vs_oracle(gpu, fmt, fn, lens):
    """Expert boundaries: blocks restart at each boundary, empty and tiny experts."""
    m = sum(lens)
    g = torch.Generator().manual_seed(len(lens) * 100 + m)
    x = torch.randn(max(m, 1), 96, generator=g).bfloat16()[:m]
    xd = x.to(gpu)
    q, s, qc, sc = _quant(xd, fmt, 0, gpu, lens=lens)
    if m:
        rq, rs = o.quantize_mx_rowwise(x, fmt)
        assert np.array_equal(q, rq) and np.array_equal(s, rs)
    cq, cs = o.quantize_mx_colwise_segmented(x, lens, fmt)
    assert qc.shape == cq.shape and sc.shape == cs.shape
    assert np.array_equal(qc, cq) and np.array_equal(sc, cs)


@pytest.mark.parametrize("fmt,fn", FMTS)
@pytest.mark.parametrize("mode,mn", MODES)
@pytest.mark.parametrize("shape", [(3, 160, 96), (1, 32, 32), (2, 256, 2880), (96, 224)])
def test_weight_2d_vs_oracle(gpu, fmt, fn, mode, mn, shape):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(sum(shape))
    w = (torch.randn(*shape, generator=g) * 0.02).bfloat16()
    got = [_np(t) for t in K.quantize_mx_weight_2d_impl(w.to(gpu), fmt, mode)]
    want = o.quantize_mx_2d(w, fmt, mode)
    for a, b in zip(got, want):
        assert a.shape == b.shape and np.array_equal(a, b)
    # single copies
    r = [_np(t) for t in K.quantize_mx_weight_2d_impl(w.to(gpu), fmt, mode, colwise=False)]
    assert np.array_equal(r[0], want[0]) and r[2] is None
    t = [_np(t) for t in K.quantize_mx_weight_2d_impl(w.to(gpu), fmt, mode, rowwise=False)]
    assert np.array_equal(t[2], want[2]) and np.array_equal(t[3], want[3]) and t[0] is None


@pytest.mark.parametrize("fmt,fn", FMTS)
def test_padded_pitch_for_gemm(gpu, fmt, fn):
    """Row-wise copies padded to the GEMM's K granularity: the real columns match
    the oracle, the padding is zero codes with scale byte 0."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(21)
    x = torch.randn(70, 2880, generator=g).bfloat16()
    q, s, qc, sc = [_np(t) for t in K.quantize_mx_impl(x.to(gpu), fmt, 0, rowwise=True, colwise=True, pad_to=128)]
    per = 2 if fmt == o.FMT_E2M1 else 1
    rq, rs = o.quantize_mx_rowwise(x, fmt)
    assert q.shape == (70, 2944 // per) and s.shape == (70, 92)
    assert np.array_equal(q[:, : 2880 // per], rq) and np.array_equal(s[:, :90], rs)
    assert not q[:, 2880 // per :].any() and not s[:, 90:].any()
    cq, cs = o.quantize_mx_colwise_segmented(x, [70], fmt)
    assert np.array_equal(qc, cq) and np.array_equal(sc, cs)
    w = (torch.randn(2, 96, 160, generator=g) * 0.02).bfloat16()
    got = [_np(t) for t in K.quantize_mx_weight_2d_impl(w.to(gpu), fmt, 0, pad_to=128)]
    want = o.quantize_mx_2d(w, fmt)
    assert got[0].shape == (2, 96, 256 // per) and got[2].shape == (2, 160, 128 // per)
    assert np.array_equal(got[0][..., : 160 // per], want[0]) and np.array_equal(got[1][..., :5], want[1])
    assert np.array_equal(got[2][..., : 96 // per], want[2]) and np.array_equal(got[3][..., :3], want[3])
    assert not got[0][..., 160 // per :].any() and not got[2][..., 96 // per :].any()
    assert not got[1][..., 5:].any() and not got[3][..., 3:].any()


@pytest.mark.parametrize("fmt,fn", FMTS)
def test_special_values(gpu, fmt, fn):
    x = torch.zeros(8, 64).bfloat16()
    x[0, 3] = float("inf")
    x[0, 5] = -2.0
    x[0, 40] = float("nan")
    x[1, 0] = -0.0
    x[2, :] = 1e-38  # bf16 subnormal range -> scale byte clamps at 0
    x[3, :] = 3e38  # near the largest finite bf16
    x[3, 1] = -3.3e38
    x[4, 0] = 448.0
    x[4, 1] = 464.0
    x[4, 2] = 480.0
    x[5, 0] = float("-inf")
    x[6, 33] = 6.0
    x[6, 34] = 5.0
    x[6, 35] = -0.25
    q, s, qc, sc = _quant(x.to(gpu), fmt, 0, gpu)
    rq, rs = o.quantize_mx_rowwise(x, fmt)
    assert np.array_equal(s, rs) and np.array_equal(q, rq)
    cq, cs = o.quantize_mx_colwise_segmented(x, [8], fmt)
    assert np.array_equal(sc, cs) and np.array_equal(qc, cq)


@pytest.mark.parametrize("fmt,fn", FMTS)
def test_dequantize_vs_oracle(gpu, fmt, fn):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(77)
    x = (torch.randn(70, 160, generator=g) * torch.exp2(torch.randint(-40, 40, (70, 1), generator=g).float())).bfloat16()
    x[3] = 0
    q, s = o.quantize_mx_rowwise(x, fmt)
    dt = torch.float8_e4m3fn if fmt == o.FMT_E4M3 else torch.float4_e2m1fn_x2
    out = K.dequantize_mx_impl(torch.from_numpy(q).to(gpu).view(dt), torch.from_numpy(s).to(gpu).view(torch.float8_e8m0fnu))
    want = o.f32_to_bf16_bits(o.dequantize_mx(q, s, fmt))
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), want)


def test_full_size_properties(gpu):
    """Config-3 sized activation [32768, 4096]: size-independent properties.
    (a) quantising an already representable tensor is the identity on codes;
    (b) the transposed copy equals the row-wise copy of the transposed tensor;
    (c) dequantised values are within the format's bound of the input."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator(device=gpu).manual_seed(1003)
    x = torch.randn(32768, 4096, generator=g, device=gpu, dtype=torch.float32).bfloat16()
    lens = torch.tensor([4096, 0, 8000, 1, 6287, 5000, 9384, 0], dtype=torch.int64, device=gpu)
    assert int(lens.sum()) == 32768
    q, s, qc, sc = K.quantize_mx_impl(x, 0, 0, rowwise=True, colwise=True, group_lens=lens)
    dq = K.dequantize_mx_impl(q, s)
    q2, s2, _, _ = K.quantize_mx_impl(dq, 0, 0, rowwise=True, colwise=False)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2.view(torch.uint8), s.view(torch.uint8))
    amax = x.float().abs().view(32768, 128, 32).amax(-1, keepdim=True)
    err = (dq.float() - x.float()).abs().view(32768, 128, 32)
    assert bool((err <= amax * 0.125).all())
    # group 0 starts at padded offset 0 and is 128-aligned: its transposed copy is the plain transpose-quantise
    xt = x[:4096].t().contiguous()
    qt, st, _, _ = K.quantize_mx_impl(xt, 0, 0, rowwise=True, colwise=False)
    assert torch.equal(qc.view(torch.uint8)[:, :4096], qt.view(torch.uint8))
    assert torch.equal(sc.view(torch.uint8)[:, :128], st.view(torch.uint8))


def test_error_codes_not_aborts(gpu):
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    x = torch.zeros(4, 48, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        K.quantize_mx_impl(x, 0)  # 48 is not a multiple of 32
    with pytest.raises(ValueError):
        K.quantize_mx_impl(torch.zeros(4, 64, dtype=torch.bfloat16), 0)  # CPU tensor
    L = _lib.load()
    assert L.mxl_quantize(x.data_ptr(), 4, 48, 0, 0, 0, None, 0, x.data_ptr(), x.data_ptr(), None, None, None) == -1
    assert L.mxl_quantize(x.data_ptr(), 4, 64, 0, 7, 0, None, 0, x.data_ptr(), x.data_ptr(), None, None, None) == -1
    assert L.mxl_quantize(x.data_ptr(), 4, 64, 32, 0, 0, None, 0, x.data_ptr(), x.data_ptr(), None, None, None) == -1  # row_ld < cols
    assert L.mxl_gemm_nt(None, None, 0, None, None, 0, None, 1, 32, 32, None) == -1
