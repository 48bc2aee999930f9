"""Tensor-wise ("current") FP8 scaling on the GPU: abs-max, the quantiser's codes and reciprocal scale
against the oracle bit for bit, the scaled GEMMs against the oracle within 1e-2 of the result's largest
magnitude (and exactly where every product and sum is exact)."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
TOL = 1e-2
DT = {0: torch.float8_e4m3fn, 2: torch.float8_e5m2}


def _u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def _f(t):
    return o.bf16_bits_to_f32(t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16))


def _x(seed, rows, cols, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, cols, generator=g) * spread * torch.logspace(-2, 1, cols)[None, :]).bfloat16()


@pytest.mark.parametrize("n", [1, 7, 8, 9, 4096, 100003, 8 * 256 * 4096 + 5])
def test_amax(gpu, n):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g).bfloat16()
    x[n // 2] = -77.5
    got = K.amax_impl(x.to(gpu))
    assert got.dtype == torch.float32 and got.item() == x.float().abs().max().item() == 77.5
    assert K.amax_impl(torch.empty(0, dtype=torch.bfloat16, device=gpu)).item() == 0.0
    x[0] = float("inf")
    assert K.amax_impl(x.to(gpu)).item() == float("inf")
    x[n - 1] = float("nan")
    assert np.isnan(K.amax_impl(x.to(gpu)).item())


@pytest.mark.parametrize("fmt", [0, 2])
@pytest.mark.parametrize("rows,cols,lens", [(37, 32, None), (300, 160, None), (257, 4096, None),
                                            (256, 96, [33, 0, 130, 1, 92]), (600, 256, [300, 300])])
@pytest.mark.parametrize("kchunk", [False, True, 2])
def test_quantiser_equals_the_oracle(gpu, fmt, rows, cols, lens, kchunk):
    from primus_amd.pytorch import kernels as K

    x = _x(rows + cols + fmt, rows, cols, spread=3.0 if fmt == 0 else 100.0)
    x[0, 0] = 0.0
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    qr, sr, qc, sc, si = K.quantize_tensorwise_impl(x.to(gpu), fmt, rowwise=True, colwise=True, group_lens=gl,
                                                    pad_to=128, kchunk=kchunk)
    want, want_si = o.quantize_tensorwise(x, fmt)
    assert si.cpu().numpy().view(np.uint32)[0] == np.float32(want_si).view(np.uint32)
    assert qr.dtype == DT[fmt] and qc.dtype == DT[fmt]
    row = _u8(K.unchunk(qr) if kchunk else qr)
    assert row.shape[0] == rows and row.shape[1] % 128 == 0
    assert np.array_equal(row[:, :cols], want) and not row[:, cols:].any()
    if kchunk == 2:
        # K-step-major scale panels: the entries of the row-wise copy's K blocks hold the unit byte (the transposed
        # copy's panels restart per expert segment and are covered by the GEMM test below)
        assert np.all(_u8(K.unpanel(sr.view(torch.uint8), row.shape[1] // 32)) == 127)
    else:
        assert np.all(_u8(sr) == 127) and np.all(_u8(sc) == 127)
    # transposed copy: per expert segment, padded to 128 tokens with zero codes
    col = _u8(K.unchunk(qc) if kchunk else qc)
    lens_ = [rows] if lens is None else lens
    pos = 0
    src = 0
    for ln in lens_:
        seg = -(-ln // 128) * 128
        assert np.array_equal(col[:, pos:pos + ln], want[src:src + ln].T)
        assert not col[:, pos + ln:pos + seg].any()
        pos += seg
        src += ln
    assert not col[:, pos:].any()
    # single copies give the same bytes
    r1 = K.quantize_tensorwise_impl(x.to(gpu), fmt, rowwise=True, colwise=False, pad_to=128, kchunk=kchunk)
    c1 = K.quantize_tensorwise_impl(x.to(gpu), fmt, rowwise=False, colwise=True, group_lens=gl, kchunk=kchunk)
    assert torch.equal(r1[0].view(torch.uint8), qr.view(torch.uint8)) and torch.equal(c1[2].view(torch.uint8), qc.view(torch.uint8))


@pytest.mark.parametrize("fmt", [0, 2])
def test_quantiser_special_tensors(gpu, fmt):
    from primus_amd.pytorch import kernels as K

    z = torch.zeros(64, 64, dtype=torch.bfloat16)
    q, _, _, _, si = K.quantize_tensorwise_impl(z.to(gpu), fmt)
    want, want_si = o.quantize_tensorwise(z, fmt)
    assert not _u8(q).any() and si.item() == float(want_si)
    x = _x(1, 64, 64)
    x[3, 5] = float("inf")
    q, _, _, _, si = K.quantize_tensorwise_impl(x.to(gpu), fmt)
    assert np.all(_u8(q) == 0x7F)                    # every code NaN
    want, _ = o.quantize_tensorwise(x, fmt)
    assert np.array_equal(_u8(q), want)
    # the largest element lands on the format's largest value, sign kept
    x = _x(2, 64, 64)
    x[7, 9] = -1000.0
    q, _, _, _, si = K.quantize_tensorwise_impl(x.to(gpu), fmt)
    assert _u8(q)[7, 9] == (0xFE if fmt == 0 else 0xFB)


@pytest.mark.parametrize("fmt", [0, 2])
@pytest.mark.parametrize("shape", [(96, 160), (3, 256, 128), (2, 416, 288)])
@pytest.mark.parametrize("kchunk", [False, True, 2])
def test_weight_quantiser_equals_the_oracle(gpu, fmt, shape, kchunk):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(sum(shape))
    w = (torch.randn(*shape, generator=g) * 0.05).bfloat16()
    qr, sr, qc, sc, si = K.quantize_weight_tensorwise_impl(w.to(gpu), fmt, rowwise=True, colwise=True, pad_to=128, kchunk=kchunk)
    n, k = shape[-2], shape[-1]
    want, want_si = o.quantize_tensorwise(w.reshape(-1, k), fmt)
    assert si.item() == float(want_si)
    row = _u8(K.unchunk(qr) if kchunk else qr).reshape(-1, -(-k // 128) * 128)
    assert np.array_equal(row[:, :k], want) and not row[:, k:].any()
    col = _u8(K.unchunk(qc) if kchunk else qc).reshape(-1, k, -(-n // 128) * 128)
    wt = want.reshape(-1, n, k).transpose(0, 2, 1)
    assert np.array_equal(col[:, :, :n], wt) and not col[:, :, n:].any()


@pytest.mark.parametrize("afmt", [0, 2])
@pytest.mark.parametrize("lens,n,k", [(None, 96, 160), ([33, 0, 130, 1, 92], 160, 96), ([300, 212], 384, 256), (None, 512, 1024)])
@pytest.mark.parametrize("kchunk", [False, True, 2])
def test_scaled_gemms_vs_oracle(gpu, afmt, lens, n, k, kchunk):
    from primus_amd.pytorch import kernels as K

    rows = 200 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + n + k)
    x = torch.randn(rows, k, generator=g).bfloat16()
    w = (torch.randn(*((n, k) if lens is None else (len(lens), n, k)), generator=g) * 0.05).bfloat16()
    dy = torch.randn(rows, n, generator=g).bfloat16()
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    lens_ = [rows] if lens is None else lens
    # forward-shaped GEMM: a = x (afmt) , b = w (E4M3)
    xa = K.quantize_tensorwise_impl(x.to(gpu), afmt, rowwise=True, colwise=True, group_lens=gl, pad_to=128, kchunk=kchunk)
    wq = K.quantize_weight_tensorwise_impl(w.to(gpu), 0, rowwise=True, colwise=True, pad_to=128, kchunk=kchunk)
    y = K.gemm_tw_nt_impl(xa[0], xa[1], xa[4], wq[0], wq[1], wq[4], gl, kchunk=kchunk)
    xc, xsi = o.quantize_tensorwise(x, afmt)
    wc, wsi = o.quantize_tensorwise(w.reshape(-1, k), 0)
    wc = wc.reshape(-1, n, k)
    want = np.zeros((rows, n), dtype=np.float32)
    pos = 0
    for e, ln in enumerate(lens_):
        want[pos:pos + ln] = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(xc[pos:pos + ln], xsi, wc[e], wsi, afmt, 0))
        pos += ln
    assert y.shape == (rows, n)
    assert np.abs(_f(y) - want).max() <= TOL * np.abs(want).max()
    # wgrad-shaped GEMM: a = dy^T (afmt), b = x^T (E4M3)
    da = K.quantize_tensorwise_impl(dy.to(gpu), afmt, rowwise=False, colwise=True, group_lens=gl, kchunk=kchunk)
    xb = K.quantize_tensorwise_impl(x.to(gpu), 0, rowwise=False, colwise=True, group_lens=gl, kchunk=kchunk)
    dw = K.gemm_tw_wgrad_impl(da[2], da[3], da[4], xb[2], xb[3], xb[4], gl, rows, kchunk=kchunk)
    dc, dsi = o.quantize_tensorwise(dy, afmt)
    xc0, xsi0 = o.quantize_tensorwise(x, 0)
    pos = 0
    got = _f(dw).reshape(-1, n, k)
    for e, ln in enumerate(lens_):
        if ln == 0:
            assert not got[e].any()
            continue
        want_e = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(dc[pos:pos + ln].T, dsi, xc0[pos:pos + ln].T, xsi0, afmt, 0))
        assert np.abs(got[e] - want_e).max() <= TOL * np.abs(want_e).max()
        pos += ln


@pytest.mark.parametrize("afmt", [0, 2])
def test_scaled_gemm_is_exact_on_exact_operands(gpu, afmt):
    """Codes of small integers and power-of-two factors: every product, sum and the scaling are exact, so the
    output equals the integer matrix product bit for bit."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(5)
    rows, n, k = 384, 256, 256
    a_int = rng.integers(-3, 4, size=(rows, k))
    b_int = rng.integers(-4, 5, size=(n, k))
    a_codes = (o.cast_e5m2 if afmt == 2 else o.cast_e4m3)(a_int.astype(np.float32))
    b_codes = o.cast_e4m3(b_int.astype(np.float32))
    dev = lambda arr, dt: torch.from_numpy(arr).to(gpu).view(dt)  # noqa: E731
    ones = lambda r: torch.full((r, k // 32), 127, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)  # noqa: E731
    sa = torch.tensor([0.5], device=gpu)
    sb = torch.tensor([0.25], device=gpu)
    y = K.gemm_tw_nt_impl(dev(a_codes, DT[afmt]), ones(rows), sa, dev(b_codes, DT[0]), ones(n), sb)
    want = (a_int @ b_int.T).astype(np.float32) * 0.125
    assert np.array_equal(_f(y), o.bf16_bits_to_f32(o.f32_to_bf16_bits(want)))


@pytest.mark.parametrize("kchunk", [False, True, 2])
def test_e5m2_times_e5m2_is_exact_on_exact_operands(gpu, kchunk):
    """Both operands in the gradient format (the FP8 backward of the MXFP4 linear re-quantises dY, X and W to E5M2):
    forward-shaped and wgrad-shaped GEMMs on integer codes, bit for bit, then through the quantisers in every layout
    (row-major and K-chunk-major: 2-slot kernel; K-step-major: ring kernel) against the oracle."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(17)
    lens = [130, 0, 62, 192]
    rows, n, k = sum(lens), 160, 256
    a_int = torch.randint(-3, 4, (rows, k), generator=g).float()
    d_int = torch.randint(-3, 4, (rows, n), generator=g).float()
    w_int = torch.randint(-3, 4, (len(lens), n, k), generator=g).float()
    # first the GEMM alone on codes written here (small integers are exact in E5M2, the factors are powers of two)
    def codes(t):
        return torch.from_numpy(o.cast_e5m2(t.numpy().astype(np.float32))).view(torch.float8_e5m2)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    one = torch.ones(1, device=gpu)
    half = torch.full((1,), 0.5, device=gpu)
    unit = lambda r, c: torch.full((r, c // 32), 127, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)  # noqa: E731
    if not kchunk:
        y = K.gemm_tw_nt_impl(codes(a_int).to(gpu), unit(rows, k), one, codes(w_int).to(gpu), unit(len(lens) * n, k).view(len(lens), n, -1),
                              half, gl)
        want = torch.cat([a @ w_int[e].T for e, a in enumerate(torch.split(a_int, lens))]) * 0.5
        assert torch.equal(y.float().cpu(), want.bfloat16().float())
    # through the quantisers (tensor-wise, E5M2 for every operand) against the oracle
    x = (a_int * 0.37).bfloat16(); dy = (d_int * 1.3).bfloat16(); w = (w_int * 0.011).bfloat16()
    da = K.quantize_tensorwise_impl(dy.to(gpu), 2, rowwise=True, colwise=True, group_lens=gl, pad_to=128, kchunk=kchunk)
    xa = K.quantize_tensorwise_impl(x.to(gpu), 2, rowwise=False, colwise=True, group_lens=gl, kchunk=kchunk)
    wq = K.quantize_weight_tensorwise_impl(w.to(gpu), 2, rowwise=False, colwise=True, pad_to=128, kchunk=kchunk)
    dx = K.gemm_tw_nt_impl(da[0], da[1], da[4], wq[2], wq[3], wq[4], gl, kchunk=kchunk)[:, :k]
    dw = K.gemm_tw_wgrad_impl(da[2], da[3], da[4], xa[2], xa[3], xa[4], gl, rows, kchunk=kchunk)
    dc, dsi = o.quantize_tensorwise(dy, 2)
    xc, xsi = o.quantize_tensorwise(x, 2)
    wc, wsi = o.quantize_tensorwise(w.reshape(-1, k), 2)
    wc = wc.reshape(-1, n, k)
    pos = 0
    for e, ln in enumerate(lens):
        if ln:
            want_dx = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(dc[pos:pos + ln], dsi, np.ascontiguousarray(wc[e].T), wsi, 2, 2))
            assert np.abs(_f(dx)[pos:pos + ln] - want_dx).max() <= TOL * max(np.abs(want_dx).max(), 1e-30)
            want_dw = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(np.ascontiguousarray(dc[pos:pos + ln].T), dsi,
                                                                  np.ascontiguousarray(xc[pos:pos + ln].T), xsi, 2, 2))
            assert np.abs(_f(dw)[e] - want_dw).max() <= TOL * max(np.abs(want_dw).max(), 1e-30)
        else:
            assert not _f(dw)[e].any()
        pos += ln


def _tw_cfg(hybrid):
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    return Float8QuantConfig(format=Format.HYBRID if hybrid else Format.E4M3, granularity=ScalingGranularity.TENSORWISE)


@pytest.mark.parametrize("hybrid", [False, True])
@pytest.mark.parametrize("lens,n,k", [(None, 96, 160), ([33, 0, 130, 1, 92], 160, 96), ([300, 212], 384, 256)])
def test_operators_forward_backward_vs_oracle(gpu, hybrid, lens, n, k):
    """gemm_fp8 / grouped_gemm_fp8 under the tensor-wise recipe: forward, dgrad and wgrad against the oracle's
    quantise -> decode -> float32 matmul -> scale, per expert (operand flow of
    primus_turbo_float8_local.py:215-306)."""
    import primus_amd.pytorch as turbo

    cfg = _tw_cfg(hybrid)
    bfmt = o.FMT_E5M2 if hybrid else o.FMT_E4M3
    rows = 200 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + n + k)
    x = torch.randn(rows, k, generator=g).bfloat16()
    w = (torch.randn(*((n, k) if lens is None else (len(lens), n, k)), generator=g) * 0.05).bfloat16()
    dy = torch.randn(rows, n, generator=g).bfloat16()
    xd, wd = x.to(gpu).requires_grad_(), w.to(gpu).requires_grad_()
    if lens is None:
        y = turbo.ops.gemm_fp8(xd, wd, config=cfg)
    else:
        y = turbo.ops.grouped_gemm_fp8(xd, wd, torch.tensor(lens, device=gpu), config=cfg)
    dx, dw = torch.autograd.grad(y, [xd, wd], dy.to(gpu))
    xc, xsi = o.quantize_tensorwise(x, o.FMT_E4M3)
    wc, wsi = o.quantize_tensorwise(w.reshape(-1, k), o.FMT_E4M3)
    wc = wc.reshape(-1, n, k)
    dc, dsi = o.quantize_tensorwise(dy, bfmt)
    pos = 0
    gy, gdx, gdw = _f(y), _f(dx), _f(dw).reshape(-1, n, k)
    for e, ln in enumerate([rows] if lens is None else lens):
        sl = slice(pos, pos + ln)
        pos += ln
        if ln == 0:
            assert not gdw[e].any()
            continue
        wy = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(xc[sl], xsi, wc[e], wsi))
        wdx = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(dc[sl], dsi, wc[e].T, wsi, bfmt, o.FMT_E4M3))
        wdw = o.bf16_bits_to_f32(o.tensorwise_gemm_nt_ref(dc[sl].T, dsi, xc[sl].T, xsi, bfmt, o.FMT_E4M3))
        assert np.abs(gy[sl] - wy).max() <= TOL * np.abs(wy).max()
        assert np.abs(gdx[sl] - wdx).max() <= TOL * np.abs(wdx).max()
        assert np.abs(gdw[e] - wdw).max() <= TOL * np.abs(wdw).max()
    # and the recipe is a usable approximation of the bf16 linear
    if lens is None:
        ref = x.float() @ w.float().t()
        assert torch.nn.functional.cosine_similarity(torch.from_numpy(gy).flatten(), ref.flatten(), dim=0) > 0.998


@pytest.mark.parametrize("hybrid", [False, True])
@pytest.mark.parametrize("transpose_cache", [True, False])
def test_cached_weights_give_the_same_results(gpu, hybrid, transpose_cache):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import QuantizedTensorPair, create_quantized_weight, float8_e4m3

    cfg = _tw_cfg(hybrid)
    lens = [70, 0, 58]
    g = torch.Generator().manual_seed(3)
    x = torch.randn(sum(lens), 160, generator=g).bfloat16().to(gpu).requires_grad_()
    w = (torch.randn(3, 96, 160, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(sum(lens), 96, generator=g).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y0 = turbo.ops.grouped_gemm_fp8(x, w, gl, config=cfg)
    (dx0,) = torch.autograd.grad(y0, [x], dy)
    pair = QuantizedTensorPair(*create_quantized_weight(w, float8_e4m3, cfg, need_weight_transpose_cache=transpose_cache))
    assert (pair.data_t is None) is (not transpose_cache) and pair.data.tensor_scale_inv is not None
    assert pair.data.kchunk == 2          # stored for the ring kernel, like the operands of a call on bf16 weights
    y1 = turbo.ops.grouped_gemm_fp8(x, pair, gl, config=cfg)
    (dx1,) = torch.autograd.grad(y1, [x], dy)
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1)
    # caches in the other layouts serve the call as well
    for lay in (0, 1):
        other = QuantizedTensorPair(*create_quantized_weight(w, float8_e4m3, cfg, need_weight_transpose_cache=transpose_cache,
                                                             kchunk=lay))
        y2 = turbo.ops.grouped_gemm_fp8(x, other, gl, config=cfg)
        (dx2,) = torch.autograd.grad(y2, [x], dy)
        assert torch.equal(y0, y2) and torch.equal(dx0, dx2), lay
    deq = pair.data.dequantize()
    assert deq.shape == w.shape and (deq.float() - w.float()).abs().max() <= 0.07 * w.float().abs().max()


def test_operator_argument_errors(gpu):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    x = torch.randn(64, 64, device=gpu).bfloat16()
    w = torch.randn(32, 64, device=gpu).bfloat16()
    with pytest.raises(NotImplementedError):
        turbo.ops.gemm_fp8(x, w, config=Float8QuantConfig(format=Format.E5M2, granularity=ScalingGranularity.TENSORWISE))
    with pytest.raises(NotImplementedError):
        turbo.ops.gemm_fp8(x, w, config=Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.ROWWISE))
    with pytest.raises(NotImplementedError):
        turbo.ops.rmsnorm_gemm_fp8(x, torch.ones(64, device=gpu).bfloat16(), 1e-5, w, config=_tw_cfg(False))
