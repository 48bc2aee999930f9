"""The 128-blockwise FP8 recipe on the GPU through the C-ABI: the quantisers' codes and reciprocal scales against the
oracle bit for bit (1 x 128 blocks, the transposed 128 x 1 copy, 128 x 128 weight blocks; E4M3 and E5M2), the GEMM
against the oracle within one bf16 rounding plus the float32 accumulation bound, and the operator / Megatron module
under the recipe against bf16 arithmetic."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
DT = {0: torch.float8_e4m3fn, 2: torch.float8_e5m2}


def _u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def _f(t):
    return o.bf16_bits_to_f32(t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16))


def _x(seed, rows, cols, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, cols, generator=g) * spread * torch.logspace(-2, 1, cols)[None, :]).bfloat16()


@pytest.mark.parametrize("fmt", [0, 2])
@pytest.mark.parametrize("rows,cols", [(1, 128), (37, 256), (128, 128), (200, 384), (513, 1024)])
def test_quantiser_equals_the_oracle(gpu, fmt, rows, cols):
    from primus_amd.pytorch import kernels as K

    x = _x(rows * 7 + cols + fmt, rows, cols, 2.0)
    x[rows // 2, 3] = 0.0
    q, s, qt, st = K.quantize_blockwise_impl(x.to(gpu), fmt, rowwise=True, colwise=True)
    wq, ws = o.quantize_blockwise(x, fmt, axis=-1)
    wqt, wst = o.quantize_blockwise(x, fmt, axis=0)
    assert q.dtype == DT[fmt] and np.array_equal(_u8(q), wq) and np.array_equal(s.cpu().numpy(), ws)
    assert tuple(qt.shape) == wqt.shape and np.array_equal(_u8(qt), wqt) and np.array_equal(st.cpu().numpy(), wst)
    # one copy at a time gives the same bytes
    q1, s1, n1, n2 = K.quantize_blockwise_impl(x.to(gpu), fmt, rowwise=True, colwise=False)
    assert n1 is None and n2 is None and torch.equal(q1.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s1, s)
    n1, n2, qt1, st1 = K.quantize_blockwise_impl(x.to(gpu), fmt, rowwise=False, colwise=True)
    assert n1 is None and torch.equal(qt1.view(torch.uint8), qt.view(torch.uint8)) and torch.equal(st1, st)


@pytest.mark.parametrize("fmt", [0, 2])
@pytest.mark.parametrize("n,k", [(128, 128), (256, 384), (384, 1024)])
def test_weight_quantiser_equals_the_oracle(gpu, fmt, n, k):
    from primus_amd.pytorch import kernels as K

    w = (_x(n + k + fmt, n, k) * 0.02).bfloat16()
    q, s, qt, st = K.quantize_blockwise_weight_impl(w.to(gpu), fmt, rowwise=True, colwise=True)
    wq, ws, wqt, wst = o.quantize_blockwise_2d(w, fmt)
    assert np.array_equal(_u8(q), wq) and np.array_equal(s.cpu().numpy(), ws)
    assert np.array_equal(_u8(qt), wqt) and np.array_equal(st.cpu().numpy(), wst)


def test_zero_and_nonfinite_blocks(gpu):
    from primus_amd.pytorch import kernels as K

    x = torch.zeros(4, 256).bfloat16()
    x[1, 130] = float("inf")
    x[2, 5] = 3.0
    x[3, 200] = float("nan")
    q, s, _, _ = K.quantize_blockwise_impl(x.to(gpu), 0)
    wq, ws = o.quantize_blockwise(x, 0)
    assert np.array_equal(_u8(q), wq)
    fin = np.ones((4, 2), bool)
    fin[3, 1] = False                                        # the reciprocal scale of a block with a NaN is not specified
    assert np.array_equal(s.cpu().numpy()[fin], ws[fin])


@pytest.fixture(params=[128, 256])
def tile(request):
    """Runs the test once per output-tile height of the blockwise GEMMs (the library picks by the shape otherwise)."""
    from primus_amd.pytorch import kernels as K

    K.set_blockwise_gemm_tile(request.param)
    yield request.param
    K.set_blockwise_gemm_tile(0)


def _bound(a_codes, sa, b_codes, sb, a_fmt, b_fmt, want32):
    da = np.abs(o.decode_fp8(a_codes, a_fmt)).astype(np.float64) * np.repeat(np.abs(sa).astype(np.float64), 128, axis=1)
    sbr = sb if sb.shape[0] == b_codes.shape[0] else np.repeat(sb, 128, axis=0)
    db = np.abs(o.decode_fp8(b_codes, b_fmt)).astype(np.float64) * np.repeat(np.abs(sbr).astype(np.float64), 128, axis=1)
    k = a_codes.shape[1]
    return 2.0 ** -8 * np.abs(want32) + (k + 1024) * 2.0 ** -23 * (da @ db.T) + 1e-30


@pytest.mark.parametrize("a_fmt,b_fmt", [(0, 0), (2, 2), (2, 0), (0, 2)])
@pytest.mark.parametrize("m,n,k,per_row", [(70, 128, 128, False), (300, 256, 384, False), (129, 384, 1024, True), (1, 128, 256, True)])
def test_gemm_against_the_oracle(gpu, tile, a_fmt, b_fmt, m, n, k, per_row):
    from primus_amd.pytorch import kernels as K

    x = _x(m + n + k, m, k)
    w = (_x(n * 3 + k, n, k) * 0.05).bfloat16()
    a, sa = o.quantize_blockwise(x, a_fmt)
    if per_row:
        b, sb = o.quantize_blockwise(w, b_fmt)
    else:
        b, sb, _, _ = o.quantize_blockwise_2d(w, b_fmt)
    want32 = o.blockwise_gemm_nt_ref(a, sa, b, sb, a_fmt, b_fmt, out_bf16=False)
    dev = lambda arr, dt=None: (torch.from_numpy(arr).to(gpu) if dt is None else torch.from_numpy(arr).to(gpu).view(dt))
    got = K.gemm_blockwise_nt_impl(dev(a, DT[a_fmt]), dev(sa), dev(b, DT[b_fmt]), dev(sb))
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (m, n)
    err = np.abs(_f(got).astype(np.float64) - want32)
    assert np.all(err <= _bound(a, sa, b, sb, a_fmt, b_fmt, want32))
    assert err.max() <= 1e-2 * np.abs(want32).max()


def test_gemm_is_exact_where_the_arithmetic_is(gpu, tile):
    """Small integers times power-of-two scales: every product and every sum is exact in float32 and in bf16."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(5)
    m, n, k = 200, 256, 512
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    b = torch.randint(-2, 3, (n, k), generator=g).float()
    sa = torch.tensor([0.5, 1.0, 2.0, 4.0])[torch.randint(0, 4, (m, k // 128), generator=g)]
    sb = torch.tensor([0.25, 1.0, 2.0])[torch.randint(0, 3, (n // 128, k // 128), generator=g)]
    want = ((a * sa.repeat_interleave(128, 1)) @ (b * sb.repeat_interleave(128, 0).repeat_interleave(128, 1)).t())
    assert want.abs().max() < 256 * 128                      # stays on bf16's integer grid? checked below
    got = K.gemm_blockwise_nt_impl(a.to(torch.float8_e4m3fn).to(gpu), sa.contiguous().to(gpu),
                                   b.to(torch.float8_e4m3fn).to(gpu), sb.contiguous().to(gpu))
    assert torch.equal(got.float().cpu(), want.bfloat16().float())


def test_both_tile_heights_give_the_same_bits(gpu):
    """Dense (weight factors and per-row factors), grouped forward and grouped weight gradient on shapes with ragged
    row tiles, a half-empty last column tile and several K blocks: the 128 x 256 and the 256 x 256 kernel multiply and
    add in the same order."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(77)
    m, n, k = 777, 640, 896
    x = (torch.randn(m, k, generator=g) * torch.logspace(-2, 1, k)[None, :]).bfloat16().to(gpu)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(gpu)
    lens = [300, 0, 1, 476]
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    wg = (torch.randn(len(lens), n, k, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(m, n, generator=g).bfloat16().to(gpu)
    xq, xs, _, _ = K.quantize_blockwise_impl(x, 0, rowwise=True, colwise=False)
    wq, ws, _, _ = K.quantize_blockwise_weight_impl(w, 0, rowwise=True, colwise=False)
    wr, wrs, _, _ = K.quantize_blockwise_impl(w, 0, rowwise=True, colwise=False)
    wgq, wgs, _, _ = K.quantize_blockwise_weight_impl(wg, 0, rowwise=True, colwise=False)
    _, _, xt, xts = K.quantize_blockwise_impl(x, 2, rowwise=False, colwise=True, group_lens=gl)
    _, _, dt, dts = K.quantize_blockwise_impl(dy, 2, rowwise=False, colwise=True, group_lens=gl)
    out = {}
    try:
        for rows in (128, 256):
            K.set_blockwise_gemm_tile(rows)
            out[rows] = (K.gemm_blockwise_nt_impl(xq, xs, wq, ws), K.gemm_blockwise_nt_impl(xq, xs, wr, wrs),
                         K.gemm_blockwise_nt_impl(xq, xs, wgq, wgs, gl), K.grouped_gemm_blockwise_wgrad_impl(dt, dts, xt, xts, gl, m))
    finally:
        K.set_blockwise_gemm_tile(0)
    for a, b in zip(out[128], out[256]):
        assert torch.isfinite(a.float()).all() and a.float().abs().max() > 0
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    with pytest.raises(Exception):
        K.set_blockwise_gemm_tile(64)


@pytest.mark.parametrize("m,n", [(56 * 256 + 77, 4096), (4096, 14336)])
def test_a_dense_gemm_split_over_both_tile_heights_gives_the_same_bits(gpu, m, n):
    """56.3 x 16 tiles of 256 x 256 are 3.5 rounds on 256 CUs: left to itself the library runs the first 48 row tiles
    on 256-row tiles and the remaining rows (a ragged end included) on 128-row tiles, in two launches; with 16 x 56
    tiles it is the last 8 column tiles that go to the 128-row kernel."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(78)
    k = 256
    x = torch.randn(m, k, generator=g).bfloat16().to(gpu)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(gpu)
    xq, xs, _, _ = K.quantize_blockwise_impl(x, 0, rowwise=True, colwise=False)
    wr, wrs, _, _ = K.quantize_blockwise_impl(w, 2, rowwise=True, colwise=False)
    auto = K.gemm_blockwise_nt_impl(xq, xs, wr, wrs)
    try:
        K.set_blockwise_gemm_tile(128)
        low = K.gemm_blockwise_nt_impl(xq, xs, wr, wrs)
    finally:
        K.set_blockwise_gemm_tile(0)
    assert auto.float().abs().max() > 0 and torch.equal(auto.view(torch.int16), low.view(torch.int16))
    want = x[-300:].float() @ w.float().t()
    assert _cos(auto[-300:], want) > 0.998


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()


@pytest.mark.parametrize("hybrid", [False, True])
def test_operator_forward_and_backward_follow_the_oracle_and_bf16(gpu, hybrid):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    cfg = Float8QuantConfig(format=Format.HYBRID if hybrid else Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    bwd = o.FMT_E5M2 if hybrid else o.FMT_E4M3
    x = _x(1, 300, 256).to(gpu).requires_grad_()
    w = (_x(2, 384, 256) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = _x(3, 300, 384).to(gpu)
    y = turbo.ops.gemm_fp8(x, w, config=cfg)
    dx, dw = torch.autograd.grad(y, [x, w], dy)
    # forward: X row-wise x W in 2-D blocks; dgrad: dY row-wise x W^T; wgrad: dY^T x X^T, blocks along the tokens
    xa, xs = o.quantize_blockwise(x.detach().cpu(), o.FMT_E4M3)
    wq, ws, _, _ = o.quantize_blockwise_2d(w.detach().cpu(), o.FMT_E4M3)
    want_y = o.blockwise_gemm_nt_ref(xa, xs, wq, ws, out_bf16=False)
    da, ds = o.quantize_blockwise(dy.cpu(), bwd)
    _, _, wt, wts = o.quantize_blockwise_2d(w.detach().cpu(), bwd)
    want_dx = o.blockwise_gemm_nt_ref(da, ds, wt, wts, bwd, bwd, out_bf16=False)
    dt_, dts = o.quantize_blockwise(dy.cpu(), bwd, axis=0)
    xt, xts = o.quantize_blockwise(x.detach().cpu(), bwd, axis=0)
    want_dw = o.blockwise_gemm_nt_ref(dt_, dts, xt, xts, bwd, bwd, out_bf16=False)
    for got, want in ((y, want_y), (dx, want_dx), (dw, want_dw)):
        assert tuple(got.shape) == want.shape
        assert np.abs(_f(got) - want).max() <= 1e-2 * np.abs(want).max()
    xr, wr = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    yr = xr @ wr.t()
    dxr, dwr = torch.autograd.grad(yr, [xr, wr], dy)
    bar = 0.99 if hybrid else 0.998
    assert _cos(y, yr) > 0.998 and _cos(dx, dxr) > bar and _cos(dw, dwr) > bar


def test_operator_refuses_what_the_recipe_does_not_cover(gpu):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    x = torch.zeros(8, 96, device=gpu).bfloat16()
    w = torch.zeros(128, 96, device=gpu).bfloat16()
    with pytest.raises(ValueError):
        turbo.ops.gemm_fp8(x, w, config=cfg)                       # K is not a multiple of 128
    wg = torch.zeros(2, 96, 128, device=gpu).bfloat16()
    with pytest.raises(ValueError):
        turbo.ops.grouped_gemm_fp8(torch.zeros(8, 128, device=gpu).bfloat16(), wg, torch.tensor([4, 4], device=gpu), config=cfg)   # N = 96
    with pytest.raises(NotImplementedError):
        turbo.ops.rmsnorm_gemm_fp8(torch.zeros(8, 128, device=gpu).bfloat16(), torch.ones(128, device=gpu).bfloat16(), 1e-5,
                                   torch.zeros(128, 128, device=gpu).bfloat16(), config=cfg)


@pytest.mark.parametrize("microbatches", [1, 2])
def test_megatron_linear_under_the_blockwise_recipe(gpu, microbatches):
    from types import SimpleNamespace

    from primus_amd.megatron import runtime
    from primus_amd.megatron.extensions import primus_turbo as pt
    from primus_amd.pytorch.core import Format, ScalingGranularity

    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.bind()
    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=True)
    runtime.set_num_microbatches(microbatches)
    try:
        qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.BLOCKWISE, format=Format.E4M3, block_size=128)
        assert qc.block_scaling() and not qc.mxfp8_scaling() and not qc.current_scaling()
        torch.manual_seed(3)
        cfg = SimpleNamespace(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                              tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                              layernorm_epsilon=1e-5)
        lin = pt.PrimusTurboLinear(256, 384, parallel_mode=None, config=cfg, bias=False, skip_bias_add=False)
        lin.weight.main_grad = torch.zeros_like(lin.weight, dtype=torch.float32)
        lin.weight.grad_added_to_main_grad = False
        x = torch.randn(16, 8, 256, device=gpu).bfloat16().requires_grad_()
        dy = torch.randn(16, 8, 384, device=gpu).bfloat16()
        with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
            y, _ = lin(x)
        y.backward(dy)
        xr = x.detach().clone().requires_grad_()
        wr = lin.weight.detach().clone().requires_grad_()
        yr = torch.nn.functional.linear(xr, wr)
        yr.backward(dy)
        assert _cos(y, yr) > 0.998 and _cos(x.grad, xr.grad) > 0.998 and _cos(lin.weight.grad, wr.grad) > 0.998
    finally:
        pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
        runtime.set_args()
        runtime.set_num_microbatches(1)


GROUPS = [([5, 0, 130, 64, 0, 1], 256), ([128, 128], 128), ([300], 384), ([0, 0, 7], 128), ([1] * 40 + [0] * 5 + [200], 256)]


@pytest.mark.parametrize("fmt", [0, 2])
@pytest.mark.parametrize("lens,cols", GROUPS)
def test_grouped_quantiser_equals_the_oracle(gpu, fmt, lens, cols):
    """The copy with blocks along the tokens of a grouped tensor: transposed, segment-padded, blocks restarting at
    every group; the row-wise copy of the same launch is the ungrouped one."""
    from primus_amd.pytorch import kernels as K

    rows = sum(lens)
    x = _x(rows + cols + fmt, rows, cols, 2.0)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    q, s, qt, st = K.quantize_blockwise_impl(x.to(gpu), fmt, rowwise=True, colwise=True, group_lens=gl)
    wq, ws = o.quantize_blockwise(x, fmt, axis=-1)
    wqt, wst = o.quantize_blockwise_segmented(x, lens, fmt)
    assert np.array_equal(_u8(q), wq) and np.array_equal(s.cpu().numpy(), ws)
    assert tuple(qt.shape) == wqt.shape == (cols, o.padded_width(rows, len(lens), 128))
    assert np.array_equal(_u8(qt), wqt) and np.array_equal(st.cpu().numpy(), wst)


@pytest.mark.parametrize("fmt", [0, 2])
def test_weight_batch_equals_the_oracle(gpu, fmt):
    from primus_amd.pytorch import kernels as K

    w = (_x(9 + fmt, 3 * 256, 384) * 0.02).bfloat16().reshape(3, 256, 384)
    q, s, qt, st = K.quantize_blockwise_weight_impl(w.to(gpu), fmt, rowwise=True, colwise=True)
    for e in range(3):
        wq, ws, wqt, wst = o.quantize_blockwise_2d(w[e], fmt)
        assert np.array_equal(_u8(q[e]), wq) and np.array_equal(s[e].cpu().numpy(), ws)
        assert np.array_equal(_u8(qt[e]), wqt) and np.array_equal(st[e].cpu().numpy(), wst)


@pytest.mark.parametrize("a_fmt,b_fmt", [(0, 0), (2, 2)])
@pytest.mark.parametrize("lens,k", GROUPS)
def test_grouped_gemms_against_the_oracle(gpu, tile, a_fmt, b_fmt, lens, k):
    from primus_amd.pytorch import kernels as K

    rows, G, n = sum(lens), len(lens), 256
    x = _x(rows + k, rows, k)
    w = (_x(n * G + k, G * n, k) * 0.05).bfloat16().reshape(G, n, k)
    dy = _x(rows + n + 1, rows, n)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    dev = lambda arr, dt=None: (torch.from_numpy(arr).to(gpu) if dt is None else torch.from_numpy(arr).to(gpu).view(dt))
    # forward shape: rows of a grouped, one weight per group
    a, sa = o.quantize_blockwise(x, a_fmt)
    bq = [o.quantize_blockwise_2d(w[e], b_fmt) for e in range(G)]
    b, sb = np.stack([t[0] for t in bq]), np.stack([t[1] for t in bq])
    want = o.grouped_blockwise_gemm_nt_ref(a, sa, b, sb, lens, a_fmt, b_fmt, out_bf16=False)
    got = K.gemm_blockwise_nt_impl(dev(a, DT[a_fmt]), dev(sa), dev(b, DT[b_fmt]), dev(sb), gl)
    assert tuple(got.shape) == (rows, n)
    err = np.abs(_f(got).astype(np.float64) - want)
    assert err.max() <= 1e-2 * max(np.abs(want).max(), 1e-30)
    pos = 0
    for e, ln in enumerate(lens):
        if ln:
            assert np.all(err[pos:pos + ln] <= _bound(a[pos:pos + ln], sa[pos:pos + ln], b[e], sb[e], a_fmt, b_fmt, want[pos:pos + ln]))
        pos += ln
    # wgrad shape: contraction over each group's token segment
    at, sat = o.quantize_blockwise_segmented(dy, lens, a_fmt)
    bt, sbt = o.quantize_blockwise_segmented(x, lens, b_fmt)
    want_w = o.grouped_blockwise_wgrad_ref(at, sat, bt, sbt, lens, a_fmt, b_fmt, out_bf16=False)
    got_w = K.grouped_gemm_blockwise_wgrad_impl(dev(at, DT[a_fmt]), dev(sat), dev(bt, DT[b_fmt]), dev(sbt), gl, rows)
    assert tuple(got_w.shape) == (G, n, k)
    gw = _f(got_w).reshape(G, n, k)
    for e, ln in enumerate(lens):
        if ln == 0:
            assert not gw[e].any()
        else:
            assert np.abs(gw[e] - want_w[e]).max() <= 1e-2 * np.abs(want_w[e]).max()


@pytest.mark.parametrize("hybrid", [False, True])
def test_grouped_operator_follows_bf16(gpu, hybrid):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    cfg = Float8QuantConfig(format=Format.HYBRID if hybrid else Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    lens = [100, 0, 257, 27]
    x = _x(1, sum(lens), 256).to(gpu).requires_grad_()
    w = (_x(2, 4 * 384, 256) * 0.05).bfloat16().reshape(4, 384, 256).to(gpu).requires_grad_()
    dy = _x(3, sum(lens), 384).to(gpu)
    gl = torch.tensor(lens, device=gpu)
    y = turbo.ops.grouped_gemm_fp8(x, w, gl, config=cfg)
    dx, dw = torch.autograd.grad(y, [x, w], dy)
    xr, wr = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    yr = torch.cat([xs @ wr[e].t() for e, xs in enumerate(torch.split(xr, lens))])
    dxr, dwr = torch.autograd.grad(yr, [xr, wr], dy)
    bar = 0.99 if hybrid else 0.998
    assert _cos(y, yr) > 0.998 and _cos(dx, dxr) > bar and _cos(dw, dwr) > bar
    assert not dw[1].any()


def test_megatron_grouped_linear_under_the_blockwise_recipe(gpu):
    from types import SimpleNamespace

    from primus_amd.megatron import runtime
    from primus_amd.megatron.extensions import primus_turbo as pt
    from primus_amd.pytorch.core import Format, ScalingGranularity

    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.bind()
    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=True)
    runtime.set_num_microbatches(2)
    try:
        qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.BLOCKWISE, format=Format.E4M3, block_size=128)
        torch.manual_seed(4)
        cfg = SimpleNamespace(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                              tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                              layernorm_epsilon=1e-5)
        lens = [33, 0, 130, 1, 92]
        gl = pt.PrimusTurboColumnParallelGroupedLinear(5, 128, 256, config=cfg)
        xg = torch.randn(sum(lens), 128, device=gpu).bfloat16().requires_grad_()
        dyg = torch.randn(sum(lens), 256, device=gpu).bfloat16()
        with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
            yg, _ = gl(xg, torch.tensor(lens))
        yg.backward(dyg)
        want = torch.cat([xs @ gl.weights[e].detach().t() for e, xs in enumerate(torch.split(xg.detach(), lens))])
        assert _cos(yg, want) > 0.998
        assert not gl.weights.grad[1].any() and gl.weights.grad[0].abs().sum() > 0
    finally:
        pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
        runtime.set_args()
        runtime.set_num_microbatches(1)


def test_operator_replays_under_a_graph(gpu):
    """Forward and backward of the dense operator captured once (after an eager pass, so every kernel's launch
    attributes are in place before the capture) and replayed on new inputs: every replay equals the eager result."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    x = _x(1, 300, 256).to(gpu).requires_grad_()
    w = (_x(2, 384, 256) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = _x(3, 300, 384).to(gpu)

    def step():
        y = turbo.ops.gemm_fp8(x, w, config=cfg)
        dx, dw = torch.autograd.grad(y, [x, w], dy)
        return y, dx, dw

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for seed in (4, 5, 6):
        with torch.no_grad():
            x.copy_(_x(seed, 300, 256))
            dy.copy_(_x(seed + 10, 300, 384))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for u, v in zip(got, want):
            assert torch.equal(u.view(torch.int16), v.view(torch.int16)), seed


def _exact_operands(gen, m, n, k, per_row, dev):
    """Small integers times power-of-two factors: every product and partial sum is exact in float32 whatever the order."""
    a = torch.randint(-2, 3, (m, k), generator=gen, device=dev).float()
    b = torch.randint(-2, 3, (n, k), generator=gen, device=dev).float()
    sa = torch.tensor([0.5, 1.0, 2.0, 4.0], device=dev)[torch.randint(0, 4, (m, k // 128), generator=gen, device=dev)]
    sb_rows = n if per_row else n // 128
    sb = torch.tensor([0.25, 1.0, 2.0], device=dev)[torch.randint(0, 3, (sb_rows, k // 128), generator=gen, device=dev)]
    bs = b * (sb if per_row else sb.repeat_interleave(128, 0)).repeat_interleave(128, 1)
    want = ((a * sa.repeat_interleave(128, 1)) @ bs.t()).bfloat16()
    return a, sa.contiguous(), b, sb.contiguous(), want


@pytest.mark.parametrize("m,n,k,per_row", [(8192, 14336, 4096, False), (8192, 4096, 14336, False), (14336, 4096, 8192, True)])
def test_llama_mlp_shapes_at_full_size_are_exact(gpu, m, n, k, per_row):
    """The three GEMMs of the Llama-3-8B MLP under this recipe at their real sizes (forward, dgrad, weight gradient: the
    last one is split over both tile heights) on operands whose exact result does not depend on the order of the sums."""
    from primus_amd.pytorch import kernels as K

    gen = torch.Generator(device=gpu).manual_seed(m + n + k)
    a, sa, b, sb, want = _exact_operands(gen, m, n, k, per_row, gpu)
    fa, fb = (torch.float8_e5m2, torch.float8_e5m2) if per_row else (torch.float8_e4m3fn, torch.float8_e4m3fn)
    got = K.gemm_blockwise_nt_impl(a.to(fa), sa, b.to(fb), sb, b_rows_per_scale=1 if per_row else 128)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_seeded_sweep_of_ragged_gemms_under_every_tile_height(gpu):
    """40 random shapes (dense with either kind of b factors, grouped forward with empty and ragged groups): the 128-row
    kernel, the 256-row kernel and the library's choice give the same bits, and they are the exact result."""
    import random

    from primus_amd.pytorch import kernels as K

    rnd = random.Random(2024)
    gen = torch.Generator(device=gpu).manual_seed(2024)
    try:
        for case in range(40):
            n, k = 128 * rnd.randint(1, 10), 128 * rnd.randint(1, 5)
            if case % 2 == 0:
                m, per_row = rnd.choice([1, 127, 129, 255, 257, 700, rnd.randint(1, 3000)]), rnd.random() < 0.5
                a, sa, b, sb, want = _exact_operands(gen, m, n, k, per_row, gpu)
                run = lambda: K.gemm_blockwise_nt_impl(a.to(torch.float8_e4m3fn), sa, b.to(torch.float8_e5m2), sb,
                                                       b_rows_per_scale=1 if per_row else 128)
            else:
                lens = [rnd.choice([0, 1, 128, 129, 255, 256, 257, 513, rnd.randint(1, 900)]) for _ in range(rnd.randint(1, 7))]
                lens[rnd.randrange(len(lens))] += 1
                m, G = sum(lens), len(lens)
                a, sa, _, _, _ = _exact_operands(gen, m, 128, k, False, gpu)
                ws = [_exact_operands(gen, 1, n, k, False, gpu) for _ in range(G)]
                b, sb = torch.stack([w[2] for w in ws]), torch.stack([w[3] for w in ws])
                asc, rows, off = a * sa.repeat_interleave(128, 1), [], 0
                for e, ln in enumerate(lens):
                    rows.append(asc[off:off + ln] @ (b[e] * sb[e].repeat_interleave(128, 0).repeat_interleave(128, 1)).t())
                    off += ln
                want = torch.cat(rows).bfloat16()
                gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
                run = lambda: K.gemm_blockwise_nt_impl(a.to(torch.float8_e4m3fn), sa, b.to(torch.float8_e4m3fn), sb, gl)
            outs = []
            for rows_ in (128, 256, 0):
                K.set_blockwise_gemm_tile(rows_)
                outs.append(run())
            for o_ in outs:
                assert torch.equal(o_.view(torch.int16), want.view(torch.int16)), (case, m, n, k)
    finally:
        K.set_blockwise_gemm_tile(0)


def test_mixtral_routing_at_full_row_count_is_exact(gpu):
    """32 768 routed rows in the benchmark's eight ragged groups against per-group weights (n and k of fc2's dgrad):
    the grouped forward kernel on 256-row tiles, exact on exactly representable operands."""
    from primus_amd.pytorch import kernels as K

    lens = [3615, 1451, 2686, 6852, 6436, 4634, 1493, 5601]
    m, G, n, k = sum(lens), len(lens), 4096, 4096
    gen = torch.Generator(device=gpu).manual_seed(11)
    a, sa, _, _, _ = _exact_operands(gen, m, 128, k, False, gpu)
    ws = [_exact_operands(gen, 1, n, k, False, gpu) for _ in range(G)]
    b, sb = torch.stack([w[2] for w in ws]), torch.stack([w[3] for w in ws])
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    got = K.gemm_blockwise_nt_impl(a.to(torch.float8_e4m3fn), sa, b.to(torch.float8_e4m3fn), sb, gl)
    asc, off = a * sa.repeat_interleave(128, 1), 0
    for e, ln in enumerate(lens):
        want = (asc[off:off + ln] @ (b[e] * sb[e].repeat_interleave(128, 0).repeat_interleave(128, 1)).t()).bfloat16()
        assert torch.equal(got[off:off + ln].view(torch.int16), want.view(torch.int16)), e
        off += ln


def test_a_split_launch_replays_under_a_graph(gpu):
    """The GEMM whose output the library splits over the two tile heights (two launches per call) captured once, after
    an eager call, and replayed on new operands: every replay equals the eager result."""
    from primus_amd.pytorch import kernels as K

    gen = torch.Generator(device=gpu).manual_seed(5)
    m, n, k = 56 * 256 + 77, 4096, 256
    a, sa, b, sb, _ = _exact_operands(gen, m, n, k, True, gpu)
    aq, bq = a.to(torch.float8_e5m2), b.to(torch.float8_e5m2)
    run = lambda: K.gemm_blockwise_nt_impl(aq, sa, bq, sb, b_rows_per_scale=1)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run()
    for seed in (6, 7, 8):
        a2, sa2, _, _, _ = _exact_operands(torch.Generator(device=gpu).manual_seed(seed), m, 128, k, True, gpu)
        with torch.no_grad():
            aq.copy_(a2.to(torch.float8_e5m2))
            sa.copy_(sa2)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run()
        torch.cuda.synchronize()
        assert want.float().abs().max() > 0 and torch.equal(got.view(torch.int16), want.view(torch.int16)), seed


def test_an_output_that_is_only_8_byte_aligned(gpu):
    """The C entry point accepts an output pointer aligned to 8 bytes: such a call stays on the 128-row kernel and stores
    straight from the accumulator layout, with the same bits as the aligned call (and a misaligned one is refused)."""
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    gen = torch.Generator(device=gpu).manual_seed(21)
    m, n, k = 777, 384, 512
    a, sa, b, sb, want = _exact_operands(gen, m, n, k, False, gpu)
    aq, bq = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    buf = torch.zeros(m * n + 16, dtype=torch.bfloat16, device=gpu)
    lib, stream = _lib.load(), torch.cuda.current_stream().cuda_stream
    for tile in (0, 256):
        K.set_blockwise_gemm_tile(tile)
        try:
            buf.zero_()
            rc = lib.mxl_gemm_nt_blockwise(aq.data_ptr(), sa.data_ptr(), 0, bq.data_ptr(), sb.data_ptr(), 0, 128, buf.data_ptr() + 8, m, n, k, stream)
        finally:
            K.set_blockwise_gemm_tile(0)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(buf[4:4 + m * n].view(m, n).view(torch.int16), want.view(torch.int16))
        assert not buf[:4].any() and not buf[4 + m * n:].any()
    assert lib.mxl_gemm_nt_blockwise(aq.data_ptr(), sa.data_ptr(), 0, bq.data_ptr(), sb.data_ptr(), 0, 128, buf.data_ptr() + 2, m, n, k, stream) != 0
