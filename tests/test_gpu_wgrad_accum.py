"""Gradient-accumulation fusion: the wgrad GEMM adds its result, in float32, to the buffer it is given
(fuse_bgrad_accum_pattern = "megatron" of the reference's operators: the GEMM's beta = 1 epilogue adds into
weight.main_grad, primus/backends/megatron/core/extensions/primus_turbo.py:166-240, 243-275).

Bars: on exactly representable operands buffer_after == buffer_before + integer product, bit for bit; on
random operands (buffer_after - buffer_before) agrees with the separately computed bf16 gradient to the bf16
rounding of that gradient (2^-8 relative) plus float32 rounding of the sum."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _cfg(kind):
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    if kind == "mxfp4":
        return Float4QuantConfig(format=Format.E2M1_X2, granularity=ScalingGranularity.MX_BLOCKWISE,
                                 scale_dtype=ScaleDtype.E8M0, block_size=32)
    if kind == "mxfp8":
        return Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0,
                                 block_size=32)
    return Float8QuantConfig(format=Format.HYBRID if kind == "hybrid" else Format.E4M3, granularity=ScalingGranularity.TENSORWISE)


@pytest.mark.parametrize("lens,n,k", [(None, 96, 160), ([33, 0, 130, 1, 92], 160, 96), ([300, 212], 384, 256), ([0, 0], 64, 64),
                                      ([700, 0, 1300], 544, 320)])
@pytest.mark.parametrize("fmt,layout", [(0, 1), (0, 2), (1, 1), (1, 3)])
def test_kernel_adds_exactly(gpu, lens, n, k, fmt, layout):
    """K-chunk-major operands: the 2-slot kernel loads the old values and stores the sums; K-step-major operands: the ring
    kernel adds with float atomics.  Either way every element receives exactly one float32 add per call."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(n + k)
    rows = 200 if lens is None else sum(lens)
    dy = torch.from_numpy(rng.integers(-3, 4, size=(rows, n)).astype(np.float32)).bfloat16().to(gpu)
    x = torch.from_numpy(rng.integers(-4, 5, size=(rows, k)).astype(np.float32)).bfloat16().to(gpu)
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    G = 1 if lens is None else len(lens)
    shape = (n, k) if lens is None else (G, n, k)
    before = torch.from_numpy(rng.integers(-1000, 1000, size=shape).astype(np.float32)).to(gpu)
    buf = before.clone()
    _, _, dq, ds = K.quantize_mx_impl(dy, fmt, rowwise=False, colwise=True, group_lens=gl, kchunk=layout)
    _, _, xq, xs = K.quantize_mx_impl(x, fmt, rowwise=False, colwise=True, group_lens=gl, kchunk=layout)
    out = K.grouped_gemm_mx_wgrad_impl(dq, ds, xq, xs, gl, rows, kchunk=layout, accum_into=buf)
    assert out.data_ptr() == buf.data_ptr()
    want = before.cpu().numpy().reshape(G, n, k).copy()
    pos = 0
    for e, ln in enumerate([rows] if lens is None else lens):
        want[e] += dy[pos:pos + ln].float().cpu().numpy().T @ x[pos:pos + ln].float().cpu().numpy()
        pos += ln
    assert np.array_equal(buf.cpu().numpy().reshape(G, n, k), want)
    # a second call adds again
    K.grouped_gemm_mx_wgrad_impl(dq, ds, xq, xs, gl, rows, kchunk=layout, accum_into=buf)
    assert np.array_equal(buf.cpu().numpy().reshape(G, n, k), 2 * want - before.cpu().numpy().reshape(G, n, k))
    with pytest.raises(ValueError):
        K.grouped_gemm_mx_wgrad_impl(dq, ds, xq, xs, gl, rows, kchunk=layout, accum_into=buf.bfloat16())
    with pytest.raises(ValueError):
        a = K.quantize_mx_impl(dy, fmt, rowwise=False, colwise=True, group_lens=gl)
        b = K.quantize_mx_impl(x, fmt, rowwise=False, colwise=True, group_lens=gl)
        K.grouped_gemm_mx_wgrad_impl(a[2], a[3], b[2], b[3], gl, rows, accum_into=buf)   # row-major operands


@pytest.mark.parametrize("kind", ["mxfp8", "mxfp4", "e4m3", "hybrid"])
@pytest.mark.parametrize("lens,n,k", [(None, 96, 160), ([33, 0, 130, 1, 92], 160, 96), ([300, 212], 384, 256)])
@pytest.mark.parametrize("kchunk", [True, False])
def test_operator_pattern_accumulates_into_main_grad(gpu, kind, lens, n, k, kchunk):
    import primus_amd.pytorch as turbo

    cfg = _cfg(kind)
    fp4 = kind == "mxfp4"
    rows = 200 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + n + k)
    x = torch.randn(rows, k, generator=g).bfloat16().to(gpu)
    w = (torch.randn(*((n, k) if lens is None else (len(lens), n, k)), generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(rows, n, generator=g).bfloat16().to(gpu)
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)

    def run(xx, ww, pattern):
        if lens is None:
            return (turbo.ops.gemm_fp4 if fp4 else turbo.ops.gemm_fp8)(xx, ww, config=cfg, fuse_bgrad_accum_pattern=pattern)
        return (turbo.ops.grouped_gemm_fp4 if fp4 else turbo.ops.grouped_gemm_fp8)(xx, ww, gl, config=cfg,
                                                                                   fuse_bgrad_accum_pattern=pattern)

    try:
        turbo.ops.set_kchunk_layout(kchunk)
        x0, w0 = x.clone().requires_grad_(), w.clone().requires_grad_()
        y0 = run(x0, w0, None)
        dx0, dw0 = torch.autograd.grad(y0, [x0, w0], dy)
        x1, w1 = x.clone().requires_grad_(), w.clone().requires_grad_()
        before = torch.randn(w.shape, generator=g).to(gpu)
        w1.main_grad = before.clone()
        w1.grad_added_to_main_grad = False
        y1 = run(x1, w1, "megatron")
        y1.backward(dy)
    finally:
        turbo.ops.set_kchunk_layout(True)
    assert torch.equal(y0, y1) and torch.equal(dx0, x1.grad)
    assert w1.grad_added_to_main_grad is True
    assert w1.grad is not None and w1.grad.shape == w.shape            # the placeholder reached the parameter
    delta = (w1.main_grad - before).double()
    ref = dw0.double()
    tol = ref.abs() * 2.0 ** -8 + ref.abs().max() * 1e-6 + before.abs().double() * 2.0 ** -22
    assert torch.all((delta - ref).abs() <= tol)


def test_pattern_argument_errors(gpu):
    import primus_amd.pytorch as turbo

    cfg = _cfg("mxfp8")
    x = torch.randn(64, 64, device=gpu).bfloat16().requires_grad_()
    w = torch.randn(32, 64, device=gpu).bfloat16().requires_grad_()
    with pytest.raises(ValueError):
        turbo.ops.gemm_fp8(x, w, config=cfg, fuse_bgrad_accum_pattern="megatron")     # no main_grad on the weight
    with pytest.raises(ValueError):
        turbo.ops.gemm_fp8(x, w, config=cfg, fuse_bgrad_accum_pattern="other")
    w.main_grad = torch.zeros(16, 64, device=gpu, dtype=torch.float32)
    w.grad_added_to_main_grad = False
    with pytest.raises(ValueError):
        turbo.ops.gemm_fp8(x, w, config=cfg, fuse_bgrad_accum_pattern="megatron")     # main_grad must have the weight's shape
