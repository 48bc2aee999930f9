"""The differentiable operators (ops.gemm_fp8 / gemm_fp4 / grouped_gemm_fp8 /
grouped_gemm_fp4) against the oracle's end-to-end linear: forward, dgrad,
wgrad; bf16 weights and cached QuantizedTensorPair weights."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _f(t):
    return o.bf16_bits_to_f32(t.detach().view(torch.int16).cpu().numpy().view(np.uint16))


def _close(got, want_bits, tol=TOL):
    want = o.bf16_bits_to_f32(want_bits)
    err = np.abs(_f(got) - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= tol, err


def _cfg8():
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    return Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0, block_size=32)


def test_gemm_fp8_fwd_bwd(gpu):
    import primus_amd.pytorch as pt

    g = torch.Generator().manual_seed(1)
    x = torch.randn(200, 256, generator=g).bfloat16()
    w = (torch.randn(160, 256, generator=g) * 0.05).bfloat16()
    dy = torch.randn(200, 160, generator=g).bfloat16()
    xd, wd = x.to(gpu).requires_grad_(), w.to(gpu).requires_grad_()
    y = pt.ops.gemm_fp8(xd, wd, trans_a=False, trans_b=True, out_dtype=None, config=_cfg8(), fuse_bgrad_accum_pattern=None)
    y.backward(dy.to(gpu))
    _close(y, o.linear_fwd_ref(x, w))
    dx, dw = o.linear_bwd_ref(x, w, dy)
    _close(xd.grad, dx)
    _close(wd.grad, dw)
    assert wd.grad.shape == wd.shape and xd.grad.shape == xd.shape and y.dtype == torch.bfloat16


@pytest.mark.parametrize("lens", [[33, 0, 130, 1, 136], [0, 0, 64], [256, 256, 256]])
def test_grouped_gemm_fp8_fwd_bwd(gpu, lens):
    import primus_amd.pytorch as pt

    m, k, n, G = sum(lens), 160, 96, len(lens)
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(G, n, k, generator=g) * 0.05).bfloat16()
    dy = torch.randn(m, n, generator=g).bfloat16()
    xd, wd = x.to(gpu).requires_grad_(), w.to(gpu).requires_grad_()
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = pt.ops.grouped_gemm_fp8(xd, wd, gl, trans_b=True, config=_cfg8())
    y.backward(dy.to(gpu))
    xq, xs = o.quantize_mx_rowwise(x)
    wq, ws, _, _ = o.quantize_mx_2d(w)
    _close(y, o.grouped_gemm_nt_ref(xq, xs, wq, ws, lens))
    dx, dw = o.linear_bwd_ref(x, w, dy, group_lens=lens)
    _close(xd.grad, dx)
    _close(wd.grad, dw)
    for e, ln in enumerate(lens):
        if ln == 0:
            assert not wd.grad[e].any()
    # keyword form used by the second backend (torchtitan/models/moe/moe.py:38-48)
    y2 = pt.ops.grouped_gemm_fp8(xd.detach(), wd.detach(), group_lens=gl, trans_b=True, config=_cfg8())
    assert torch.equal(y2, y.detach())


@pytest.mark.parametrize("fp4", [False, True])
def test_no_tokens_at_all(gpu, fp4):
    """A step in which no token reaches this rank's experts (and a dense linear on an empty batch):
    empty output, empty input gradient, all-zero weight gradient, no error."""
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import Float4QuantConfig

    cfg = Float4QuantConfig() if fp4 else _cfg8()
    grouped = pt.ops.grouped_gemm_fp4 if fp4 else pt.ops.grouped_gemm_fp8
    dense = pt.ops.gemm_fp4 if fp4 else pt.ops.gemm_fp8
    x = torch.empty(0, 160, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    w = (torch.randn(3, 96, 160, device=gpu) * 0.05).bfloat16().requires_grad_()
    gl = torch.zeros(3, dtype=torch.int64, device=gpu)
    y = grouped(x, w, gl, trans_b=True, config=cfg)
    assert y.shape == (0, 96)
    y.backward(torch.empty(0, 96, device=gpu, dtype=torch.bfloat16))
    assert x.grad.shape == (0, 160) and w.grad.shape == w.shape and not w.grad.any()
    w2 = w.detach()[0].clone().requires_grad_()
    x2 = torch.empty(0, 160, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y2 = dense(x2, w2, trans_a=False, trans_b=True, out_dtype=None, config=cfg)
    y2.backward(torch.empty(0, 96, device=gpu, dtype=torch.bfloat16))
    assert y2.shape == (0, 96) and not w2.grad.any()


def test_cached_weight_pair_matches_bf16_weight_path(gpu):
    """QuantizedTensorPair path (primus_turbo.py:1105-1134): same bytes as
    quantising inside the op, gradient flows to pair.data."""
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import QuantizedTensorPair, create_quantized_weight, float8_e4m3

    g = torch.Generator().manual_seed(2)
    x = torch.randn(96, 128, generator=g).bfloat16().to(gpu)
    w = (torch.randn(64, 128, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(96, 64, generator=g).bfloat16().to(gpu)
    cfg = _cfg8()
    x1, w1 = x.clone().requires_grad_(), w.clone().requires_grad_()
    y1 = pt.ops.gemm_fp8(x1, w1, trans_b=True, config=cfg)
    y1.backward(dy)
    row, col = create_quantized_weight(w, float8_e4m3, cfg, need_weight_transpose_cache=True)
    row.requires_grad_()
    x2 = x.clone().requires_grad_()
    y2 = pt.ops.gemm_fp8(x2, QuantizedTensorPair(data=row, data_t=col), trans_b=True, config=cfg)
    y2.backward(dy)
    assert torch.equal(y1, y2) and torch.equal(x1.grad, x2.grad)
    assert row.grad is not None and torch.equal(row.grad, w1.grad)
    # dequantize of the cached copies: row-wise in weight orientation, col-wise transposed
    wq, ws, wqt, wst = o.quantize_mx_2d(w.cpu())
    assert np.array_equal(_f(row.dequantize()), o.bf16_bits_to_f32(o.f32_to_bf16_bits(o.dequantize_mx(wq, ws))))
    assert np.array_equal(_f(col.dequantize()), o.bf16_bits_to_f32(o.f32_to_bf16_bits(o.dequantize_mx(wqt, wst))))


@pytest.mark.parametrize("act", ["fp4", "fp8"])
def test_grouped_gemm_fp4(gpu, act):
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import Float4QuantConfig, Format

    lens = [40, 0, 88, 128]
    m, k, n, G = sum(lens), 2880 if act == "fp8" else 256, 64, 4
    g = torch.Generator().manual_seed(5)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(G, n, k, generator=g) * 0.02).bfloat16()
    dy = torch.randn(m, n, generator=g).bfloat16()
    cfg = Float4QuantConfig(activation_format=Format.E4M3 if act == "fp8" else Format.E2M1_X2)
    afmt = o.FMT_E4M3 if act == "fp8" else o.FMT_E2M1
    xd, wd = x.to(gpu).requires_grad_(), w.to(gpu).requires_grad_()
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = pt.ops.grouped_gemm_fp4(xd, wd, gl, trans_b=True, config=cfg)
    y.backward(dy.to(gpu))
    xq, xs = o.quantize_mx_rowwise(x, afmt)
    wq, ws, wqt, wst = o.quantize_mx_2d(w, o.FMT_E2M1)
    _close(y, o.grouped_gemm_nt_ref(xq, xs, wq, ws, lens, afmt, o.FMT_E2M1))
    dq, ds = o.quantize_mx_rowwise(dy, afmt)
    _close(xd.grad, o.grouped_gemm_nt_ref(dq, ds, wqt, wst, lens, afmt, o.FMT_E2M1))
    dyT, dysT = o.quantize_mx_colwise_segmented(dy, lens, afmt)
    xT, xsT = o.quantize_mx_colwise_segmented(x, lens, afmt)
    _close(wd.grad, o.grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, lens, afmt, afmt))


def test_quantized_tensor_quantize_axes(gpu):
    from primus_amd.pytorch.core import MXScalingRecipe, QuantizedTensor, ScalingGranularity, float8_e4m3

    g = torch.Generator().manual_seed(3)
    w = (torch.randn(96, 160, generator=g) * 0.02).bfloat16()
    wd = w.to(gpu)
    kw = dict(dest_dtype=float8_e4m3, granularity=ScalingGranularity.MX_BLOCKWISE, block_size=32)
    r = QuantizedTensor.quantize(wd, scaling_recipe=MXScalingRecipe(), axis=-1, **kw)
    q, s = o.quantize_mx_rowwise(w)
    assert tuple(r.shape) == (96, 160) and np.array_equal(r.codes.view(torch.uint8).cpu().numpy(), q)
    c = QuantizedTensor.quantize(wd, scaling_recipe=MXScalingRecipe(), axis=-2, **kw)
    qc, sc = o.quantize_mx_colwise_segmented(w, [96])
    assert tuple(c.shape) == (160, 96) and np.array_equal(c.codes.view(torch.uint8).cpu().numpy(), qc)
    assert np.array_equal(c.scales.view(torch.uint8).cpu().numpy(), sc)
    assert tuple(c.dequantize().shape) == (160, 96)
    r2 = QuantizedTensor.quantize(wd, scaling_recipe=MXScalingRecipe(use_2d_block=True), axis=-1, **kw)
    c2 = QuantizedTensor.quantize(wd, scaling_recipe=MXScalingRecipe(use_2d_block=True), axis=-2, **kw)
    q2, s2, q2t, s2t = o.quantize_mx_2d(w)
    assert np.array_equal(r2.codes.view(torch.uint8).cpu().numpy(), q2) and np.array_equal(c2.codes.view(torch.uint8).cpu().numpy(), q2t)
    with pytest.raises(NotImplementedError):
        r.transpose(-2, -1)
    tw = QuantizedTensor.quantize(wd, dest_dtype=float8_e4m3, granularity=ScalingGranularity.TENSORWISE)
    want, want_si = o.quantize_tensorwise(w, o.FMT_E4M3)
    assert np.array_equal(tw.codes.view(torch.uint8).cpu().numpy(), want) and tw.tensor_scale_inv.item() == float(want_si)
    twt = QuantizedTensor.quantize(wd, dest_dtype=float8_e4m3, granularity=ScalingGranularity.TENSORWISE, axis=-2)
    assert tuple(twt.shape) == (160, 96) and np.array_equal(twt.codes.view(torch.uint8).cpu().numpy()[:, :96], want.T)
    deq = tw.dequantize().float().cpu().numpy()
    assert np.abs(deq - w.float().numpy()).max() <= 0.07 * np.abs(w.float().numpy()).max()   # E4M3: 2^-4 relative steps
    with pytest.raises(NotImplementedError):
        QuantizedTensor.quantize(wd, dest_dtype=float8_e4m3, granularity=ScalingGranularity.BLOCKWISE)
