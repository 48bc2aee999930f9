"""swiglu_with_probs / geglu_with_probs on the GPU against the oracle.

Tolerance: the kernel computes in fp32 and the oracle in float64, both round once to bf16, so a
result may differ by one bf16 ulp where the exact value lies next to a rounding boundary:
|got - want| <= 2^-7 * |want| (one ulp) + 1e-30; gradients likewise plus 1e-6 of the magnitude of the\nterms that cancel where the derivative of the gate activation passes through zero; dprobs (an fp32 row sum of
F products) within 1e-4 of the row's sum of magnitudes."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _f(t):
    return o.bf16_bits_to_f32(t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)


def _ulp_close(got, want_f64, ulps=1.0, floor=0.0):
    want = o.bf16_bits_to_f32(o.f32_to_bf16_bits(want_f64.astype(np.float32))).astype(np.float64)
    tol = ulps * np.abs(want) * 2.0 ** -7 + 1e-30 + floor
    bad = np.abs(got - want) > tol
    assert not bad.any(), (int(bad.sum()), float(np.abs(got - want).max()))


@pytest.mark.parametrize("activation", ["silu", "gelu"])
@pytest.mark.parametrize("rows,f,pdtype", [(37, 64, torch.float32), (300, 2048, torch.float32), (64, 14336, torch.bfloat16),
                                           (5, 8, torch.float32)])
def test_forward_backward_vs_oracle(gpu, activation, rows, f, pdtype):
    import primus_amd.pytorch as pt

    g = torch.Generator().manual_seed(rows + f)
    x = (torch.randn(rows, 2 * f, generator=g) * 2).bfloat16()
    x[0, :4] = torch.tensor([0.0, -0.0, 30.0, -30.0]).bfloat16()          # exact zero, saturated gate both ways
    p = torch.rand(rows, generator=g).to(pdtype)
    mask = torch.rand(rows, generator=g) > 0.2
    mask[0] = True
    dy = torch.randn(rows, f, generator=g).bfloat16()
    op = pt.ops.swiglu_with_probs if activation == "silu" else pt.ops.geglu_with_probs
    xd, pd = x.to(gpu).requires_grad_(), p.to(gpu).requires_grad_()
    y = op(xd, pd, mask.to(gpu))
    y.backward(dy.to(gpu))
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (rows, f)
    pn = p.float().numpy()
    _ulp_close(_f(y), o.glu_with_probs_ref(x, pn, mask.numpy(), activation, out_bf16=False))
    assert not y[~mask.to(gpu)].any() and not xd.grad[~mask.to(gpu)].any() and not pd.grad[~mask.to(gpu)].any()
    dx, dp = o.glu_with_probs_bwd_ref(dy, x, pn, mask.numpy(), activation)
    # the derivative of the gate activation passes through zero (GELU near g = -0.75, SiLU near -1.28): next
    # to that zero fp32 cancellation leaves an absolute error of a few fp32 ulps of the O(1) terms
    xf0 = x.double().numpy()
    scale = np.abs(dy.double().numpy()) * np.abs(pn)[:, None].astype(np.float64) * (1.0 + np.abs(xf0[:, :f]) + np.abs(xf0[:, f:]))
    _ulp_close(_f(xd.grad), dx, floor=np.concatenate([scale, scale], axis=1) * 1e-6)
    assert pd.grad.dtype == pdtype
    xf = x.double().numpy()
    a, _ = o._act64(xf[:, :f], activation)
    mag = (np.abs(dy.double().numpy() * a * xf[:, f:])).sum(axis=1) + 1e-30
    dp_tol = (1e-4 if pdtype == torch.float32 else 2.0 ** -7) * mag + (0 if pdtype == torch.float32 else 2.0 ** -7 * np.abs(dp))
    assert (np.abs(pd.grad.double().cpu().numpy() - dp) <= dp_tol).all()


def test_no_mask_and_mask_helper(gpu):
    import primus_amd.pytorch as pt

    x = torch.randn(16, 64).bfloat16().to(gpu)
    p = torch.ones(16, device=gpu)
    full = pt.ops.swiglu_with_probs(x, p)
    assert torch.equal(full, pt.ops.swiglu_with_probs(x, p, torch.ones(16, dtype=torch.bool, device=gpu)))
    want = (torch.nn.functional.silu(x[:, :32].float()) * x[:, 32:].float()).bfloat16()
    assert torch.equal(full, want)   # p = 1: one rounding of the fp32 product, same as torch's fp32 path
    tpe = torch.tensor([3, 0, 6, 1], device=gpu)
    mask = pt.ops.tokens_per_expert_to_mask(tpe, 16)
    assert mask.tolist() == [True] * 10 + [False] * 6
    masked = pt.ops.swiglu_with_probs(x, p, mask)
    assert torch.equal(masked[:10], full[:10]) and not masked[10:].any()


def test_bad_arguments(gpu):
    import primus_amd.pytorch as pt
    from primus_amd import _lib

    x = torch.randn(4, 64).bfloat16().to(gpu)
    with pytest.raises(ValueError):
        pt.ops.swiglu_with_probs(x.float(), torch.ones(4, device=gpu))
    with pytest.raises(ValueError):
        pt.ops.swiglu_with_probs(x, torch.ones(5, device=gpu))
    with pytest.raises(ValueError):
        pt.ops.swiglu_with_probs(x[:, :24].contiguous(), torch.ones(4, device=gpu))   # F = 12 is not a multiple of 8
    lib = _lib.load()
    assert lib.mxl_glu_probs_fwd(x.data_ptr(), x.data_ptr(), 0, None, 4, 32, 7, x.data_ptr(), None) == -1  # bad activation
    assert lib.mxl_glu_probs_fwd(None, None, 0, None, 0, 32, 0, None, None) == 0                            # no rows: nothing to do


def test_grouped_mlp_with_fused_activation(gpu):
    """PrimusGroupedMLP with use_turbo_fused_act_with_probs against the unfused arithmetic (bf16 GEMMs)."""
    from types import SimpleNamespace

    from primus_amd.megatron import runtime
    from primus_amd.megatron.transformer.experts import PrimusGroupedMLP

    def cfg():
        return SimpleNamespace(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                               tensor_model_parallel_size=1, gradient_accumulation_fusion=False, hidden_size=128,
                               ffn_hidden_size=256, moe_ffn_hidden_size=256, gated_linear_unit=True, fp8=None, fp4=None,
                               add_bias_linear=False, activation_func=torch.nn.functional.silu)

    try:
        runtime.set_args(use_turbo_grouped_gemm=True, use_turbo_fused_act_with_probs=True)
        torch.manual_seed(11)
        fused = PrimusGroupedMLP(3, cfg())
        runtime.set_args(use_turbo_grouped_gemm=True, use_turbo_fused_act_with_probs=False)
        plain = PrimusGroupedMLP(3, cfg())
        plain.load_state_dict(fused.state_dict())
        assert fused.use_turbo_fused_act_with_probs and not plain.use_turbo_fused_act_with_probs
        lens = torch.tensor([40, 0, 24], device=gpu)
        x = torch.randn(64, 128, device=gpu).bfloat16()
        probs = torch.rand(64, device=gpu)
        a, _ = fused(x, lens, probs)
        b, _ = plain(x, lens, probs)
        assert torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0) > 0.9999
    finally:
        runtime.set_args()


@pytest.mark.parametrize("activation", ["silu", "gelu"])
@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("lens,f", [([33, 0, 130, 1, 92], 160), ([300], 2048), ([0, 0], 64)])
def test_fused_activation_quantize_equals_two_kernels(gpu, activation, fmt, lens, f):
    """mxl_glu_probs_quantize writes exactly the bytes of activation followed by quantisation
    (row-wise, padded to the GEMM's K granularity, and transposed per expert)."""
    from primus_amd.pytorch import kernels as K

    rows = sum(lens)
    g = torch.Generator().manual_seed(rows + f + fmt)
    x = (torch.randn(rows, 2 * f, generator=g) * 2).bfloat16().to(gpu)
    p = torch.rand(rows, generator=g).to(gpu)
    mask = (torch.rand(rows, generator=g) > 0.1).to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    y = K.glu_with_probs_fwd_impl(x, p, mask, activation)
    want = K.quantize_mx_impl(y, fmt, rowwise=True, colwise=True, group_lens=gl, pad_to=128)
    got = K.glu_with_probs_quantize_impl(x, p, mask, activation, fmt, colwise=True, group_lens=gl, pad_to=128)
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    row_only = K.glu_with_probs_quantize_impl(x, p, mask, activation, fmt)
    assert row_only[2] is None and row_only[3] is None
    per = 2 if fmt == 1 else 1
    assert torch.equal(row_only[0].view(torch.uint8), want[0].view(torch.uint8)[:, : f // per])
    # and the activation itself is checked against the oracle above, so the fused bytes are the oracle's
    # quantisation of the oracle's activation wherever the fp32 and float64 roundings agree
    if rows:
        yq, ys = o.quantize_mx_rowwise(y.cpu(), fmt)
        assert np.array_equal(got[0].view(torch.uint8).cpu().numpy()[:, : f // per], yq)
        assert np.array_equal(got[1].view(torch.uint8).cpu().numpy()[:, : f // 32], ys)


@pytest.mark.parametrize("activation", ["silu", "gelu"])
@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("lens,f,n", [([33, 0, 130, 1, 92], 160, 96), ([300, 212], 512, 256), ([0, 0], 64, 32)])
def test_glu_grouped_gemm_equals_activation_then_grouped_gemm(gpu, activation, fp4, lens, f, n):
    """ops.glu_grouped_gemm_fp8 / _fp4 give exactly what the activation operator followed by the
    grouped GEMM operator gives -- output, and the gradients of fc1's output, the probabilities and
    the weight -- since the fused quantiser writes the same bytes and the backward runs the same kernels."""
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    if fp4:
        cfg = Float4QuantConfig(activation_format=Format.E4M3)
        fused_op, plain_op = pt.ops.glu_grouped_gemm_fp4, pt.ops.grouped_gemm_fp4
    else:
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
        fused_op, plain_op = pt.ops.glu_grouped_gemm_fp8, pt.ops.grouped_gemm_fp8
    act_op = pt.ops.swiglu_with_probs if activation == "silu" else pt.ops.geglu_with_probs
    rows, G = sum(lens), len(lens)
    g = torch.Generator().manual_seed(rows + f + n)
    h = (torch.randn(rows, 2 * f, generator=g) * 1.5).bfloat16().to(gpu)
    p = torch.rand(rows, generator=g).to(gpu)
    w = (torch.randn(G, n, f, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(rows, n, generator=g).bfloat16().to(gpu)
    mask = (torch.rand(rows, generator=g) > 0.1).to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)

    outs = []
    for fused in (True, False):
        hh, pp, ww = h.clone().requires_grad_(), p.clone().requires_grad_(), w.clone().requires_grad_()
        if fused:
            y = fused_op(hh, pp, ww, gl, activation=activation, row_mask=mask, config=cfg)
        else:
            y = plain_op(act_op(hh, pp, mask), ww, gl, trans_b=True, config=cfg)
        y.backward(dy)
        outs.append((y.detach(), hh.grad, pp.grad, ww.grad))
    for a, b in zip(*outs):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a, b)
    # only the probabilities need a gradient: dgrad still runs, fc1's output gets none
    hh, pp = h.clone(), p.clone().requires_grad_()
    fused_op(hh, pp, w, gl, activation=activation, row_mask=mask, config=cfg).backward(dy)
    assert torch.equal(pp.grad, outs[0][2])
    with pytest.raises(ValueError):
        fused_op(h, p, w[:, :, : f // 2].contiguous(), gl, activation=activation, config=cfg)   # K mismatch
    with pytest.raises(ValueError):
        fused_op(h, p, w, gl, activation="relu", config=cfg)
