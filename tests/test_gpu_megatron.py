"""The Megatron-side modules on the real kernels: linear / grouped linear /
expert MLP under the MXFP8 and MXFP4 autocasts, cached quantised weights with
``main_grad`` accumulation, the MXFP4 local function and the optimizer's
quantisation grid -- against the oracle where it restates the arithmetic, and
against the reference's own acceptance bars where it states them (MXFP8 MoE
cosine >= 0.90 vs bf16: tests/unit_tests/megatron/moe/test_mega_moe.py:243-280;
MXFP4 gradient SNR > 10 dB vs bf16: test_primus_turbo_mxfp4_local.py:182-189)."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
TOL = 1e-2  # max abs error / max abs value of the oracle's result


def _f(t):
    return o.bf16_bits_to_f32(t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16))


def _close(got, want_bits, tol=TOL):
    want = o.bf16_bits_to_f32(want_bits)
    err = np.abs(_f(got).reshape(want.shape) - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= tol, err


def _snr_db(got, truth):
    got, truth = got.float(), truth.float()
    return (10 * torch.log10(truth.pow(2).sum() / (got - truth).pow(2).sum())).item()


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()


@pytest.fixture
def mg(gpu):
    from primus_amd.megatron import runtime
    from primus_amd.megatron.extensions import primus_turbo as pt

    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.bind()
    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=True)
    runtime.set_num_microbatches(1)
    yield pt
    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.set_args()
    runtime.set_num_microbatches(1)


def _cfg(**kw):
    values = dict(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                  tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                  layernorm_epsilon=1e-5)
    values.update(kw)
    return SimpleNamespace(**values)


def _mxfp8(pt):
    from primus_amd.pytorch.core import Format, ScaleDtype, ScalingGranularity

    return pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E4M3, block_size=32,
                                     scale_dtype=ScaleDtype.E8M0)


def _mxfp4(pt, **kw):
    from primus_amd.pytorch.core import Format, ScaleDtype, ScalingGranularity

    return pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E2M1_X2, block_size=32,
                                     scale_dtype=ScaleDtype.E8M0, use_gradient_sr=False, **kw)


def test_linear_mxfp8_forward_backward_matches_oracle(mg, gpu):
    pt = mg
    torch.manual_seed(3)
    lin = pt.PrimusTurboLinear(256, 160, parallel_mode=None, config=_cfg(), bias=True, skip_bias_add=False)
    with torch.no_grad():
        lin.bias.copy_(torch.linspace(-1, 1, 160))
    x = torch.randn(25, 8, 256, device=gpu).bfloat16().requires_grad_()
    dy = torch.randn(25, 8, 160, device=gpu).bfloat16()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt)):
        y, bias = lin(x)
    assert bias is None and y.shape == (25, 8, 160) and y.dtype == torch.bfloat16
    y.backward(dy)
    x2, w = x.detach().cpu().view(-1, 256), lin.weight.detach().cpu()
    y_ref = o.bf16_bits_to_f32(o.linear_fwd_ref(x2, w)) + lin.bias.detach().float().cpu().numpy()
    err = np.abs(_f(y).reshape(y_ref.shape) - y_ref).max() / np.abs(y_ref).max()
    assert err <= TOL, err
    dx, dw = o.linear_bwd_ref(x2, w, dy.cpu().view(-1, 160))
    _close(x.grad, dx)
    _close(lin.weight.grad, dw)
    torch.testing.assert_close(lin.bias.grad.float(), dy.float().sum((0, 1)), rtol=2e-2, atol=2e-1)
    # outside the autocast the same module is a plain bf16 linear
    y_bf16, _ = lin(x.detach())
    want = torch.nn.functional.linear(x.detach(), lin.weight, lin.bias)
    torch.testing.assert_close(y_bf16.float(), want.float(), rtol=2e-2, atol=2e-2)


def test_cached_weights_accumulate_into_main_grad_over_microbatches(mg, gpu):
    pt = mg
    from primus_amd.megatron import runtime

    runtime.set_num_microbatches(3)
    torch.manual_seed(4)
    lin = pt.PrimusTurboColumnParallelLinear(128, 96, config=_cfg(), bias=False)
    lin.weight.main_grad = torch.zeros(96, 128, dtype=torch.float32, device=gpu)
    lin.weight.grad_added_to_main_grad = False
    xs = [torch.randn(40, 1, 128, device=gpu).bfloat16().requires_grad_() for _ in range(3)]
    dys = [torch.randn(40, 1, 96, device=gpu).bfloat16() for _ in range(3)]
    want = np.zeros((96, 128), dtype=np.float32)
    w_cpu = lin.weight.detach().cpu()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt)):
        for i, (x, dy) in enumerate(zip(xs, dys)):
            y, _ = lin(x)
            if i == 0:
                first_codes = lin.quantized_weight_buffer.codes
            assert lin.quantized_weight_buffer.codes.data_ptr() == first_codes.data_ptr()  # quantised once
            lin.weight.grad_added_to_main_grad = False  # what the DDP wrapper does per microbatch
            y.backward(dy)
            _close(y, o.linear_fwd_ref(x.detach().cpu().view(-1, 128), w_cpu))
            dx, dw = o.linear_bwd_ref(x.detach().cpu().view(-1, 128), w_cpu, dy.cpu().view(-1, 96))
            _close(x.grad, dx)
            want += o.bf16_bits_to_f32(dw)
    got = lin.weight.main_grad.cpu().numpy()
    assert np.abs(got - want).max() / np.abs(want).max() <= TOL
    assert lin.weight.grad_added_to_main_grad is True
    assert lin.weight.grad is not None and lin.weight.grad.shape == lin.weight.shape  # placeholder fired the hooks
    assert lin.quantized_weight_t_buffer.axis == -2 and tuple(lin.quantized_weight_t_buffer.shape) == (128, 96)


@pytest.mark.parametrize("fp4", [False, True])
def test_grouped_linear_ragged_groups(mg, gpu, fp4):
    pt = mg
    torch.manual_seed(5)
    lens = [33, 0, 130, 1, 92]
    gl = pt.PrimusTurboColumnParallelGroupedLinear(5, 128, 96, config=_cfg())
    x = torch.randn(sum(lens), 128, device=gpu).bfloat16().requires_grad_()
    dy = torch.randn(sum(lens), 96, device=gpu).bfloat16()
    splits = torch.tensor(lens)  # on the host on purpose: the module moves it to the device
    if fp4:
        ctx = pt.primus_turbo_fp4_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp4(pt))
        fmt = o.FMT_E2M1
    else:
        ctx = pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt))
        fmt = o.FMT_E4M3
    with ctx:
        y, _ = gl(x, splits)
    y.backward(dy)
    xc, wc = x.detach().cpu(), gl.weights.detach().cpu()
    xq, xs = o.quantize_mx_rowwise(xc, fmt)
    wq, ws, _, _ = o.quantize_mx_2d(wc, fmt)
    tol = 3e-2 if fp4 else TOL  # FP4 sums carry larger bf16 rounding of larger partials; still the reference's 3e-2 bar
    _close(y, o.grouped_gemm_nt_ref(xq, xs, wq, ws, lens, fmt, fmt), tol)
    dx, dw = o.linear_bwd_ref(xc, wc, dy.cpu(), fmt=fmt, group_lens=lens)
    _close(x.grad, dx, tol)
    _close(gl.weights.grad, dw, tol)
    assert not gl.weights.grad[1].any()  # expert without tokens


def _mlp(pt, gpu, experts, hidden, ffn, **cfg):
    from primus_amd.megatron.transformer.experts import PrimusGroupedMLP

    return PrimusGroupedMLP(experts, _cfg(hidden_size=hidden, ffn_hidden_size=ffn, moe_ffn_hidden_size=ffn,
                                          gated_linear_unit=True, fp8="e4m3", fp8_recipe="mxfp8", fp4=None,
                                          add_bias_linear=False, **cfg))


def test_grouped_mlp_mxfp8_close_to_bf16(mg, gpu):
    """Forward, dX and dW of the expert MLP in MXFP8 against the same module in bf16."""
    pt = mg
    torch.manual_seed(6)
    mlp = _mlp(pt, gpu, 4, 256, 512)
    lens = [100, 0, 257, 27]
    x = torch.randn(sum(lens), 256, device=gpu).bfloat16()
    probs = torch.rand(sum(lens), device=gpu).bfloat16()
    tpe = torch.tensor(lens, device=gpu)
    dy = torch.randn(sum(lens), 256, device=gpu).bfloat16()

    def run(ctx):
        mlp.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_()
        with ctx:
            out, _ = mlp(xi, tpe, probs)
        out.backward(dy)
        return out.detach(), xi.grad, mlp.linear_fc1.weights.grad.clone(), mlp.linear_fc2.weights.grad.clone()

    import contextlib

    ref = run(contextlib.nullcontext())
    got = run(pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt)))
    for name, a, b in zip(("y", "dx", "dw1", "dw2"), got, ref):
        assert torch.isfinite(a.float()).all(), name
        assert _cos(a, b) >= 0.99, (name, _cos(a, b))  # the reference's bar is 0.90


@pytest.mark.parametrize("fp4", [False, True])
def test_grouped_mlp_fc2_takes_the_activation(mg, gpu, fp4):
    """With the fused activation, fc2 consumes fc1's output directly (activation inside its
    quantiser): forward and every gradient equal those of the separate activation kernel bit for
    bit, and no activation launch is left in the forward."""
    from contextlib import contextmanager

    from primus_amd.megatron import runtime
    from primus_amd.pytorch import kernels as K

    pt = mg
    common = dict(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                  turbo_grouped_gemm_without_padding=True, use_turbo_fused_act_with_probs=True)
    torch.manual_seed(5)
    runtime.set_args(**common)
    a = _mlp(pt, gpu, 4, 256, 384)
    runtime.set_args(turbo_fuse_act_into_fc2_quantize=False, **common)
    b = _mlp(pt, gpu, 4, 256, 384)
    b.load_state_dict(a.state_dict())
    assert a.fuse_act_into_fc2 and not b.fuse_act_into_fc2
    lens = torch.tensor([100, 0, 37, 55], device=gpu)
    x = torch.randn(192, 256, device=gpu).bfloat16()
    probs = torch.rand(192, device=gpu)
    dy = torch.randn(192, 256, device=gpu).bfloat16()
    launches = []

    @contextmanager
    def hook(name, info):
        launches.append(name)
        yield

    res = []
    for mod in (a, b):
        del launches[:]
        xx, pp = x.clone().requires_grad_(), probs.clone().requires_grad_()
        K.set_launch_hook(hook)
        try:
            if fp4:
                ctx = pt.primus_turbo_fp4_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp4(pt))
            else:
                ctx = pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt))
            with ctx:
                y, _ = mod(xx, lens, pp)
            y.backward(dy)
        finally:
            K.set_launch_hook(None)
        res.append((y.detach(), xx.grad, pp.grad, mod.linear_fc1.weights.grad, mod.linear_fc2.weights.grad,
                    list(launches)))
    for u, v in zip(res[0][:5], res[1][:5]):
        assert u is not None and torch.equal(u, v)
    assert "glu_probs_quantize" in res[0][5] and "glu_probs_fwd" not in res[0][5]
    assert "glu_probs_fwd" in res[1][5] and "glu_probs_quantize" not in res[1][5]
    assert len(res[0][5]) == len(res[1][5]) - 1          # one launch fewer per step


def test_grouped_mlp_explicit_padding_gives_the_same_forward(mg, gpu):
    """Padding rows are zeros and row-wise blocks never mix rows, so the padded
    and the ragged path quantise every real row identically."""
    pt = mg
    from primus_amd.megatron import runtime

    torch.manual_seed(7)
    lens = [5, 0, 33, 64]
    x = torch.randn(sum(lens), 128, device=gpu).bfloat16()
    probs = torch.rand(sum(lens), device=gpu).bfloat16()
    tpe = torch.tensor(lens, device=gpu)
    ragged = _mlp(pt, gpu, 4, 128, 256)
    runtime.set_args(enable_primus_turbo=True, use_turbo_grouped_gemm=True, turbo_grouped_gemm_without_padding=False)
    padded = _mlp(pt, gpu, 4, 128, 256)
    padded.load_state_dict(ragged.state_dict())
    assert padded._use_explicit_quantization_padding() and not ragged._use_explicit_quantization_padding()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt)):
        a, _ = ragged(x, tpe, probs)
        b, _ = padded(x, tpe, probs)
    assert a.shape == b.shape == (sum(lens), 128)
    assert torch.equal(a, b)


def test_mxfp4_dual_quantize_op_matches_oracle_bytes(mg, gpu):
    from primus_amd.megatron.extensions import primus_turbo_mxfp4_local as m4

    torch.manual_seed(8)
    x = torch.randn(100, 96, device=gpu).bfloat16()        # activation recipe: 1-D blocks
    row, row_s, col, col_s = m4._quantize_input_dual(x)
    assert tuple(row.shape) == (100, 64) and tuple(row_s.shape) == (100, 4)
    assert tuple(col.shape) == (96, 64) and tuple(col_s.shape) == (96, 4)
    q, s = o.quantize_mx_rowwise(x.cpu(), o.FMT_E2M1)
    assert np.array_equal(row.view(torch.uint8).cpu().numpy()[:, :48], q)
    assert np.array_equal(row_s.view(torch.uint8).cpu().numpy()[:, :3], s)
    assert not row.view(torch.uint8)[:, 48:].any() and not row_s.view(torch.uint8)[:, 3:].any()
    # the col-wise copy of an activation goes through the Hadamard transform, like the reference's
    qT, sT = o.quantize_mx_colwise_segmented_fp4(x.cpu(), [100], rht_signs=m4.RHT_SIGNS)
    assert np.array_equal(col.view(torch.uint8).cpu().numpy(), qT)
    assert np.array_equal(col_s.view(torch.uint8).cpu().numpy(), sT)
    _, _, col0, col0_s = m4._quantize_input_dual(x, use_rht=False)
    qT, sT = o.quantize_mx_colwise_segmented(x.cpu(), [100], o.FMT_E2M1)
    assert np.array_equal(col0.view(torch.uint8).cpu().numpy(), qT)
    assert np.array_equal(col0_s.view(torch.uint8).cpu().numpy(), sT)

    w = (torch.randn(64, 96, device=gpu) * 0.05).bfloat16()  # weight recipe: 2-D blocks
    wr, wrs, wc, wcs = m4._quantize_weight_dual(w)
    q, s, qt, st = o.quantize_mx_2d(w.cpu(), o.FMT_E2M1)
    assert np.array_equal(wr.view(torch.uint8).cpu().numpy()[:, :48], q)
    assert np.array_equal(wrs.view(torch.uint8).cpu().numpy()[:, :3], s)
    assert np.array_equal(wc.view(torch.uint8).cpu().numpy()[:, :32], qt)
    assert np.array_equal(wcs.view(torch.uint8).cpu().numpy()[:, :2], st)
    with pytest.raises(NotImplementedError, match="rowwise_use_rht"):
        m4._quantize_mxfp4_dual_op(x, m4._FP4_DTYPE, 128, False, False, True, False, False, True, False, False, False, False)
    # the pre-shuffled copies are byte permutations of the plain ones, in the shapes the reference's shape function states
    g_plain = m4._quantize_grad_dual(x, use_rht=False)
    g_pre = m4._quantize_grad_dual(x, preshuffle=True, use_rht=False)       # gradients: scales shuffled, codes not
    assert torch.equal(g_pre[0].view(torch.uint8), g_plain[0].view(torch.uint8))
    assert torch.equal(g_pre[2].view(torch.uint8), g_plain[2].view(torch.uint8))
    assert tuple(g_pre[1].shape) == (256, 8) and tuple(g_pre[3].shape) == (256, 8)
    assert np.array_equal(g_pre[1].view(torch.uint8).cpu().numpy(), o.shuffle_e8m0(g_plain[1].view(torch.uint8).cpu().numpy()))
    assert np.array_equal(g_pre[3].view(torch.uint8).cpu().numpy(), o.shuffle_e8m0(g_plain[3].view(torch.uint8).cpu().numpy()))
    w_pre = m4._quantize_weight_dual(w, preshuffle=True)                    # weights: everything shuffled
    for got, plain in ((w_pre[0], wr), (w_pre[2], wc)):
        assert np.array_equal(got.view(torch.uint8).cpu().numpy(), o.shuffle_codes_16x16(plain.view(torch.uint8).cpu().numpy()))
    for got, plain in ((w_pre[1], wrs), (w_pre[3], wcs)):
        assert np.array_equal(got.view(torch.uint8).cpu().numpy(), o.shuffle_e8m0(plain.view(torch.uint8).cpu().numpy()))
    # stochastic rounding keeps shapes and scales (the codes are checked in test_gpu_fp4_options.py)
    sr = m4._quantize_grad_dual(x, use_sr=True)
    assert torch.equal(sr[1].view(torch.uint8), row_s.view(torch.uint8)) and sr[0].shape == row.shape


def test_mxfp4_linear_function_snr_against_bf16(mg, gpu):
    """Shapes of the reference's test (x[128, 256], w[512, 256]); its bar is SNR > 10 dB."""
    from primus_amd.megatron.extensions.primus_turbo_mxfp4_local import MXFP4LinearFunction

    torch.manual_seed(9)
    x = torch.randn(128, 256, device=gpu).bfloat16().requires_grad_()
    w = (torch.randn(512, 256, device=gpu) * 0.05).bfloat16().requires_grad_()
    dy = torch.randn(128, 512, device=gpu).bfloat16()
    y = MXFP4LinearFunction.apply(x, w, False, False, None, 0, 0, False)[0]
    y.backward(dy)
    xr, wr = x.detach().float().requires_grad_(), w.detach().float().requires_grad_()
    yr = xr @ wr.T
    yr.backward(dy.float())
    assert y.shape == (128, 512) and x.grad.shape == x.shape and w.grad.shape == w.shape
    for name, a, b in (("y", y, yr), ("dx", x.grad, xr.grad), ("dw", w.grad, wr.grad)):
        assert _snr_db(a.detach(), b.detach()) > 10.0, (name, _snr_db(a.detach(), b.detach()))
    # and the forward equals the oracle's MXFP4 linear
    _close(y, o.linear_fwd_ref(x.detach().cpu(), w.detach().cpu(), o.FMT_E2M1, o.FMT_E2M1), 3e-2)


def test_mxfp4_linear_function_preshuffled_is_bit_identical(mg, gpu):
    """With the pre-shuffle switch on, the bytes between the quantiser and the GEMM travel in the shuffled order and
    every result is the same bit for bit."""
    from primus_amd.megatron.extensions.primus_turbo_mxfp4_local import MXFP4LinearFunction, mxfp4_linear

    torch.manual_seed(11)
    res = []
    for pre in (False, True):
        x = torch.randn(3, 100, 256, device=gpu).bfloat16().requires_grad_()
        w = (torch.randn(192, 256, device=gpu) * 0.05).bfloat16().requires_grad_()
        if res:
            x.data.copy_(res[0][3]), w.data.copy_(res[0][4])
        out = MXFP4LinearFunction.apply(x, w, pre, False, None, 0, 0, False)
        assert len(out) == 5 and all(t.dtype == torch.uint8 for t in out[1:])
        assert tuple(out[2].shape) == ((256, 16) if pre else (256, 12))          # X^T scales: 256 features x 384/32 blocks
        dy = torch.ones_like(out[0]) * 0.5 + out[0].detach() * 0.01
        out[0].backward(dy)
        res.append((out[0].detach(), x.grad, w.grad, x.detach().clone(), w.detach().clone()))
    for a, b in zip(res[0][:3], res[1][:3]):
        assert torch.equal(a, b)
    assert torch.equal(mxfp4_linear(res[0][3], res[0][4], preshuffle=True), res[0][0])


def test_mxfp4_linear_function_fp8_backward(mg, gpu):
    """The hybrid mode: MXFP4 forward, backward on the saved bf16 tensors re-quantised to E5M2 with one scale per
    tensor; checked against the oracle's tensor-wise quantiser and GEMM."""
    from primus_amd.megatron.extensions.primus_turbo_mxfp4_local import MXFP4LinearFunction
    from primus_amd.pytorch.core.low_precision import ScalingGranularity, float8_e5m2

    torch.manual_seed(12)
    x = torch.randn(128, 256, device=gpu).bfloat16().requires_grad_()
    w = (torch.randn(192, 256, device=gpu) * 0.05).bfloat16().requires_grad_()
    dy = torch.randn(128, 192, device=gpu).bfloat16()
    out = MXFP4LinearFunction.apply(x, w, False, True, float8_e5m2, ScalingGranularity.TENSORWISE.value, 0, False)
    assert len(out) == 3
    y = out[0]
    y.backward(dy)
    plain = MXFP4LinearFunction.apply(x.detach(), w.detach(), False, False, None, 0, 0, False)[0]
    assert torch.equal(y.detach(), plain)                                           # the forward is the same
    qd, sd = o.quantize_tensorwise(dy.cpu(), o.FMT_E5M2)
    qx, sx = o.quantize_tensorwise(x.detach().cpu(), o.FMT_E5M2)
    qw, sw = o.quantize_tensorwise(w.detach().cpu(), o.FMT_E5M2)
    want_dx = o.tensorwise_gemm_nt_ref(qd, sd, np.ascontiguousarray(qw.T), sw, o.FMT_E5M2, o.FMT_E5M2)
    want_dw = o.tensorwise_gemm_nt_ref(np.ascontiguousarray(qd.T), sd, np.ascontiguousarray(qx.T), sx, o.FMT_E5M2, o.FMT_E5M2)
    _close(x.grad, want_dx, 1e-2)
    _close(w.grad, want_dw, 1e-2)
    with pytest.raises(ValueError, match="tensor-wise"):
        MXFP4LinearFunction.apply(x, w, False, True, float8_e5m2, ScalingGranularity.MX_BLOCKWISE.value, 0, False)


def test_mxfp4_linear_function_traces_without_graph_breaks(mg, gpu):
    """What the reference's own tests ask of the function (test_primus_turbo_mxfp4_local.py:202-287): torch.compile
    traces it without a graph break in both modes, and the traced forward and backward equal the eager ones."""
    from primus_amd.megatron.extensions.primus_turbo_mxfp4_local import MXFP4LinearFunction
    from primus_amd.pytorch.core.low_precision import ScalingGranularity, float8_e5m2

    torch.manual_seed(42)
    x = torch.randn(128, 256, dtype=torch.bfloat16, device=gpu)
    w = torch.randn(512, 256, dtype=torch.bfloat16, device=gpu)
    modes = ((False, False, None, 0, 0, False), (True, False, None, 0, 0, False),
             (False, True, float8_e5m2, ScalingGranularity.TENSORWISE.value, 0, False))
    for args in modes:
        torch._dynamo.reset()
        explanation = torch._dynamo.explain(MXFP4LinearFunction.apply)(x, w, *args)
        assert explanation.graph_break_count == 0, explanation.break_reasons
    torch._dynamo.reset()
    for args in modes:
        xe, we = x.clone().requires_grad_(), w.clone().requires_grad_()
        xc, wc = x.clone().requires_grad_(), w.clone().requires_grad_()
        eager = MXFP4LinearFunction.apply(xe, we, *args)[0]
        compiled = torch.compile(MXFP4LinearFunction.apply, backend="aot_eager")(xc, wc, *args)[0]
        assert torch.equal(eager, compiled)
        dy = torch.randn_like(eager)
        eager.backward(dy)
        compiled.backward(dy)
        assert torch.equal(xe.grad, xc.grad) and torch.equal(we.grad, wc.grad)
    torch._dynamo.reset()


def test_qdq_mxfp4_is_the_forward_weight_grid(mg, gpu):
    from primus_amd.megatron.optimizer.weight_deosc import qdq_mxfp4, qdq_mxfp4_local_shard

    torch.manual_seed(10)
    w = (torch.randn(3, 64, 96, device=gpu) * 0.05).bfloat16()
    got = qdq_mxfp4(w)
    q, s, _, _ = o.quantize_mx_2d(w.cpu(), o.FMT_E2M1)
    want = o.dequantize_mx(q, s, o.FMT_E2M1)
    assert got.shape == w.shape and got.dtype == w.dtype
    assert np.array_equal(_f(got), want.astype(np.float32).reshape(_f(got).shape))
    assert torch.equal(qdq_mxfp4(w[1]), got[1])             # experts are independent 2-D matrices
    assert torch.equal(qdq_mxfp4(got), got)                 # idempotent: grid points stay put
    # a shard that covers whole tile rows of expert 1 reproduces the full result there
    per = 64 * 96
    start, end = per + 32 * 96, per + 64 * 96
    shard = w.reshape(-1)[start:end].float()
    local = qdq_mxfp4_local_shard(shard, tuple(w.shape), start, end, torch.bfloat16)
    assert torch.equal(local, got.reshape(-1)[start:end])


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("microbatches", [1, 2])
def test_layernorm_linear_folds_the_rmsnorm_into_the_quantiser(mg, gpu, fp4, microbatches):
    """RMSNorm + column-parallel linear: with the normalisation folded into the GEMM's quantiser the module
    returns the same output and gradients, bit for bit, as with the two operators run one after the other
    (the reference's sequence, primus_turbo.py:1689-1741), and both stay close to the bf16 module."""
    pt = mg
    from primus_amd.megatron import runtime

    runtime.set_num_microbatches(microbatches)
    res = {}
    for fuse in (True, False):
        runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                         turbo_grouped_gemm_without_padding=True, turbo_fuse_norm_into_quantize=fuse)
        torch.manual_seed(9)
        ln = pt.PrimusTurboLayerNormColumnParallelLinear(256, 160, config=_cfg(), bias=True)
        assert ln.fuse_norm_into_quantize is fuse
        with torch.no_grad():
            ln.layer_norm_weight.copy_(1 + 0.1 * torch.randn(256))
        ln.weight.main_grad = torch.zeros_like(ln.weight, dtype=torch.float32)
        ln.weight.grad_added_to_main_grad = False
        x = torch.randn(12, 8, 256, device=gpu).bfloat16().requires_grad_()
        dy = torch.randn(12, 8, 160, device=gpu).bfloat16()
        calls = []
        from primus_amd.pytorch import kernels as K
        import contextlib

        def hook(name, info):
            calls.append(name)
            return contextlib.nullcontext()

        K.set_launch_hook(hook)
        try:
            if fp4:
                ctx = pt.primus_turbo_fp4_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp4(pt))
            else:
                ctx = pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=_mxfp8(pt))
            with ctx:
                y, _ = ln(x)
            y.backward(dy)
        finally:
            K.set_launch_hook(None)
        assert ("rmsnorm_quantize" in calls) is fuse
        wgrad = ln.weight.main_grad.clone() if microbatches > 1 else ln.weight.grad.float()
        res[fuse] = (y.detach(), x.grad, ln.layer_norm_weight.grad, wgrad, ln.bias.grad)
        if fuse:
            y_bf16, _ = ln(x.detach())
            want = torch.nn.functional.linear(
                torch.nn.functional.rms_norm(x.detach(), [256], ln.layer_norm_weight, 1e-5), ln.weight, ln.bias)
            assert _cos(y_bf16, want) > 0.9999
            assert _cos(y, want) > (0.97 if fp4 else 0.999)
    for a, b in zip(res[True], res[False]):
        assert a.shape == b.shape and torch.equal(a, b)


@pytest.mark.parametrize("hybrid", [False, True])
@pytest.mark.parametrize("microbatches", [1, 2])
def test_linear_and_grouped_linear_under_the_tensorwise_recipe(mg, gpu, hybrid, microbatches):
    """The non-MX "current scaling" recipe through the same modules (quant_config.current_scaling(),
    primus_turbo.py:1087-1135): close to the bf16 module, and with several microbatches the cached row-wise
    weight copy (no transposed cache under current scaling, :1105-1115) gives the same gradients."""
    pt = mg
    from primus_amd.megatron import runtime
    from primus_amd.pytorch.core import Format, ScalingGranularity

    runtime.set_num_microbatches(microbatches)
    qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.TENSORWISE, format=Format.HYBRID if hybrid else Format.E4M3)
    assert qc.current_scaling() and not qc.mxfp8_scaling()
    torch.manual_seed(21)
    lin = pt.PrimusTurboLinear(256, 160, parallel_mode=None, config=_cfg(), bias=False, skip_bias_add=False)
    lin.weight.main_grad = torch.zeros_like(lin.weight, dtype=torch.float32)
    lin.weight.grad_added_to_main_grad = False
    x = torch.randn(16, 8, 256, device=gpu).bfloat16().requires_grad_()
    dy = torch.randn(16, 8, 160, device=gpu).bfloat16()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
        y, _ = lin(x)
    y.backward(dy)
    if microbatches > 1:
        assert lin.quantized_weight_buffer.tensor_scale_inv is not None and lin.quantized_weight_t_buffer is None
    xr = x.detach().clone().requires_grad_()
    wr = lin.weight.detach().clone().requires_grad_()
    yr = torch.nn.functional.linear(xr, wr)
    yr.backward(dy)
    wgrad = lin.weight.main_grad if microbatches > 1 else lin.weight.grad
    assert _cos(y, yr) > 0.998 and _cos(x.grad, xr.grad) > (0.99 if hybrid else 0.998)
    assert _cos(wgrad, wr.grad) > (0.99 if hybrid else 0.998)

    lens = [33, 0, 130, 1, 92]
    gl = pt.PrimusTurboColumnParallelGroupedLinear(5, 128, 96, config=_cfg())
    gl.weights.main_grad = torch.zeros_like(gl.weights, dtype=torch.float32)
    gl.weights.grad_added_to_main_grad = False
    xg = torch.randn(sum(lens), 128, device=gpu).bfloat16().requires_grad_()
    dyg = torch.randn(sum(lens), 96, device=gpu).bfloat16()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
        yg, _ = gl(xg, torch.tensor(lens))
    yg.backward(dyg)
    want = torch.cat([xs @ gl.weights[e].detach().t() for e, xs in enumerate(torch.split(xg.detach(), lens))])
    assert _cos(yg, want) > 0.998
    wg = gl.weights.main_grad if microbatches > 1 else gl.weights.grad
    assert not wg[1].any() and wg[0].abs().sum() > 0


@pytest.mark.parametrize("microbatches", [1, 2])
def test_fused_prologue_modules_under_the_tensorwise_recipe(mg, gpu, microbatches):
    """The modules that fold RMSNorm / the gated activation into the MX quantiser still work under the tensor-wise
    recipe: there the prologue runs as an operator of its own in front of the FP8 GEMM (the reference's sequence,
    primus_turbo.py:1689-1741 and the GroupedMLP forward), with the switches for the folded forms left on."""
    pt = mg
    from primus_amd.megatron import runtime
    from primus_amd.pytorch.core import Format, ScalingGranularity

    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=True, use_turbo_fused_act_with_probs=True,
                     turbo_fuse_norm_into_quantize=True)
    runtime.set_num_microbatches(microbatches)
    qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.TENSORWISE, format=Format.E4M3)

    def autocast():
        return pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc)

    torch.manual_seed(31)
    ln = pt.PrimusTurboLayerNormColumnParallelLinear(256, 160, config=_cfg(), bias=True)
    assert ln.fuse_norm_into_quantize
    with torch.no_grad():
        ln.layer_norm_weight.copy_(1 + 0.1 * torch.randn(256))
    ln.weight.main_grad = torch.zeros_like(ln.weight, dtype=torch.float32)
    ln.weight.grad_added_to_main_grad = False
    x = torch.randn(12, 8, 256, device=gpu).bfloat16().requires_grad_()
    dy = torch.randn(12, 8, 160, device=gpu).bfloat16()
    with autocast():
        y, _ = ln(x)
    y.backward(dy)
    xr = x.detach().clone().requires_grad_()
    wr, gr = ln.weight.detach().clone().requires_grad_(), ln.layer_norm_weight.detach().clone().requires_grad_()
    yr = torch.nn.functional.linear(torch.nn.functional.rms_norm(xr, [256], gr, 1e-5), wr, ln.bias.detach())
    yr.backward(dy)
    wgrad = ln.weight.main_grad if microbatches > 1 else ln.weight.grad
    assert _cos(y, yr) > 0.998 and _cos(x.grad, xr.grad) > 0.998
    assert _cos(wgrad, wr.grad) > 0.998 and _cos(ln.layer_norm_weight.grad, gr.grad) > 0.998

    mlp = _mlp(pt, gpu, 4, 256, 384)
    assert mlp.fuse_act_into_fc2
    lens = [100, 0, 37, 55]
    tpe = torch.tensor(lens, device=gpu)
    xm = torch.randn(sum(lens), 256, device=gpu).bfloat16()
    probs = torch.rand(sum(lens), device=gpu)
    dym = torch.randn(sum(lens), 256, device=gpu).bfloat16()

    def run(ctx):
        mlp.zero_grad(set_to_none=True)
        for lin in (mlp.linear_fc1, mlp.linear_fc2):
            lin.weights.main_grad = torch.zeros_like(lin.weights, dtype=torch.float32)
            lin.weights.grad_added_to_main_grad = False
            lin.set_is_first_microbatch()                    # every run is the first microbatch of a new step
        xi, pi = xm.clone().requires_grad_(), probs.clone().requires_grad_()
        with ctx:
            out, _ = mlp(xi, tpe, pi)
        out.backward(dym)
        grads = [(lin.weights.main_grad if microbatches > 1 and ctx is not plain else lin.weights.grad).float().clone()
                 for lin in (mlp.linear_fc1, mlp.linear_fc2)]
        return [out.detach(), xi.grad, pi.grad] + grads

    import contextlib

    plain = contextlib.nullcontext()
    want = run(plain)
    got = run(autocast())
    for name, a, b in zip(("y", "dx", "dprobs", "dw1", "dw2"), got, want):
        assert torch.isfinite(a.float()).all(), name
        assert _cos(a, b) > 0.995, (name, _cos(a, b))
    assert not got[3][1].any() and not got[4][1].any()       # the expert without tokens has no gradient


@pytest.mark.parametrize("recipe", ["bf16", "tensorwise", "mxfp8"])
def test_gradient_accumulation_fusion_adds_into_main_grad(mg, gpu, recipe):
    """config.gradient_accumulation_fusion: the wgrad GEMM adds into weight.main_grad itself
    (_fuse_wgrad_accum_pattern, primus_turbo.py:243-275: bf16 and tensor-wise FP8 in the reference; the MX
    recipes with the switch turbo_fuse_wgrad_accum_mx).  Two microbatches; the sum equals the unfused run's."""
    pt = mg
    from primus_amd.megatron import runtime
    from primus_amd.pytorch.core import Format, ScalingGranularity

    runtime.set_num_microbatches(2)
    qc = None
    if recipe == "tensorwise":
        qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.TENSORWISE, format=Format.HYBRID)
    elif recipe == "mxfp8":
        qc = _mxfp8(pt)
    res = {}
    for fuse in (False, True):
        runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                         turbo_grouped_gemm_without_padding=True, turbo_fuse_wgrad_accum_mx=True)
        torch.manual_seed(31)
        lin = pt.PrimusTurboLinear(256, 160, parallel_mode=None, config=_cfg(gradient_accumulation_fusion=fuse), bias=False,
                                   skip_bias_add=False)
        gl = pt.PrimusTurboColumnParallelGroupedLinear(3, 128, 96, config=_cfg(gradient_accumulation_fusion=fuse))
        for p_ in (lin.weight, gl.weights):
            p_.main_grad = torch.zeros_like(p_, dtype=torch.float32)
        outs = []
        calls = []
        for mb in range(2):
            for p_ in (lin.weight, gl.weights):
                p_.grad_added_to_main_grad = False
            x = torch.randn(16, 8, 256, device=gpu).bfloat16().requires_grad_()
            dy = torch.randn(16, 8, 160, device=gpu).bfloat16()
            xg = torch.randn(200, 128, device=gpu).bfloat16().requires_grad_()
            dyg = torch.randn(200, 96, device=gpu).bfloat16()
            if qc is not None:
                ctx = pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc)
            else:
                import contextlib
                ctx = contextlib.nullcontext()
            with ctx:
                assert (pt._fuse_wgrad_accum_pattern(lin.config, lin.weight) == "megatron") is fuse
                y, _ = lin(x)
                yg, _ = gl(xg, torch.tensor([70, 0, 130]))
            y.backward(dy)
            yg.backward(dyg)
            assert lin.weight.grad_added_to_main_grad is (fuse or qc is not None)
            outs += [y.detach(), x.grad, yg.detach(), xg.grad]
        res[fuse] = (outs, lin.weight.main_grad.clone(), gl.weights.main_grad.clone(), lin.weight.grad, gl.weights.grad)
    for a, b in zip(res[False][0], res[True][0]):
        assert torch.equal(a, b)
    if recipe == "bf16":     # outside an autocast the unfused run leaves the gradient in .grad (summed by autograd)
        assert not res[False][1].any() and not res[False][2].any()
        ref_lin, ref_gl = res[False][3].float(), res[False][4].float()
    else:
        ref_lin, ref_gl = res[False][1], res[False][2]
    for ref, got in ((ref_lin, res[True][1]), (ref_gl, res[True][2])):
        assert ref.abs().sum() > 0 and (ref - got).abs().max() <= 2.0 ** -6 * ref.abs().max()
    assert not res[True][2][1].any()
