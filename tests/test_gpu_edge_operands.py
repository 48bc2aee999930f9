"""Operand cases at the edges of the operators: cached weight copies whose K is not a multiple of the GEMM's
granularity, a main_grad that is not float32 under gradient-accumulation fusion, E5M2 codes through dequantize."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()


def test_cached_pair_from_quantize_with_k_160(gpu):
    """A pair built with the reference's own calls (QuantizedTensor.quantize(w, axis=-1 / -2), primus_turbo.py:321-354)
    keeps K = 160; the operator pads the activations to 192: both are brought to the same length."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import (Float8QuantConfig, Format, MXScalingRecipe, QuantizedTensor, QuantizedTensorPair,
                                         ScaleDtype, ScalingGranularity, float8_e4m3)

    cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0, block_size=32)
    torch.manual_seed(1)
    x = torch.randn(70, 160, device=gpu).bfloat16().requires_grad_()
    w = (torch.randn(96, 160, device=gpu) * 0.05).bfloat16()
    recipe = MXScalingRecipe(use_2d_block=True)
    row = QuantizedTensor.quantize(w, float8_e4m3, ScalingGranularity.MX_BLOCKWISE, 32, recipe, axis=-1)
    col = QuantizedTensor.quantize(w, float8_e4m3, ScalingGranularity.MX_BLOCKWISE, 32, recipe, axis=-2)
    pair = QuantizedTensorPair(row, col)
    y = turbo.ops.gemm_fp8(x, pair, config=cfg)
    want = turbo.ops.gemm_fp8(x, w, config=cfg)
    assert tuple(y.shape) == (70, 96) and torch.equal(y, want)
    (dx,) = torch.autograd.grad(y, x, torch.ones_like(y))
    (dxw,) = torch.autograd.grad(want, x, torch.ones_like(want))
    assert torch.equal(dx, dxw)
    # and directly through the low-level GEMM: one operand padded, the other not
    from primus_amd.pytorch import kernels as K

    a, a_s, _, _ = K.quantize_mx_impl(x.detach(), 0, rowwise=True, colwise=False, pad_to=128)
    assert a.shape[1] == 256 and row.rowmajor_codes().shape[-1] == 160
    got = K.gemm_mx_nt_impl(a, a_s, row.rowmajor_codes(), row.rowmajor_scales())
    assert torch.equal(got, want)


@pytest.mark.parametrize("recipe", ["bf16", "mxfp8", "tensorwise"])
def test_fused_accumulation_into_a_bf16_main_grad(gpu, recipe):
    """fuse_bgrad_accum_pattern="megatron" with a main_grad that is not float32 (gradients reduced in bf16): the
    weight gradient is added after the GEMM instead of inside it, as the reference's bridge does for any dtype
    (primus_turbo.py:166-240)."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    torch.manual_seed(2)
    x = torch.randn(200, 256, device=gpu).bfloat16().requires_grad_()
    w = (torch.randn(128, 256, device=gpu) * 0.05).bfloat16().requires_grad_()
    dy = torch.randn(200, 128, device=gpu).bfloat16()
    w.main_grad = torch.full((128, 256), 0.5, device=gpu, dtype=torch.bfloat16)
    w.grad_added_to_main_grad = False
    if recipe == "bf16":
        y = turbo.ops.gemm(x, w, fuse_bgrad_accum_pattern="megatron")
    else:
        cfg = (Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0, block_size=32)
               if recipe == "mxfp8" else Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.TENSORWISE))
        y = turbo.ops.gemm_fp8(x, w, config=cfg, fuse_bgrad_accum_pattern="megatron")
    y.backward(dy)
    assert w.grad_added_to_main_grad
    want = 0.5 + dy.float().t() @ x.detach().float()
    assert w.main_grad.dtype == torch.bfloat16 and _cos(w.main_grad, want) > 0.998


def test_dequantize_e5m2_codes(gpu):
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core import QuantizedTensor, ScalingGranularity

    codes = torch.arange(256, dtype=torch.uint8).repeat(4).reshape(8, 128)
    scales = torch.full((8, 4), 127, dtype=torch.uint8)
    scales[1] = 130
    out = K.dequantize_mx_impl(codes.view(torch.float8_e5m2).to(gpu), scales.to(gpu))
    want = codes.view(torch.float8_e5m2).float() * torch.exp2(scales.float() - 127).repeat_interleave(32, 1)
    got = out.float().cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan) and torch.equal(got[~nan], want.bfloat16().float()[~nan])
    # a tensor-wise scaled E5M2 copy comes back to within the format's precision
    x = torch.randn(64, 128, device=gpu).bfloat16()
    q = QuantizedTensor.quantize(x, torch.float8_e5m2, ScalingGranularity.TENSORWISE, None, None, axis=-1)
    back = q.dequantize()
    assert back.shape == x.shape and float((back.float() - x.float()).abs().max()) <= 0.125 * float(x.float().abs().max())
    codes_o, sinv = o.quantize_tensorwise(x.cpu(), o.FMT_E5M2)
    want = (o.decode_e5m2(codes_o) * sinv).astype(np.float32)
    assert np.array_equal(back.float().cpu().numpy(), torch.from_numpy(want).bfloat16().float().numpy())
