"""Pre-shuffled MXFP4 layouts on the GPU: the byte permutations against the oracle, the GEMM wrapper that takes
pre-shuffled operands, and the config flags that ask for them."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _np(t):
    return t.view(torch.uint8).cpu().numpy()


@pytest.mark.parametrize("rows,row_bytes", [(16, 32), (32, 64), (48, 96), (128, 128), (512, 1440), (4096, 2048)])
def test_code_shuffle_and_back(gpu, rows, row_bytes):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator(device="cpu").manual_seed(rows + row_bytes)
    x = torch.randint(0, 256, (rows, row_bytes), dtype=torch.uint8, generator=g)
    xd = x.to(gpu)
    got = K.shuffle_codes_impl(xd)
    assert got.shape == xd.shape and got.dtype == xd.dtype
    assert np.array_equal(_np(got), o.shuffle_codes_16x16(x.numpy()))
    assert torch.equal(K.shuffle_codes_impl(got, inverse=True), xd)
    fp4 = K.shuffle_codes_impl(xd.view(torch.float4_e2m1fn_x2))
    assert fp4.dtype == torch.float4_e2m1fn_x2 and torch.equal(fp4.view(torch.uint8), got)


@pytest.mark.parametrize("rows,blocks", [(1, 1), (32, 8), (256, 8), (100, 5), (300, 90), (2880, 90), (4096, 128)])
def test_scale_shuffle_and_back(gpu, rows, blocks):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator(device="cpu").manual_seed(rows * 3 + blocks)
    s = torch.randint(1, 256, (rows, blocks), dtype=torch.uint8, generator=g)
    sd = s.to(gpu)
    got = K.shuffle_scales_impl(sd)
    assert tuple(got.shape) == K.shuffled_scale_shape(rows, blocks) == o.shuffled_scale_shape(rows, blocks)
    assert np.array_equal(_np(got), o.shuffle_e8m0(s.numpy()))
    assert torch.equal(K.unshuffle_scales_impl(got, rows, blocks), sd)
    e8 = K.shuffle_scales_impl(sd.view(torch.float8_e8m0fnu))
    assert e8.dtype == torch.float8_e8m0fnu and torch.equal(e8.view(torch.uint8), got)


def test_shuffle_argument_errors(gpu):
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    with pytest.raises(ValueError, match="rows % 16"):
        K.shuffle_codes_impl(torch.zeros(8, 32, dtype=torch.uint8, device=gpu))
    with pytest.raises(ValueError, match="rows % 16"):
        K.shuffle_codes_impl(torch.zeros(16, 48, dtype=torch.uint8, device=gpu))
    with pytest.raises(ValueError, match="pre-shuffled scales"):
        K.unshuffle_scales_impl(torch.zeros(256, 8, dtype=torch.uint8, device=gpu), 300, 8)
    with pytest.raises(ValueError):
        K.shuffle_codes_impl(torch.zeros(16, 32, dtype=torch.uint8))            # a CPU tensor
    lib = _lib.load()
    buf = torch.zeros(16 * 32 + 16, dtype=torch.uint8, device=gpu)
    p = buf.data_ptr()
    assert lib.mxl_shuffle_codes(p, 16, 32, p, 0, None) == -1                    # in place
    assert lib.mxl_shuffle_codes(p, 16, 33, p + 16, 0, None) == -1               # ragged rows
    assert lib.mxl_shuffle_codes(p + 1, 16, 32, p + 32, 0, None) == -1           # unaligned
    assert lib.mxl_shuffle_codes(None, 0, 32, None, 0, None) == 0                # nothing to do
    assert lib.mxl_shuffle_scales(p, 4, 4, p, 0, None) == -1                     # in place
    assert lib.mxl_shuffle_scales(None, 0, 4, None, 1, None) == 0


@pytest.mark.parametrize("m,n,k", [(128, 256, 256), (100, 192, 96), (300, 64, 640), (1000, 2880, 2880), (37, 544, 1152)])
def test_gemm_fp4_takes_preshuffled_operands(gpu, m, n, k, monkeypatch):
    """a: plain codes with pre-shuffled scales, b: pre-shuffled codes and scales (what the reference's MXFP4 linear
    hands to gemm_fp4_impl with its switch on): the result equals the plain call bit for bit."""
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core.low_precision import ScalingGranularity

    torch.manual_seed(m + n + k)
    x = torch.randn(m, k, device=gpu).bfloat16()
    w = (torch.randn(n, k, device=gpu) * 0.05).bfloat16()
    a, a_s, _, _ = K.quantize_mx_impl(x, _lib.FMT_E2M1, rowwise=True, colwise=False, pad_to=128)
    b, b_s, _, _ = K.quantize_mx_weight_2d_impl(w, _lib.FMT_E2M1, rowwise=True, colwise=False, pad_to=128)
    gran = ScalingGranularity.MX_BLOCKWISE.value
    plain = K.gemm_fp4_impl(a, a_s, False, b, b_s, True, torch.bfloat16, False, granularity=gran)
    shuffled_b = K.shuffle_codes_impl(b)

    def no_unshuffle(*args, **kw):      # the GEMM reads the pre-shuffled codes as they lie
        raise AssertionError("the weight codes were converted back in front of the GEMM")

    monkeypatch.setattr(K, "shuffle_codes_impl", no_unshuffle)
    pre = K.gemm_fp4_impl(a, K.shuffle_scales_impl(a_s), False, shuffled_b, K.shuffle_scales_impl(b_s), True,
                          torch.bfloat16, False, granularity=gran, preshuffled=True)
    assert torch.equal(plain, pre)
    monkeypatch.undo()
    pre = K.gemm_fp4_impl(a, K.shuffle_scales_impl(a_s), False, K.shuffle_codes_impl(b), K.shuffle_scales_impl(b_s), True,
                          torch.bfloat16, False, granularity=gran, preshuffled=True)
    assert torch.equal(plain, pre)
    want = o.gemm_nt_ref(_np(a), _np(a_s), _np(b), _np(b_s), o.FMT_E2M1, o.FMT_E2M1)
    got = plain.float().cpu().numpy()
    ref = o.bf16_bits_to_f32(want)
    assert np.abs(got - ref).max() <= 1e-2 * max(np.abs(ref).max(), 1e-30)


def test_config_flags_and_tensor_accessors(gpu):
    from primus_amd.pytorch.core.low_precision import Float4QuantConfig, Format, MXScalingRecipe, float4_e2m1fn_x2
    from primus_amd.pytorch.core.quantized_tensor import QuantizedTensor
    import primus_amd.pytorch as pt

    torch.manual_seed(5)
    w = (torch.randn(64, 128, device=gpu) * 0.05).bfloat16()
    x = torch.randn(96, 128, device=gpu).bfloat16()
    recipe = MXScalingRecipe(use_2d_block=True, shuffle_scale=True, shuffle_out=True)
    q = QuantizedTensor.quantize(w, dest_dtype=float4_e2m1fn_x2, scaling_recipe=recipe, axis=-1)
    codes, scales = _np(q.codes), _np(q.scales)
    assert np.array_equal(_np(q.preshuffled_codes()), o.shuffle_codes_16x16(codes))
    assert np.array_equal(_np(q.preshuffled_scales()), o.shuffle_e8m0(scales))
    # the operators compute the same with the switch on
    y0 = pt.ops.gemm_fp4(x, w, trans_b=True, config=Float4QuantConfig(format=Format.E2M1_X2))
    y1 = pt.ops.gemm_fp4(x, w, trans_b=True, config=Float4QuantConfig(format=Format.E2M1_X2, use_preshuffle=True))
    assert torch.equal(y0, y1)
