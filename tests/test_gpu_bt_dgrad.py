"""dgrad on the ROW-WISE weight codes (``MXL_GF_B_TRANSPOSED``): with 2-D 32 x 32 blocks the transposed copy of a weight
is its row-wise codes transposed, so the ring kernel reads them as they lie (transposing LDS reads) and the weight
quantiser writes only the transposed copy's scales.  Everything here is compared BIT FOR BIT with the route through a
transposed copy of the codes, which the other GEMM tests hold against the oracle."""

import pytest
import torch

from primus_amd import _lib

pytestmark = pytest.mark.gpu

L = 2   # K-step-major


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("lens,n,k", [
    ([300, 0, 129, 700], 256, 384),
    ([1000], 512, 128),
    ([5, 250, 257], 640, 896),          # k (the dgrad's output width) not a multiple of the 256-wide tile
    ([64] * 16, 128, 256),
])
@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
def test_dgrad_from_rowwise_codes_matches_the_transposed_copy(gpu, lens, n, k, fmt):
    from primus_amd.pytorch import kernels as K

    FMT, L = (_lib.FMT_E4M3, 2) if fmt == "e4m3" else (_lib.FMT_E2M1, 3)     # E2M1 x E2M1: steps of 128 elements
    G, m = len(lens), sum(lens)
    gen = torch.Generator().manual_seed(n + k + m)
    w = (torch.randn(G, n, k, generator=gen) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(m, n, generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    full = K.quantize_mx_weight_2d_impl(w, FMT, rowwise=True, colwise=True, pad_to=128, kchunk=L)
    lean = K.quantize_mx_weight_2d_impl(w, FMT, rowwise=True, colwise=True, pad_to=128, kchunk=L, col_scales_only=True)
    assert lean[2] is None
    # the same copies, minus one (a scale panel's bytes past a row's last block are never written: compare the blocks)
    assert _same(full[0], lean[0])
    assert _same(K.unpanel(full[1].view(torch.uint8), k // 32), K.unpanel(lean[1].view(torch.uint8), k // 32))
    assert _same(K.unpanel(full[3].view(torch.uint8), n // 32), K.unpanel(lean[3].view(torch.uint8), n // 32))
    dq = K.quantize_mx_impl(dy, FMT, rowwise=True, colwise=False, group_lens=gl, pad_to=128, kchunk=L)
    want = K.grouped_gemm_mx_nt_impl(dq[0], dq[1], full[2], full[3], gl, kchunk=L)
    got = K.grouped_gemm_mx_nt_impl(dq[0], dq[1], lean[0], lean[3], gl, kchunk=L, b_transposed=True)
    assert got.shape == (m, k) and _same(got, want)
    if G == 1:
        got = K.gemm_mx_nt_impl(dq[0], dq[1], lean[0], lean[3], kchunk=L, b_transposed=True)
        assert _same(got, want)


@pytest.mark.parametrize("grouped", [True, False])
@pytest.mark.parametrize("recipe", ["mx", "mxfp4", "tensorwise_e4m3", "tensorwise_hybrid"])
def test_operator_gradients_do_not_depend_on_the_route(gpu, grouped, recipe):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    if recipe == "mx":
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0, block_size=32)
    elif recipe == "mxfp4":
        from primus_amd.pytorch.core import Float4QuantConfig
        cfg = Float4QuantConfig(activation_format=Format.E2M1_X2)
    else:
        cfg = Float8QuantConfig(format=Format.E4M3 if recipe.endswith("e4m3") else Format.HYBRID, granularity=ScalingGranularity.TENSORWISE)
    lens = [200, 0, 312] if grouped else [512]
    G, m, n, k = len(lens), sum(lens), 384, 256
    gen = torch.Generator().manual_seed(17)
    x0 = torch.randn(m, k, generator=gen).bfloat16().to(gpu)
    w0 = (torch.randn(*((G, n, k) if grouped else (n, k)), generator=gen) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(m, n, generator=gen).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    outs = []
    try:
        for flag in (True, False):
            turbo.ops.set_dgrad_reads_rowwise_weight(flag)
            x, w = x0.clone().requires_grad_(), w0.clone().requires_grad_()
            if recipe == "mxfp4":
                y = turbo.ops.grouped_gemm_fp4(x, w, gl, config=cfg) if grouped else turbo.ops.gemm_fp4(x, w, trans_b=True, config=cfg)
            else:
                y = turbo.ops.grouped_gemm_fp8(x, w, gl, config=cfg) if grouped else turbo.ops.gemm_fp8(x, w, trans_b=True, config=cfg)
            y.backward(dy)
            outs.append((y.detach(), x.grad, w.grad))
    finally:
        turbo.ops.set_dgrad_reads_rowwise_weight(True)
    for a, b in zip(*outs):
        assert _same(a, b)


def test_entry_point_refuses_what_the_mode_does_not_serve(gpu):
    lib = _lib.load()
    z = torch.zeros(1 << 16, dtype=torch.uint8, device=gpu)
    p = z.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    # without the K-step-major flag, and with E2M1 weights
    assert lib.mxl_grouped_gemm_nt_ex(p, p, 0, p, p, 0, p, None, 1, 64, 128, 128, _lib.GF_B_TRANSPOSED, st) == -1
    assert lib.mxl_grouped_gemm_nt_ex(p, p, 0, p, p, 1, p, None, 1, 64, 128, 128, _lib.GF_KSTEP | _lib.GF_B_TRANSPOSED, st) == -1
