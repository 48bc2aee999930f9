"""Configuration 1 of the baseline at full size (dense 4096 x 4096 x 4096, seed 1001), a per-element error bound
for the GEMM, and the two low-level entry points called with the reference's literal argument lists.

Per-element bound (instead of one normaliser for the whole tensor): a bf16 output of an fp32-accumulated dot
product of exactly representable terms may differ from the exact value by its own rounding (2^-8 relative; 2^-9
for round-to-nearest, doubled for ties that fall the other way in the reference) plus the accumulation error,
(K + 1024) * 2^-23 * sum |a_i b_i|: K fp32 additions and a floor of 2^-13 for the MFMA's 64-term dot product, whose
products are aligned to a common exponent in a finite datapath (measured excess over the output rounding: at most
2^-16 of sum |a_i b_i|, at K = 128 as at K = 14336).
"""

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _u8(t):
    return t.view(torch.uint8).cpu().numpy()


def _bf(t):
    return o.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)


def elementwise_bound(want: np.ndarray, absdot: np.ndarray, k: int) -> np.ndarray:
    return 2.0 ** -8 * np.abs(want) + (k + 1024) * 2.0 ** -23 * absdot + 1e-30


def test_cfg1_dense_4096(gpu):
    """X [4096, 4096] ~ N(0, 1), W [4096, 4096] ~ N(0, 0.02), MXFP8 E4M3: ALL quantised bytes and scales against
    the oracle, every output element against the oracle's dequantise-then-fp32-matmul."""
    import primus_amd.pytorch as pt
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    C.load()
    g = torch.Generator(device="cpu").manual_seed(1001)
    x = torch.randn(4096, 4096, generator=g).bfloat16()
    w = (torch.randn(4096, 4096, generator=g) * 0.02).bfloat16()
    xb, wb = o.to_bf16_bits(x), o.to_bf16_bits(w)
    xq, xs = C.quantize_rowwise(xb, o.FMT_E4M3)           # the C restatement is byte-equal to the numpy oracle (test_oracle_c.py)
    wq, ws, wqt, wst = C.quantize_2d(wb, o.FMT_E4M3)
    # the numpy oracle itself on a band, so that the check does not rest on the C port alone
    q2, s2 = o.quantize_mx_rowwise(x[:64], o.FMT_E4M3)
    assert np.array_equal(q2, xq[:64]) and np.array_equal(s2, xs[:64])
    q2, s2, _, _ = o.quantize_mx_2d(w[:64], o.FMT_E4M3)
    assert np.array_equal(q2, wq[:64]) and np.array_equal(s2, ws[:64])

    xd, wd = x.to(gpu), w.to(gpu)
    gq, gs, _, _ = K.quantize_mx_impl(xd, o.FMT_E4M3, rowwise=True, colwise=False)
    assert np.array_equal(_u8(gq), xq) and np.array_equal(_u8(gs), xs)
    hq, hs, hqt, hst = K.quantize_mx_weight_2d_impl(wd, o.FMT_E4M3, rowwise=True, colwise=True)
    assert np.array_equal(_u8(hq), wq) and np.array_equal(_u8(hs), ws)
    assert np.array_equal(_u8(hqt), wqt) and np.array_equal(_u8(hst), wst)

    cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0,
                            block_size=32)
    y = pt.ops.gemm_fp8(xd, wd, trans_a=False, trans_b=True, out_dtype=None, config=cfg)
    got = _bf(y)
    a = torch.from_numpy(C.dequantize(xq, xs, o.FMT_E4M3))
    b = torch.from_numpy(C.dequantize(wq, ws, o.FMT_E4M3))
    want = (a.double() @ b.double().t()).numpy()          # exact products, float64 sums
    absdot = (a.abs() @ b.abs().t()).double().numpy()
    err = np.abs(got - want)
    bound = elementwise_bound(want, absdot, 4096)
    bad = err > bound
    assert not bad.any(), f"{int(bad.sum())} elements outside the bound; worst ratio {float((err / bound).max()):.2f}"
    assert err.max() <= 1e-2 * np.abs(want).max()          # the outer envelope of the path's stated tolerance
    # and against the reference's formulation (fp32 matmul, bf16 result) within a bf16 ulp
    ref = o.bf16_bits_to_f32(o.f32_to_bf16_bits((a @ b.t()).numpy())).astype(np.float64)
    assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max()


@pytest.mark.parametrize("lens,n,k", [([300, 0, 5, 695], 320, 288), ([200, 200, 200], 512, 96)])
def test_variable_k_with_the_references_argument_list(gpu, lens, n, k):
    """grouped_gemm_fp8_variable_k_impl exactly as zbpp_gemm.py:710-724 calls it: 13 arguments, no token count."""
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core.low_precision import ScalingGranularity

    m = sum(lens)
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    dy = torch.randn(m, n, generator=g).bfloat16()
    dyT, dysT = o.quantize_mx_colwise_segmented(dy, lens, o.FMT_E4M3)
    xT, xsT = o.quantize_mx_colwise_segmented(x, lens, o.FMT_E4M3)
    want = o.grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, lens, o.FMT_E4M3, o.FMT_E4M3, out_bf16=False)
    dev = lambda a_, dt: torch.from_numpy(np.ascontiguousarray(a_)).to(gpu).view(dt)  # noqa: E731
    _a_fp8, _a_scale_inv = dev(xT, torch.float8_e4m3fn), dev(xsT, torch.float8_e8m0fnu)
    _grad_out_fp8, _grad_out_scale_inv = dev(dyT, torch.float8_e4m3fn), dev(dysT, torch.float8_e8m0fnu)
    _group_lens = torch.tensor(lens, dtype=torch.int64, device=gpu)
    _group_offs = K.group_offs_from_lens(_group_lens)
    b_grad = K.grouped_gemm_fp8_variable_k_impl(
        _a_fp8,
        _grad_out_fp8,
        _a_scale_inv,
        _grad_out_scale_inv,
        _group_lens,
        _group_offs,
        trans_a=True,
        trans_b=False,
        trans_c=True,
        out_dtype=torch.bfloat16,
        granularity=ScalingGranularity.MX_BLOCKWISE.value,
        num_cu=None,
        default_backend=0,
    )
    got = _bf(b_grad)
    assert got.shape == want.shape == (len(lens), n, k)
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    for e, ln in enumerate(lens):
        if ln == 0:
            assert not got[e].any()


def test_dual_op_under_the_references_namespace(gpu):
    """torch.ops.primus_turbo_cpp_extension.quantize_mxfp4_dual with the 13 arguments of
    primus_turbo_mxfp4_local.py:147-161 (the activation recipe without the transform): bytes against the oracle."""
    import primus_amd.megatron.extensions.primus_turbo_mxfp4_local as m4  # noqa: F401  (registers the op)

    torch.manual_seed(8)
    x = torch.randn(100, 96, device=gpu).bfloat16()
    row, row_s, col, col_s = torch.ops.primus_turbo_cpp_extension.quantize_mxfp4_dual(
        x, torch.float4_e2m1fn_x2, 128, False, False, False, False, False, False, False, False, False, False)
    assert tuple(row.shape) == (100, 64) and tuple(row_s.shape) == (100, 4)
    assert tuple(col.shape) == (96, 64) and tuple(col_s.shape) == (96, 4)
    q, s = o.quantize_mx_rowwise(x.cpu(), o.FMT_E2M1)
    assert np.array_equal(_u8(row)[:, :48], q) and np.array_equal(_u8(row_s)[:, :3], s)
    qT, sT = o.quantize_mx_colwise_segmented(x.cpu(), [100], o.FMT_E2M1)
    assert np.array_equal(_u8(col), qT) and np.array_equal(_u8(col_s), sT)
