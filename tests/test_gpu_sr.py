"""Stochastic rounding of MXFP4 gradients on the GPU: every code byte against the oracle (same
counter hash, same integer rounding), the scales against the round-to-nearest quantiser, and the
statistical property that makes it worth having (the mean over seeds converges to the unquantised
gradient GEMM, which round-to-nearest cannot)."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _u8(t):
    return t.view(torch.uint8).cpu().numpy()


@pytest.mark.parametrize("lens,cols", [([33, 0, 130, 1, 92], 160), ([300], 2048), (None, 64), ([0, 0], 96), ([257, 255], 128)])
@pytest.mark.parametrize("seed", [0, 0x1234_5678_9ABC_DEF1])
def test_sr_codes_match_the_oracle(gpu, lens, cols, seed):
    from primus_amd.pytorch import kernels as K

    rows = 257 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-3, 3, cols)[None, :]).bfloat16()
    if rows:
        x[0, 0] = 0.0
        x[rows // 2, :32] = 0.0                       # an all-zero block: scale byte 0, codes 0
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    q, s, qT, sT = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=True, group_lens=gl, pad_to=128,
                                      sr_seed=seed)
    q0, s0, qT0, sT0 = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=True, group_lens=gl, pad_to=128)
    assert torch.equal(s.view(torch.uint8), s0.view(torch.uint8)) and torch.equal(sT.view(torch.uint8), sT0.view(torch.uint8))
    if rows:
        oq, os_ = o.quantize_mx_rowwise_sr(x, seed)
        assert np.array_equal(_u8(q)[:, : cols // 2], oq)
        assert np.array_equal(_u8(s)[:, : cols // 32], os_)
        assert not _u8(q)[:, cols // 2:].any()
        assert (_u8(q) != _u8(q0)).mean() > 0.05            # it does round differently from nearest-even
    oqT, osT = o.quantize_mx_colwise_segmented_sr(x, [rows] if lens is None else lens, seed)
    assert np.array_equal(_u8(qT), oqT) and np.array_equal(_u8(sT), osT)
    # one copy at a time gives the same bytes as the dual launch
    if rows:
        assert torch.equal(K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=False, pad_to=128, sr_seed=seed)[0]
                           .view(torch.uint8), q.view(torch.uint8))
    assert torch.equal(K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=False, colwise=True, group_lens=gl, sr_seed=seed)[2]
                       .view(torch.uint8), qT.view(torch.uint8))


def test_sr_with_non_finite_blocks_and_bad_arguments(gpu):
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    x = torch.randn(64, 64).bfloat16()
    x[3, 5] = float("inf")
    x[40, 33] = float("nan")
    q, s, qT, sT = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=True, sr_seed=77)
    oq, os_ = o.quantize_mx_rowwise_sr(x, 77)
    oqT, osT = o.quantize_mx_colwise_segmented_sr(x, [64], 77)
    assert np.array_equal(_u8(q), oq) and np.array_equal(_u8(s), os_)
    assert np.array_equal(_u8(qT), oqT) and np.array_equal(_u8(sT), osT)
    with pytest.raises(ValueError):
        K.quantize_mx_impl(x.to(gpu), o.FMT_E4M3, sr_seed=1)
    lib = _lib.load()
    xd = x.to(gpu)
    buf = torch.empty(64 * 64, dtype=torch.uint8, device=gpu)
    assert lib.mxl_quantize_sr(xd.data_ptr(), 64, 64, 64, _lib.FMT_E4M3, 0, None, 0, buf.data_ptr(), buf.data_ptr(),
                               None, None, 1, None) == -1


def test_gemm_fp4_gradient_sr_is_reproducible_and_unbiased(gpu):
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import Float4QuantConfig

    torch.manual_seed(2)
    M, K_, N = 256, 256, 384
    x = torch.randn(M, K_, device=gpu).bfloat16()
    w = (torch.randn(N, K_, device=gpu) * 0.05).bfloat16()
    dy = torch.randn(M, N, device=gpu).bfloat16()

    def grads(cfg):
        xx, ww = x.clone().requires_grad_(), w.clone().requires_grad_()
        pt.ops.gemm_fp4(xx, ww, config=cfg).backward(dy)
        return xx.grad.float(), ww.grad.float()

    rne = grads(Float4QuantConfig(use_gradient_sr=False))
    sr_cfg = Float4QuantConfig(use_gradient_sr=True)
    pt.ops.manual_sr_seed(10)
    a = grads(sr_cfg)
    b = grads(sr_cfg)                     # next seeds of the sequence: another draw
    pt.ops.manual_sr_seed(10)
    a2 = grads(sr_cfg)
    assert torch.equal(a[0], a2[0]) and torch.equal(a[1], a2[1])
    assert not torch.equal(a[0], b[0]) and not torch.equal(a[0], rne[0])
    # the gradient GEMMs with an unquantised dY (weights and activations still MXFP4) are what the
    # mean over draws approaches; nearest-even keeps its full rounding error
    from primus_amd.pytorch import kernels as K
    wq, ws, wqT, wsT = K.quantize_mx_weight_2d_impl(w, o.FMT_E2M1, rowwise=True, colwise=True)
    w_deq = torch.tensor(o.dequantize_mx(_u8(wqT), _u8(wsT), o.FMT_E2M1), device=gpu)       # [K, N]
    dx_ref = dy.float() @ w_deq.T
    n = 16
    pt.ops.manual_sr_seed(99)
    mean = sum(grads(sr_cfg)[0] for _ in range(n)) / n
    err_sr = (mean - dx_ref).norm().item()
    err_rne = (rne[0] - dx_ref).norm().item()
    assert err_sr < 0.6 * err_rne, (err_sr, err_rne)
    pt.ops.manual_sr_seed(None)


def test_dual_op_with_sr_flags(gpu):
    from primus_amd.megatron.extensions import primus_turbo_mxfp4_local as loc
    from primus_amd.pytorch import kernels as K

    x = torch.randn(200, 96, device=gpu).bfloat16()
    K.manual_sr_seed(4)
    q, s, qt, st = loc._quantize_grad_dual(x, use_sr=True)
    K.manual_sr_seed(4)
    seed = K.next_sr_seed()
    oq, os_ = o.quantize_mx_rowwise_sr(x.cpu(), seed)
    oqT, osT = o.quantize_mx_colwise_segmented_sr(x.cpu(), [200], seed)
    assert np.array_equal(_u8(q)[:, :48], oq) and np.array_equal(_u8(qt), oqT)
    assert np.array_equal(_u8(s)[:, :3], os_) and np.array_equal(_u8(st), osT)
    # only the row-wise copy stochastic: the transposed one is the nearest-even copy
    q1, s1, qt1, st1 = loc._quantize_mxfp4_dual_op(x, loc._FP4_DTYPE, 128, False, True, False, False, False, False,
                                                   False, False, False, False)
    q0, s0, qt0, st0 = loc._quantize_grad_dual(x, use_sr=False)
    assert torch.equal(qt1.view(torch.uint8), qt0.view(torch.uint8)) and not torch.equal(q1.view(torch.uint8), q0.view(torch.uint8))
    with pytest.raises(NotImplementedError):
        loc._quantize_mxfp4_dual_op(x[:128], loc._FP4_DTYPE, 128, True, True, False, True, True, False, False, False, False, False)
    K.manual_sr_seed(None)
