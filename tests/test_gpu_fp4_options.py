"""The MXFP4 recipe's quantiser options on the GPU.

Stochastic rounding of gradients: every code byte against the oracle (same counter hash, same
integer rounding), the scales against the round-to-nearest quantiser, and the statistical property
that makes it worth having (the mean over seeds converges to the unquantised gradient GEMM, which
round-to-nearest cannot).  Randomised Hadamard transform of the transposed copies: every byte against
the oracle, and the wgrad GEMM of two transformed operands against the untransformed contraction."""

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
    assert lib.mxl_quantize_ex(xd.data_ptr(), 64, 64, 48, _lib.FMT_E2M1, 0, None, 0, buf.data_ptr(), buf.data_ptr(),
                               None, None, _lib.QF_SR, 1, 0, None) == -1           # row_ld below cols
    assert lib.mxl_quantize_ex(xd.data_ptr(), 64, 64, 64, _lib.FMT_E4M3, 0, None, 0, buf.data_ptr(), buf.data_ptr(),
                               None, None, _lib.QF_SR, 1, 0, None) == -1           # stochastic rounding is E2M1 only


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
    q, s, qt, st = loc._quantize_grad_dual(x, use_sr=True)          # gradients: SR on both copies, transform on the second
    K.manual_sr_seed(4)
    seed = K.next_sr_seed()
    oq, os_ = o.quantize_mx_rowwise_sr(x.cpu(), seed)
    oqT, osT = o.quantize_mx_colwise_segmented_fp4(x.cpu(), [200], sr_seed=seed, rht_signs=loc.RHT_SIGNS)
    assert np.array_equal(_u8(q)[:, :48], oq) and np.array_equal(_u8(qt), oqT)
    assert np.array_equal(_u8(s)[:, :3], os_) and np.array_equal(_u8(st), osT)
    # only the row-wise copy stochastic: the transposed one is the nearest-even copy
    q1, s1, qt1, st1 = loc._quantize_mxfp4_dual_op(x, loc._FP4_DTYPE, 128, False, True, False, False, False, False,
                                                   False, False, False, False)
    q0, s0, qt0, st0 = loc._quantize_grad_dual(x, use_sr=False, use_rht=False)
    assert torch.equal(qt1.view(torch.uint8), qt0.view(torch.uint8)) and not torch.equal(q1.view(torch.uint8), q0.view(torch.uint8))
    with pytest.raises(NotImplementedError):
        loc._quantize_mxfp4_dual_op(x[:128], loc._FP4_DTYPE, 128, True, True, False, True, True, False, False, False, False, False)
    K.manual_sr_seed(None)


@pytest.mark.parametrize("lens,cols", [([33, 0, 130, 1, 92], 160), ([300], 2048), (None, 64), ([0, 0], 96), ([257, 255], 128)])
@pytest.mark.parametrize("signs,seed", [(0xA6C9, None), (0, None), (0xFFFF, 31337)])
def test_hadamard_transposed_copy_matches_the_oracle(gpu, lens, cols, signs, seed):
    """colwise_use_rht: every byte of the transposed copy (codes and scales) equals the oracle's
    quantisation of the oracle's transform -- the fp32 butterflies run in the same order on both
    sides -- with round-to-nearest and with stochastic rounding on top; the row-wise copy of the
    same launch is the untransformed one."""
    from primus_amd.pytorch import kernels as K

    rows = 257 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + cols + signs)
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-2, 2, cols)[None, :]).bfloat16()
    if rows:
        x[rows // 3, :] *= 50.0
    glens = [rows] if lens is None else lens
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    q, s, qT, sT = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=True, group_lens=gl, pad_to=128,
                                      sr_seed=seed, rht_signs=signs)
    oqT, osT = o.quantize_mx_colwise_segmented_fp4(x, glens, sr_seed=seed, rht_signs=signs)
    assert np.array_equal(_u8(qT), oqT) and np.array_equal(_u8(sT), osT)
    plain = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=True, colwise=True, group_lens=gl, pad_to=128, sr_seed=seed)
    assert torch.equal(q.view(torch.uint8), plain[0].view(torch.uint8)) and torch.equal(s.view(torch.uint8), plain[1].view(torch.uint8))
    only = K.quantize_mx_impl(x.to(gpu), o.FMT_E2M1, rowwise=False, colwise=True, group_lens=gl, sr_seed=seed, rht_signs=signs)
    assert only[0] is None and torch.equal(only[2].view(torch.uint8), qT.view(torch.uint8))
    if rows > 64:
        assert not torch.equal(qT.view(torch.uint8), plain[2].view(torch.uint8))


def test_hadamard_wgrad_is_the_same_contraction(gpu):
    """Both wgrad operands transformed with the same signs: the GEMM result stays the wgrad (the
    transform is orthogonal), and for heavy-tailed operands it is closer to the bf16 result than
    the untransformed MXFP4 one."""
    from primus_amd.pytorch import kernels as K

    lens = [200, 0, 312]
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    dist = torch.distributions.StudentT(3.0)
    torch.manual_seed(3)
    x = dist.sample((512, 256)).bfloat16().to(gpu)
    dy = dist.sample((512, 128)).bfloat16().to(gpu)
    exact = torch.stack([dy[a:b].float().T @ x[a:b].float() for a, b in ((0, 200), (200, 200), (200, 512))])

    def wgrad(signs):
        _, _, xq, xs = K.quantize_mx_impl(x, o.FMT_E2M1, rowwise=False, colwise=True, group_lens=gl, rht_signs=signs)
        _, _, dq, ds = K.quantize_mx_impl(dy, o.FMT_E2M1, rowwise=False, colwise=True, group_lens=gl, rht_signs=signs)
        return K.grouped_gemm_mx_wgrad_impl(dq, ds, xq, xs, gl, 512).float()

    plain, rht = wgrad(None), wgrad(0xA6C9)
    assert not rht[1].any()
    e_plain = (plain - exact).norm() / exact.norm()
    e_rht = (rht - exact).norm() / exact.norm()
    assert e_rht < 0.9 * e_plain and e_rht < 0.25, (e_rht.item(), e_plain.item())


def test_hadamard_bad_arguments(gpu):
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    x = torch.randn(64, 64, device=gpu).bfloat16()
    with pytest.raises(ValueError):
        K.quantize_mx_impl(x, o.FMT_E2M1, rowwise=True, colwise=False, rht_signs=1)
    with pytest.raises(ValueError):
        K.quantize_mx_impl(x, o.FMT_E4M3, rowwise=True, colwise=True, rht_signs=1)
    buf = torch.empty(64 * 64, dtype=torch.uint8, device=gpu)
    lib = _lib.load()
    assert lib.mxl_quantize_ex(x.data_ptr(), 64, 64, 64, _lib.FMT_E2M1, 0, None, 0, buf.data_ptr(), buf.data_ptr(), None, None,
                               _lib.QF_RHT_COL, 0, 1, None) == -1              # transform without a transposed copy
    assert lib.mxl_quantize_ex(x.data_ptr(), 64, 64, 64, _lib.FMT_E2M1, 0, None, 0, buf.data_ptr(), buf.data_ptr(), None, None,
                               64, 0, 0, None) == -1                            # unknown flag
    assert lib.mxl_quantize_ex(x.data_ptr(), 64, 64, 64, _lib.FMT_E2M1, 0, None, 0, buf.data_ptr(), buf.data_ptr(), None, None,
                               _lib.QF_KCHUNK, 0, 0, None) == -1                # chunk-major needs row_ld % 128 == 0


def test_grouped_gemm_fp4_with_hadamard_config(gpu):
    """Float4QuantConfig.colwise_rht_signs: forward and dgrad are untouched (row-wise copies), wgrad
    uses two transformed operands and stays the same quantity."""
    import primus_amd.pytorch as pt
    from primus_amd.pytorch.core import Float4QuantConfig

    torch.manual_seed(4)
    lens = [100, 0, 156]
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    x = torch.randn(256, 128, device=gpu).bfloat16()
    w = (torch.randn(3, 96, 128, device=gpu) * 0.05).bfloat16()
    dy = torch.randn(256, 96, device=gpu).bfloat16()

    def run(cfg):
        xx, ww = x.clone().requires_grad_(), w.clone().requires_grad_()
        y = pt.ops.grouped_gemm_fp4(xx, ww, gl, config=cfg)
        y.backward(dy)
        return y.detach(), xx.grad, ww.grad

    y0, dx0, dw0 = run(Float4QuantConfig())
    y1, dx1, dw1 = run(Float4QuantConfig(colwise_rht_signs=0x5A3C))
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1)
    assert not torch.equal(dw0, dw1) and not dw1[1].any()
    exact = torch.stack([dy[a:b].float().T @ x[a:b].float() for a, b in ((0, 100), (100, 100), (100, 256))])
    rel = lambda t: ((t.float() - exact).norm() / exact.norm()).item()   # noqa: E731
    assert rel(dw1) < 0.2 and abs(rel(dw1) - rel(dw0)) < 0.05
