"""MXFP4 linear of the "local" transformer spec: one dual quantisation op and
an autograd function that keeps the transposed copies for backward
(primus/backends/megatron/core/extensions/primus_turbo_mxfp4_local.py:
119-288 the op and the per-operand recipes, :291-461 the function).

Contract of the dual op for ``x [M, N]`` with both dims padded to 128
(:180-207): row-wise codes ``[M, N_pad/2]`` + scales ``[M, N_pad/32]``;
col-wise codes ``[N, M_pad/2]`` + scales ``[N, M_pad/32]`` -- the col-wise
copy is stored TRANSPOSED, ready to be the K-major operand of the next GEMM.

Per-operand recipes of the reference (:234-288): activations 1-D blocks,
weights 2-D 32x32 blocks, gradients 1-D blocks with optional stochastic
rounding; the col-wise copies of activations and gradients -- the two wgrad
operands -- go through a random Hadamard transform (16 tokens, the fixed sign
vector ``RHT_SIGNS``; orthogonal, so the contraction is unchanged).  The
pre-shuffled layouts and a transform of the row-wise copy have no kernels
here: the op raises for them.  Stochastic rounding draws its seeds from
``primus_amd.pytorch.kernels.next_sr_seed()``.
"""

from __future__ import annotations

from typing import Tuple

import torch

from ... import _lib
from ...pytorch import kernels as K
from ...pytorch.core.low_precision import ScalingGranularity, float4_e2m1fn_x2, float8_e8m0

MXFP4_BLOCK_SIZE = 32
MXFP4_PADDING_ALIGN_SIZE = 128
RHT_SIGNS = 0xA6C9   # sign vector of the Hadamard transform; any value works if both wgrad operands share it

_FP4_DTYPE = float4_e2m1fn_x2
_GRAN_VALUE = ScalingGranularity.MX_BLOCKWISE.value


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _unsupported(**flags) -> None:
    on = [name for name, value in flags.items() if value]
    if on:
        raise NotImplementedError(f"quantize_mxfp4_dual: no kernel for {', '.join(on)}")


def _quantize_mxfp4_dual_impl(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    padding_align_size: int,
    rowwise_use_2d_block: bool,
    rowwise_use_sr: bool,
    rowwise_use_rht: bool,
    colwise_use_2d_block: bool,
    colwise_use_sr: bool,
    colwise_use_rht: bool,
    shuffle_rowwise_scale: bool,
    shuffle_rowwise: bool,
    shuffle_colwise_scale: bool,
    shuffle_colwise: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """13 arguments, 4 outputs, like the reference's C++ op (:147-161)."""
    if out_dtype != _FP4_DTYPE:
        raise ValueError("quantize_mxfp4_dual produces float4_e2m1fn_x2")
    if padding_align_size != MXFP4_PADDING_ALIGN_SIZE:
        raise ValueError(f"padding_align_size must be {MXFP4_PADDING_ALIGN_SIZE}")
    if rowwise_use_2d_block != colwise_use_2d_block:
        raise NotImplementedError("2-D blocks apply to both copies of a weight or to neither")
    _unsupported(rowwise_use_rht=rowwise_use_rht, shuffle_rowwise_scale=shuffle_rowwise_scale,
                 shuffle_rowwise=shuffle_rowwise, shuffle_colwise_scale=shuffle_colwise_scale,
                 shuffle_colwise=shuffle_colwise)
    if x.dim() != 2:
        raise ValueError("quantize_mxfp4_dual expects a 2-D tensor")
    x = x.contiguous()
    rht = RHT_SIGNS if colwise_use_rht else None
    if rowwise_use_2d_block:
        if rowwise_use_sr or colwise_use_sr or colwise_use_rht:
            raise NotImplementedError("quantize_mxfp4_dual: stochastic rounding and the Hadamard transform "
                                      "exist for 1-D blocks only")
        return K.quantize_mx_weight_2d_impl(x, _lib.FMT_E2M1, rowwise=True, colwise=True,
                                            pad_to=MXFP4_PADDING_ALIGN_SIZE)
    if rowwise_use_sr == colwise_use_sr:
        return K.quantize_mx_impl(x, _lib.FMT_E2M1, rowwise=True, colwise=True, pad_to=MXFP4_PADDING_ALIGN_SIZE,
                                  sr_seed=K.next_sr_seed() if rowwise_use_sr else None, rht_signs=rht)
    # only one of the copies is rounded stochastically: one launch per copy
    q, s, _, _ = K.quantize_mx_impl(x, _lib.FMT_E2M1, rowwise=True, colwise=False, pad_to=MXFP4_PADDING_ALIGN_SIZE,
                                    sr_seed=K.next_sr_seed() if rowwise_use_sr else None)
    _, _, qt, st = K.quantize_mx_impl(x, _lib.FMT_E2M1, rowwise=False, colwise=True, pad_to=MXFP4_PADDING_ALIGN_SIZE,
                                      sr_seed=K.next_sr_seed() if colwise_use_sr else None, rht_signs=rht)
    return q, s, qt, st


def _quantize_mxfp4_dual_fake(
    x, out_dtype, padding_align_size, rowwise_use_2d_block, rowwise_use_sr, rowwise_use_rht, colwise_use_2d_block,
    colwise_use_sr, colwise_use_rht, shuffle_rowwise_scale, shuffle_rowwise, shuffle_colwise_scale, shuffle_colwise,
):
    """Output shapes and dtypes for tracing (:164-207)."""
    M, N = x.shape
    M_pad = _cdiv(M, MXFP4_PADDING_ALIGN_SIZE) * MXFP4_PADDING_ALIGN_SIZE
    N_pad = _cdiv(N, MXFP4_PADDING_ALIGN_SIZE) * MXFP4_PADDING_ALIGN_SIZE

    def scale_shape(rows, padded_other, shuffled):
        blocks = _cdiv(padded_other, MXFP4_BLOCK_SIZE)
        if shuffled:  # pre-shuffled scales: rows to 256, blocks to 8
            return _cdiv(rows, 256) * 256, _cdiv(blocks, 8) * 8
        return rows, blocks

    def u8(*shape):
        return torch.empty(*shape, dtype=torch.uint8, device=x.device)

    return (
        u8(M, N_pad // 2).view(_FP4_DTYPE),
        u8(*scale_shape(M, N_pad, shuffle_rowwise_scale)).view(float8_e8m0),
        u8(N, M_pad // 2).view(_FP4_DTYPE),
        u8(*scale_shape(N, M_pad, shuffle_colwise_scale)).view(float8_e8m0),
    )


# The op under two names: this package's own namespace and the one the reference's call sites use,
# torch.ops.primus_turbo_cpp_extension.quantize_mxfp4_dual (primus_turbo_mxfp4_local.py:147-161), so that
# code written against the reference's C++ extension finds it unchanged.
_quantize_mxfp4_dual_op = torch.library.custom_op(
    "primus_amd::quantize_mxfp4_dual", _quantize_mxfp4_dual_impl, mutates_args=(), device_types="cuda")
_quantize_mxfp4_dual_op.register_fake(_quantize_mxfp4_dual_fake)
try:
    _quantize_mxfp4_dual_ref_name = torch.library.custom_op(
        "primus_turbo_cpp_extension::quantize_mxfp4_dual", _quantize_mxfp4_dual_impl, mutates_args=(), device_types="cuda")
    _quantize_mxfp4_dual_ref_name.register_fake(_quantize_mxfp4_dual_fake)
except RuntimeError:   # the real extension is loaded in this process and owns the name
    _quantize_mxfp4_dual_ref_name = None


_quantize_mxfp4_dual_op.register_autograd(lambda ctx, *grads: (None,) * 13, setup_context=lambda ctx, inputs, output: None)


def _dual(x, two_d, sr, rht, shuffle):
    return _quantize_mxfp4_dual_op(
        x, _FP4_DTYPE, MXFP4_PADDING_ALIGN_SIZE,
        two_d, sr, False,          # row-wise copy: never transformed
        two_d, sr, rht,            # col-wise copy
        shuffle[0], shuffle[1], shuffle[2], shuffle[3],
    )


def _quantize_input_dual(input_2d, preshuffle: bool = False, use_rht: bool = True):
    """Activations: 1-D blocks (:234-250)."""
    return _dual(input_2d, False, False, use_rht, (preshuffle, False, preshuffle, preshuffle))


def _quantize_weight_dual(weight, preshuffle: bool = False):
    """Weights: 2-D 32x32 blocks, never transformed (:253-269)."""
    return _dual(weight, True, False, False, (preshuffle,) * 4)


def _quantize_grad_dual(grad_2d, preshuffle: bool = False, use_sr: bool = False, use_rht: bool = True):
    """Gradients: the activation recipe plus optional stochastic rounding (:272-288)."""
    return _dual(grad_2d, False, use_sr, use_rht, (preshuffle, False, preshuffle, False))


def _gemm_nt(a, a_scale, b, b_scale, out_dtype):
    return K.gemm_fp4_impl(a, a_scale, False, b, b_scale, True, out_dtype, False, granularity=_GRAN_VALUE,
                           default_backend=None, preshuffled=False)


class MXFP4LinearFunction(torch.autograd.Function):
    """``Y = X W^T`` with every operand in MXFP4 (:291-461, the pure-FP4 mode):

    fwd    Y  = Qrow(X) . Qrow(W)^T      and keep QcolT(X), QcolT(W)
    dgrad  dX = Qrow(dY) . QcolT(W)^T
    wgrad  dW = QcolT(dY) . QcolT(X)^T   (contraction over the padded token dim)
    """

    @staticmethod
    def forward(ctx, input, weight, use_gradient_sr=False):
        input_2d = input.reshape(-1, input.shape[-1])
        a, a_s, a_t, a_t_s = _quantize_input_dual(input_2d)
        b, b_s, b_t, b_t_s = _quantize_weight_dual(weight)
        out = _gemm_nt(a, a_s, b, b_s, input.dtype)
        ctx.save_for_backward(a_t, a_t_s, b_t, b_t_s)
        ctx.use_gradient_sr = use_gradient_sr
        ctx.out_dtype = input.dtype
        ctx.orig_shape = input.shape
        ctx.n_out, ctx.k_in = weight.shape
        return out[:, : weight.shape[0]].reshape(*input.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, grad_output):
        a_t, a_t_s, b_t, b_t_s = ctx.saved_tensors
        grad_2d = grad_output.contiguous().reshape(-1, grad_output.shape[-1])
        g, g_s, g_t, g_t_s = _quantize_grad_dual(grad_2d, use_sr=ctx.use_gradient_sr)
        grad_input = _gemm_nt(g, g_s, b_t, b_t_s, ctx.out_dtype)[:, : ctx.k_in].reshape(ctx.orig_shape)
        grad_weight = _gemm_nt(g_t, g_t_s, a_t, a_t_s, ctx.out_dtype)[: ctx.n_out, : ctx.k_in]
        return grad_input, grad_weight, None
