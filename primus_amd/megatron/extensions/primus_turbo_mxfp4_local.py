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
vector ``RHT_SIGNS``; orthogonal, so the contraction is unchanged).  A
transform of the row-wise copy has no kernel here: the op raises for it.
Stochastic rounding draws its seeds from
``primus_amd.pytorch.kernels.next_sr_seed()``.

Pre-shuffled layouts (the ``shuffle_*`` flags, :139-161; shapes :184-198): the
op permutes the bytes of the copies it is asked to shuffle after quantising
them (``kernels.shuffle_codes_impl`` / ``shuffle_scales_impl``), and
``gemm_fp4_impl(preshuffled=True)`` converts back in front of the GEMM, whose
kernels read the plain layouts: with this library the switch changes the bytes
that travel between the two calls and nothing else.

``MXFP4LinearFunction`` has the reference's calling convention (:291-461):
eight positional arguments, a tuple result whose first entry is the output, and
both modes -- FP4 backward on the transposed copies kept by the forward, or
(``backward_is_fp8``) backward on the saved bf16 tensors re-quantised to FP8
with one scale per tensor.
"""

from __future__ import annotations

from typing import Tuple

import torch

from ... import _lib
from ...pytorch import kernels as K
from ...pytorch.core.low_precision import ScalingGranularity, dtype_to_fmt_code, float4_e2m1fn_x2, float8_e5m2, float8_e8m0

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
    _unsupported(rowwise_use_rht=rowwise_use_rht)
    if x.dim() != 2:
        raise ValueError("quantize_mxfp4_dual expects a 2-D tensor")
    x = x.contiguous()
    q, s, qt, st = _quantize_plain(x, rowwise_use_2d_block, rowwise_use_sr, colwise_use_sr, colwise_use_rht)
    if shuffle_rowwise:
        q = K.shuffle_codes_impl(q)
    if shuffle_rowwise_scale:
        s = K.shuffle_scales_impl(s)
    if shuffle_colwise:
        qt = K.shuffle_codes_impl(qt)
    if shuffle_colwise_scale:
        st = K.shuffle_scales_impl(st)
    return q, s, qt, st


def _quantize_plain(x, use_2d_block, rowwise_use_sr, colwise_use_sr, colwise_use_rht):
    rht = RHT_SIGNS if colwise_use_rht else None
    if use_2d_block:
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


# The GEMMs of the function are custom ops too (the reference's gemm_fp4_impl / gemm_fp8_impl are ops of its C++
# extension): torch.compile then traces MXFP4LinearFunction without a graph break, which the reference tests
# (tests/unit_tests/backends/megatron/test_primus_turbo_mxfp4_local.py:202-287).
def _gemm_fp4_nt_impl(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor,
                      out_dtype: torch.dtype, preshuffled: bool) -> torch.Tensor:
    return K.gemm_fp4_impl(a, a_scale, False, b, b_scale, True, out_dtype, False, granularity=_GRAN_VALUE,
                           default_backend=None, preshuffled=preshuffled)


_gemm_fp4_nt_op = torch.library.custom_op("primus_amd::mxfp4_gemm_nt", _gemm_fp4_nt_impl, mutates_args=(), device_types="cuda")
_gemm_fp4_nt_op.register_fake(lambda a, a_scale, b, b_scale, out_dtype, preshuffled:
                              torch.empty((a.shape[0], b.shape[0]), dtype=out_dtype, device=a.device))


def _gemm_nt(a, a_scale, b, b_scale, out_dtype, preshuffle=False):
    return _gemm_fp4_nt_op(a, a_scale, b, b_scale, out_dtype, preshuffle)


def _fp8_tw_backward_op_impl(grad_2d: torch.Tensor, input_2d: torch.Tensor, weight: torch.Tensor,
                             fmt: int) -> Tuple[torch.Tensor, torch.Tensor]:
    dx, dw = _fp8_tw_backward(grad_2d, input_2d, weight, fmt)
    return dx.contiguous(), dw.contiguous()


_fp8_tw_backward_op = torch.library.custom_op("primus_amd::mxfp4_fp8_backward", _fp8_tw_backward_op_impl, mutates_args=(),
                                              device_types="cuda")
_fp8_tw_backward_op.register_fake(lambda grad_2d, input_2d, weight, fmt: (
    torch.empty((grad_2d.shape[0], weight.shape[1]), dtype=torch.bfloat16, device=grad_2d.device),
    torch.empty(tuple(weight.shape), dtype=torch.bfloat16, device=grad_2d.device)))


def _enable_preshuffle() -> bool:
    """The reference turns the pre-shuffled layouts on when its FP4 GEMM backend is pinned to AITER and autotuning is
    off (:61-74).  This library has one backend, which reads both layouts; the same environment switches are honoured
    so that a launch script written for the reference behaves the same way."""
    import os

    pinned = "FP4:AITER" in os.environ.get("PRIMUS_TURBO_GEMM_BACKEND", "").upper().replace(" ", "")
    return pinned and not os.environ.get("PRIMUS_TURBO_AUTO_TUNE")


def _assert_preshuffle_contract(config, preshuffle: bool) -> None:
    """The reference refuses MXFP4 without its pre-shuffle fast path, because its other backends would misread
    shuffled bytes or pay extra shuffle passes (:77-105).  Neither can happen here (the flag travels with every
    call and the GEMM converts what it is told is shuffled), so there is nothing to refuse."""
    return None


def _fp8_tw_backward(grad_2d, input_2d, weight, fmt):
    """The backward of the hybrid mode (:391-428): dY, X and W re-quantised to FP8 with one scale per tensor
    (``_quantize_fp8_tw``), dX = dY . W and dW = dY^T . X as NT GEMMs on the transposed copies."""
    n, k = weight.shape
    if n % K.BLOCK or k % K.BLOCK:
        raise ValueError(f"the FP8 backward needs weight dims that are multiples of {K.BLOCK} (got {n} x {k})")
    m = grad_2d.shape[0]
    kc = K.pick_layout(1, n, k, m, fp8=True)
    d_row, d_ru, d_col, d_cu, d_si = K.quantize_tensorwise_impl(grad_2d, fmt, rowwise=True, colwise=True,
                                                               pad_to=K.GEMM_K_ALIGN, kchunk=kc)
    _, _, x_col, x_cu, x_si = K.quantize_tensorwise_impl(input_2d.contiguous(), fmt, rowwise=False, colwise=True,
                                                         pad_to=K.GEMM_K_ALIGN, kchunk=kc)
    _, _, w_col, w_cu, w_si = K.quantize_weight_tensorwise_impl(weight.contiguous(), fmt, rowwise=False, colwise=True,
                                                                pad_to=K.GEMM_K_ALIGN, kchunk=kc)
    grad_input = K.gemm_tw_nt_impl(d_row, d_ru, d_si, w_col, w_cu, w_si, None, kchunk=kc)
    grad_weight = K.gemm_tw_wgrad_impl(d_col, d_cu, d_si, x_col, x_cu, x_si, None, m, kchunk=kc)
    return grad_input[:, :k], grad_weight[:n, :k]


class MXFP4LinearFunction(torch.autograd.Function):
    """``Y = X W^T`` with MXFP4 operands (:291-461), two modes:

    pure MXFP4 (``backward_is_fp8`` False)
        fwd    Y  = Qrow(X) . Qrow(W)^T      and keep QcolT(X), QcolT(W)
        dgrad  dX = Qrow(dY) . QcolT(W)^T
        wgrad  dW = QcolT(dY) . QcolT(X)^T   (contraction over the padded token dim)
    hybrid (``backward_is_fp8`` True)
        the same forward; the backward re-quantises the saved bf16 X, W and dY to ``fp8_bwd_dtype`` with one scale
        per tensor.

    Called like the reference's: ``apply(input, weight, preshuffle, backward_is_fp8, fp8_bwd_dtype, fp8_gran_value,
    fp8_backend_value, use_gradient_sr)[0]``; the further entries of the result are the tensors kept for backward.
    ``fp8_gran_value`` must name tensor-wise scaling (the only value the reference passes); the backend value is
    accepted and unused.
    """

    @staticmethod
    def forward(input, weight, preshuffle, backward_is_fp8, fp8_bwd_dtype, fp8_gran_value, fp8_backend_value, use_gradient_sr):
        if backward_is_fp8 and fp8_gran_value != ScalingGranularity.TENSORWISE.value:
            raise ValueError("the FP8 backward of the MXFP4 linear uses tensor-wise scaling")
        input_2d = input.reshape(-1, input.shape[-1])
        if input_2d.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise ValueError("MXFP4LinearFunction expects bfloat16 operands")
        a, a_s, a_t, a_t_s = _quantize_input_dual(input_2d, preshuffle)
        b, b_s, b_t, b_t_s = _quantize_weight_dual(weight, preshuffle)
        out = _gemm_nt(a, a_s, b, b_s, input.dtype, preshuffle)
        out = out[:, : weight.shape[0]].reshape(*input.shape[:-1], weight.shape[0])
        if backward_is_fp8:
            return out, input_2d.view_as(input_2d), weight.view_as(weight)
        # the kept copies leave as uint8 views: autograd cannot make zero gradients of the FP4 / E8M0 dtypes
        return out, a_t.view(torch.uint8), a_t_s.view(torch.uint8), b_t.view(torch.uint8), b_t_s.view(torch.uint8)

    @staticmethod
    def setup_context(ctx, inputs, output):
        input, weight, preshuffle, backward_is_fp8, fp8_bwd_dtype, _, _, use_gradient_sr = inputs
        ctx.preshuffle = preshuffle
        ctx.backward_is_fp8 = backward_is_fp8
        ctx.use_gradient_sr = use_gradient_sr
        ctx.out_dtype = input.dtype
        ctx.orig_shape = input.shape
        ctx.n_out, ctx.k_in = weight.shape
        if backward_is_fp8:
            ctx.fp8_fmt = dtype_to_fmt_code(fp8_bwd_dtype)
            ctx.save_for_backward(output[1], output[2])
        else:
            ctx.save_for_backward(*output[1:])
            ctx.mark_non_differentiable(*output[1:])

    @staticmethod
    def backward(ctx, grad_output, *_):
        grad_2d = grad_output.contiguous().reshape(-1, grad_output.shape[-1])
        if grad_2d.dtype != torch.bfloat16:
            grad_2d = grad_2d.to(torch.bfloat16)
        if ctx.backward_is_fp8:
            input_2d, weight = ctx.saved_tensors
            grad_input, grad_weight = _fp8_tw_backward_op(grad_2d, input_2d.detach().contiguous(), weight.detach().contiguous(),
                                                          ctx.fp8_fmt)
            return (grad_input.reshape(ctx.orig_shape), grad_weight) + (None,) * 6
        a_t, a_t_s, b_t, b_t_s = ctx.saved_tensors
        a_t, b_t = a_t.view(_FP4_DTYPE), b_t.view(_FP4_DTYPE)
        a_t_s, b_t_s = a_t_s.view(float8_e8m0), b_t_s.view(float8_e8m0)
        pre = ctx.preshuffle
        g, g_s, g_t, g_t_s = _quantize_grad_dual(grad_2d, pre, use_sr=ctx.use_gradient_sr)
        grad_input = _gemm_nt(g, g_s, b_t, b_t_s, ctx.out_dtype, pre)[:, : ctx.k_in].reshape(ctx.orig_shape)
        grad_weight = _gemm_nt(g_t, g_t_s, a_t, a_t_s, ctx.out_dtype, pre)[: ctx.n_out, : ctx.k_in]
        return (grad_input, grad_weight) + (None,) * 6


def mxfp4_linear(input, weight, preshuffle: bool = False, backward_precision: str = "mxfp4",
                 use_gradient_sr: bool = False):
    """``MXFP4LinearFunction`` with the arguments the reference's parallel linears derive from their config
    (:476-511): ``backward_precision`` "mxfp4" or "fp8" (``mxfp4_backward_precision``; FP8 means E5M2 codes, one
    scale per tensor), ``use_gradient_sr`` (``mxfp4_gradient_stochastic_rounding``).  Returns the output only."""
    if backward_precision not in ("mxfp4", "fp8"):
        raise ValueError("backward_precision must be 'mxfp4' or 'fp8'")
    fp8 = backward_precision == "fp8"
    return MXFP4LinearFunction.apply(input, weight, preshuffle, fp8, float8_e5m2 if fp8 else None,
                                     ScalingGranularity.TENSORWISE.value if fp8 else 0, 0, use_gradient_sr)[0]
