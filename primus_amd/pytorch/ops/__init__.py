"""Differentiable operators of the MX linear path.

Same entry points and argument meaning as the operators the reference's
Megatron modules call:

* ``gemm_fp8`` / ``gemm_fp4``: primus/backends/megatron/core/extensions/
  primus_turbo.py:1095-1103, :1142-1150 (and indexer.py:166,208 positional use)
* ``grouped_gemm_fp8`` / ``grouped_gemm_fp4``: primus_turbo.py:2122-2129,
  :2171-2178; keyword ``group_lens=`` at
  primus/backends/torchtitan/models/moe/moe.py:38-48

Operand flow per GEMM (primus_turbo_mxfp4_local.py:316-331 fwd, :432-444
dgrad, :447-459 wgrad): every GEMM is NT with both operands quantised along
its contraction dim --
  fwd   Y[M,N]  = Qrow(X)[M,K]   . Qrow(W)[N,K]^T
  dgrad dX[M,K] = Qrow(dY)[M,N]  . QcolT(W)[K,N]^T
  wgrad dW[N,K] = QcolT(dY)[N,M] . QcolT(X)[K,M]^T   (M ragged per expert)
Activations and gradients use 1-D blocks of 32, weights 2-D 32x32 blocks.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from ... import _lib
from .. import kernels as K
from ..core.low_precision import (
    Float4QuantConfig,
    Float8QuantConfig,
    Format,
    ScalingGranularity,
    fmt_code,
)
from ..core.quantized_tensor import QuantizedTensor, QuantizedTensorPair

__all__ = ["gemm", "grouped_gemm", "gemm_fp8", "gemm_fp4", "grouped_gemm_fp8", "grouped_gemm_fp4", "set_wgrad_overlap",
           "set_dgrad_reads_rowwise_weight",
           "swiglu_with_probs", "geglu_with_probs", "tokens_per_expert_to_mask", "glu_grouped_gemm_fp8",
           "glu_grouped_gemm_fp4", "manual_sr_seed", "set_kchunk_layout", "rmsnorm", "rmsnorm_gemm_fp8", "rmsnorm_gemm_fp4", "pad_groups", "unpad_groups"]

# dgrad and wgrad of one linear are independent once dY is quantised.  Both GEMMs are persistent
# kernels with one workgroup per CU, so launching wgrad on a second stream lets its workgroups move in
# as dgrad's last, partial wave of tiles drains instead of leaving those CUs idle.
_wgrad_overlap = True
_side_streams = {}


def manual_sr_seed(seed: Optional[int]) -> None:
    """Restart the seed sequence of stochastic gradient rounding (``Float4QuantConfig.use_gradient_sr``);
    ``None`` ties it to ``torch.initial_seed()`` again."""
    K.manual_sr_seed(seed)


def set_kchunk_layout(enabled: bool) -> None:
    """Store quantised operands K-chunk-major between the quantisers and the GEMMs (default on; the
    row-major layout gives the same results bit for bit and is what operands of 4 GiB or more use)."""
    K.set_kchunk_default(enabled)


_dgrad_reads_rowwise = True


def set_dgrad_reads_rowwise_weight(enabled: bool) -> None:
    """Whether the MXFP8 operators let dgrad read the row-wise weight codes transposed instead of writing a
    transposed copy of the codes in the forward (default on; same results bit for bit)."""
    global _dgrad_reads_rowwise
    _dgrad_reads_rowwise = bool(enabled)


def set_wgrad_overlap(enabled: bool) -> None:
    """Run wgrad on a side stream next to dgrad (default on)."""
    global _wgrad_overlap
    _wgrad_overlap = bool(enabled)


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    key = (device.type, device.index)
    st = _side_streams.get(key)
    if st is None:
        st = torch.cuda.Stream(device=device)   # default priority
        _side_streams[key] = st
    return st


_dummy_wgrads = {}


def _finish_wgrad(grad_b, accum, fused: bool, w_shape):
    """Gradient-accumulation fusion (``fuse_bgrad_accum_pattern="megatron"``): the weight gradient belongs in
    the float32 ``main_grad`` of the operand.  ``fused``: the GEMM has added it already; otherwise it is added
    here.  Either way the operand's ``grad_added_to_main_grad`` is set and autograd gets a placeholder of the
    weight's shape, whose only purpose is to make the parameter's gradient hooks fire
    (primus/backends/megatron/core/extensions/primus_turbo.py:141-163, 166-240)."""
    if accum is None:
        return grad_b.view(w_shape)
    target, owner = accum
    if not fused:
        target.add_(grad_b.view(w_shape))
    owner.grad_added_to_main_grad = True
    dtype = getattr(owner, "dtype", torch.bfloat16)
    key = (tuple(w_shape), dtype, target.device)
    dummy = _dummy_wgrads.get(key)
    if dummy is None:
        dummy = torch.empty(tuple(w_shape), dtype=dtype, device=target.device)
        _dummy_wgrads[key] = dummy
    return dummy


def _accum_from(b, pattern):
    """``(main_grad, operand)`` for ``fuse_bgrad_accum_pattern="megatron"``, else None."""
    if pattern is None:
        return None
    if pattern != "megatron":
        raise ValueError(f"unknown fuse_bgrad_accum_pattern {pattern!r} (the reference passes 'megatron' or None)")
    main_grad = getattr(b, "main_grad", None)
    if main_grad is None or not hasattr(b, "grad_added_to_main_grad"):
        raise ValueError("fuse_bgrad_accum_pattern='megatron' needs main_grad and grad_added_to_main_grad on the weight operand")
    if tuple(main_grad.shape) != tuple(b.shape):
        raise ValueError("main_grad must have the weight's shape")
    # any dtype is accepted, as by the reference's bridge (primus_turbo.py:166-240); only a contiguous float32
    # buffer can be the target of the GEMM's own accumulating epilogue, anything else is added to after the GEMM
    return main_grad, b


def _fusable(target) -> bool:
    return target is not None and target.dtype == torch.float32 and target.is_contiguous()


def _cached_codes(q: QuantizedTensor, kchunk) -> torch.Tensor:
    """Codes of a cached weight copy in the layout this call's GEMMs use.  A chunked cache is
    rearranged (one pass over the weight) only when this call cannot use that layout."""
    if int(q.kchunk) == int(kchunk) or (int(q.kchunk) == K.LAYOUT_KSTEP128 and int(kchunk) == K.LAYOUT_KCHUNK):
        return q.codes          # the 128-element step layout stores its codes K-chunk-major
    return q.rowmajor_codes()


def _cached_scales(q: QuantizedTensor, kchunk) -> torch.Tensor:
    return q.scales if int(q.kchunk) == int(kchunk) else q.rowmajor_scales()


def _cache_layout(b: QuantizedTensor, b_t, kc: int, fp8: bool, groups: int, fp4: bool = False) -> int:
    """Layout of a call on cached weight copies: the cache's own, row-major when the pair disagrees or
    this call cannot read that layout."""
    lay = int(b.kchunk) if (b_t is None or int(b_t.kchunk) == int(b.kchunk)) else 0
    if lay == K.LAYOUT_KSTEP and not (fp8 and groups <= K.RING_MAX_GROUPS):
        lay = 0
    if lay == K.LAYOUT_KSTEP128 and not (fp4 and groups <= K.RING_MAX_GROUPS):
        lay = K.LAYOUT_KCHUNK   # same codes; the scales are rearranged (1/16 of the bytes of the codes)
    return lay if kc else 0


class _MXLinearFunction(torch.autograd.Function):
    """Y = X . W^T on MX operands, dense (``group_lens is None``) or grouped.

    With ``activation`` set, ``a`` is the previous linear's output ``[tokens, 2F]`` and
    X = act(a[:, :F]) * a[:, F:] * probs (masked rows zero) is formed inside the quantiser: X itself
    never reaches memory, in the forward or in the backward."""

    @staticmethod
    def forward(ctx, a, b, b_t, group_lens, act_fmt, w_fmt, scale_mode, probs=None, row_mask=None, activation=None,
                grad_sr=False, rht_signs=None, norm_weight=None, norm_eps=0.0, accum=None):
        glu = activation is not None
        norm = norm_weight is not None
        need_dgrad = a.requires_grad or (glu and probs.requires_grad) or (norm and norm_weight.requires_grad)
        need_wgrad = b.requires_grad
        grouped = group_lens is not None
        # Every operand of the three GEMMs is stored in one layout, K-chunk-major unless an operand is
        # too large for it (or the layout is switched off): same codes, same results, faster loads.
        groups = b.shape[0] if grouped else 1
        # K-step-major operands (the ring kernel) whenever the activations are FP8: against FP8 weights in all three
        # GEMMs, against E2M1 weights in forward and dgrad (wgrad is FP8 x FP8 then)
        fp8 = act_fmt != _lib.FMT_E2M1
        # E2M1 x E2M1 runs on the ring kernel too, in steps of 128 elements (two MFMAs per step)
        fp4 = act_fmt == _lib.FMT_E2M1 and w_fmt == _lib.FMT_E2M1
        kc = K.pick_layout(groups, b.shape[-2], b.shape[-1], a.shape[0], fp8=fp8, fp4=fp4)
        if isinstance(b, QuantizedTensor):   # cached copies decide: the call uses the layout they are stored in
            kc = _cache_layout(b, b_t, kc, fp8, groups, fp4)
        # (a weight gradient that is added to a float32 buffer inside the GEMM runs on either chunked layout)
        # activations: row-wise for the forward GEMM, transposed col-wise kept for wgrad
        # (row-wise copies are padded to the GEMM's K granularity, like the reference pads its
        # MXFP4 operands to 128: primus_turbo_mxfp4_local.py:119-124)
        if glu:
            a_row, a_rs, a_col, a_cs = K.glu_with_probs_quantize_impl(
                a, probs, row_mask, activation, act_fmt, scale_mode, colwise=need_wgrad, group_lens=group_lens,
                pad_to=K.GEMM_K_ALIGN, kchunk=kc,
            )
        elif norm:
            # X = rmsnorm(a) is formed inside the quantiser from a, the norm weight and the row statistics
            _, rstd = K.rmsnorm_fwd_impl(a, norm_weight.detach(), norm_eps, want_y=False)
            a_row, a_rs, a_col, a_cs = K.rmsnorm_quantize_impl(
                a, norm_weight.detach(), rstd, act_fmt, scale_mode, colwise=need_wgrad, pad_to=K.GEMM_K_ALIGN, kchunk=kc,
            )
        else:
            a_row, a_rs, a_col, a_cs = K.quantize_mx_impl(
                a, act_fmt, scale_mode, rowwise=True, colwise=need_wgrad, group_lens=group_lens, pad_to=K.GEMM_K_ALIGN,
                rht_signs=rht_signs if need_wgrad else None, kchunk=kc,
            )
        if isinstance(b, QuantizedTensor):
            # cached weight copies (primus_turbo.py:1105-1115): nothing to quantise here
            if b.axis != -1:
                raise ValueError("the forward weight copy must be quantised along axis=-1")
            if b.tensor_scale_inv is not None:
                raise ValueError("the cached weight copy is tensor-wise scaled, the operator's config is an MX recipe")
            w_row, w_rs = _cached_codes(b, kc), _cached_scales(b, kc)
            w_col = w_cs = None
            if need_dgrad:
                if b_t is None:
                    raise ValueError("dgrad needs the transposed weight copy (QuantizedTensorPair.data_t)")
                if b_t.axis != -2:
                    raise ValueError("QuantizedTensorPair.data_t must be quantised along axis=-2")
                w_col, w_cs = _cached_codes(b_t, kc), _cached_scales(b_t, kc)
        else:
            # FP8 weights on the ring kernel: dgrad reads the ROW-WISE codes transposed (2-D blocks: the transposed
            # copy is the same codes transposed), so only that copy's scales are written next to the row-wise copy
            # (the same for E2M1 weights against E2M1 rows in 128-element steps, through the 4-bit transposing read)
            bt = (need_dgrad and _dgrad_reads_rowwise and b.shape[-2] % K.GEMM_K_ALIGN == 0 and b.shape[-1] % K.GEMM_K_ALIGN == 0
                  and ((kc == K.LAYOUT_KSTEP and w_fmt == _lib.FMT_E4M3 and act_fmt == _lib.FMT_E4M3)
                       or (kc == K.LAYOUT_KSTEP128 and w_fmt == _lib.FMT_E2M1 and act_fmt == _lib.FMT_E2M1)))
            w_row, w_rs, w_col, w_cs = K.quantize_mx_weight_2d_impl(
                b.detach(), w_fmt, scale_mode, rowwise=True, colwise=need_dgrad, pad_to=K.GEMM_K_ALIGN, kchunk=kc,
                col_scales_only=bt,
            )
            if bt:
                w_col = w_row
        if grouped:
            y = K.grouped_gemm_mx_nt_impl(a_row, a_rs, w_row, w_rs, group_lens, kchunk=kc)
        else:
            y = K.gemm_mx_nt_impl(a_row, a_rs, w_row, w_rs, kchunk=kc)
        if glu and need_dgrad:
            ctx.save_for_backward(a_col, a_cs, w_col, w_cs, group_lens, a, probs, row_mask)
        elif norm and need_dgrad:
            ctx.save_for_backward(a_col, a_cs, w_col, w_cs, group_lens, a, norm_weight.detach(), rstd)
        else:
            ctx.save_for_backward(a_col, a_cs, w_col, w_cs, group_lens)
        ctx.cfg = (act_fmt, scale_mode, a.shape[0], need_dgrad, need_wgrad, tuple(b.shape))
        ctx.activation = activation
        ctx.grad_sr = bool(grad_sr) and act_fmt == _lib.FMT_E2M1
        ctx.rht_signs = rht_signs
        ctx.kchunk = kc
        ctx.b_transposed = (not isinstance(b, QuantizedTensor)) and bt
        ctx.norm = norm
        ctx.accum = accum      # (float32 buffer the weight gradient is added to, object that gets the flag) or None
        return y

    @staticmethod
    def backward(ctx, dy):
        a_col, a_cs, w_col, w_cs, group_lens = ctx.saved_tensors[:5]
        act_fmt, scale_mode, total_m, need_dgrad, need_wgrad, w_shape = ctx.cfg
        grouped = group_lens is not None
        dy = dy.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        # gradients of the MXFP4 recipe may be rounded stochastically (primus_turbo_mxfp4_local.py:272-288)
        d_row, d_rs, d_col, d_cs = K.quantize_mx_impl(
            dy, act_fmt, scale_mode, rowwise=need_dgrad, colwise=need_wgrad, group_lens=group_lens, pad_to=K.GEMM_K_ALIGN,
            sr_seed=K.next_sr_seed() if ctx.grad_sr else None,
            rht_signs=ctx.rht_signs if need_wgrad else None,   # same signs as the saved activation copy
            kchunk=ctx.kchunk,
        )
        kc = ctx.kchunk
        grad_a = grad_b = None
        overlap = _wgrad_overlap and need_dgrad and need_wgrad
        if overlap:
            main = torch.cuda.current_stream(dy.device)
            side = _side_stream(dy.device)
            side.wait_stream(main)   # the quantised operands are ready
        if need_dgrad:
            if grouped:
                grad_a = K.grouped_gemm_mx_nt_impl(d_row, d_rs, w_col, w_cs, group_lens, kchunk=kc, b_transposed=ctx.b_transposed)
            else:
                grad_a = K.gemm_mx_nt_impl(d_row, d_rs, w_col, w_cs, kchunk=kc, b_transposed=ctx.b_transposed)
        if need_wgrad:
            target = ctx.accum[0] if ctx.accum is not None else None
            fused = _fusable(target) and kc != K.LAYOUT_ROWMAJOR   # the GEMM's epilogue adds into the float32 buffer

            def wgrad():
                return K.grouped_gemm_mx_wgrad_impl(d_col, d_cs, a_col, a_cs, group_lens, total_m, kchunk=kc,
                                                    accum_into=target if fused else None)

            if overlap:
                with torch.cuda.stream(side):
                    grad_b = wgrad()
                for t in (d_col, d_cs, a_col, a_cs, grad_b):
                    t.record_stream(side)
                grad_b.record_stream(main)
                main.wait_stream(side)
            else:
                grad_b = wgrad()
            grad_b = _finish_wgrad(grad_b, ctx.accum, fused, w_shape)
        grad_p = None
        if ctx.activation is not None and need_dgrad:
            # grad_a so far is dL/dX; take it through the activation to fc1's output and the probabilities
            pre, probs, row_mask = ctx.saved_tensors[5:8]
            grad_a, grad_p = K.glu_with_probs_bwd_impl(grad_a, pre, probs, row_mask, ctx.activation)
            grad_p = grad_p.to(probs.dtype)
        grad_nw = None
        if ctx.norm and need_dgrad:
            # grad_a so far is dL/dX for X = rmsnorm(a); take it through the normalisation
            pre, nw, rstd = ctx.saved_tensors[5:8]
            grad_a, grad_nw = K.rmsnorm_bwd_impl(grad_a, pre, nw, rstd)
        return grad_a, grad_b, None, None, None, None, None, grad_p, None, None, None, None, grad_nw, None, None


def _transposed_cache(q: QuantizedTensor, kchunk: bool):
    """Transposed copy (codes, unit scales) of a tensor-wise scaled weight cache that holds the row-wise copy
    only (the reference keeps no transposed cache under current scaling, primus_turbo.py:1105-1115: its
    dgrad GEMM reads the same codes in NN layout).  The scale belongs to the whole tensor, so transposing
    the codes is all there is to do: one pass over the weight's bytes per call."""
    codes = q.rowmajor_codes()
    k = q.shape[-1]
    t = codes[..., :k].transpose(-1, -2)                       # [..., k, n]
    n = t.shape[-1]
    n_ld = (n + K.GEMM_K_ALIGN - 1) // K.GEMM_K_ALIGN * K.GEMM_K_ALIGN
    out = torch.zeros(tuple(t.shape[:-1]) + (n_ld,), dtype=torch.uint8, device=codes.device)
    out[..., :n] = t.view(torch.uint8)
    unit = torch.full(tuple(t.shape[:-1]) + (n_ld // _lib.BLOCK,), 127, dtype=torch.uint8, device=codes.device)
    if kchunk:
        # K-chunk-major or K-step-major: [n_ld / step][rows][step]
        step = K.KSTEP if int(kchunk) == K.LAYOUT_KSTEP else K.KCHUNK
        rows = out.numel() // n_ld
        laid = torch.empty((n_ld // step, rows, step), dtype=torch.uint8, device=codes.device)
        laid.copy_(out.reshape(rows, n_ld // step, step).permute(1, 0, 2))
        out = laid
        if int(kchunk) == K.LAYOUT_KSTEP:
            unit = torch.empty(K._scale_shape(rows, n_ld, kchunk), dtype=torch.uint8, device=codes.device).fill_(127)
    return out.view(codes.dtype), unit.view(q.scales.dtype)


class _TWLinearFunction(torch.autograd.Function):
    """Y = X . W^T on tensor-wise scaled FP8 operands (one float32 scale per tensor, computed from the
    tensor's abs-max at every call: "current" scaling), dense or grouped.  Operand flow of the reference's
    tensor-wise linear (primus_turbo_float8_local.py:215-306): X and W in the forward format, dY in the
    backward format (E5M2 for Format.HYBRID); here every GEMM is NT, so the quantisers also write the
    transposed copies that dgrad and wgrad read."""

    @staticmethod
    def forward(ctx, a, b, b_t, group_lens, fwd_fmt, bwd_fmt, accum=None):
        need_dgrad = a.requires_grad
        need_wgrad = b.requires_grad
        grouped = group_lens is not None
        groups = b.shape[0] if grouped else 1
        if isinstance(b, QuantizedTensor):
            # cached copies decide: the call uses the layout they are stored in, row-major when it cannot
            kc = int(b.kchunk) if (b_t is None or int(b_t.kchunk) == int(b.kchunk)) else 0
            if not (K.kchunk_default() and K.kchunk_fits(groups, b.shape[-2], b.shape[-1], a.shape[0])):
                kc = 0
            if kc == K.LAYOUT_KSTEP and groups > K.RING_MAX_GROUPS:
                kc = 0          # the ring kernel does not take more groups
            if kc == K.LAYOUT_KSTEP128:
                kc = 0
        else:
            kc = K.pick_layout(groups, b.shape[-2], b.shape[-1], a.shape[0], fp8=True)
        a_row, a_ru, a_col, a_cu, a_si = K.quantize_tensorwise_impl(
            a, fwd_fmt, rowwise=True, colwise=need_wgrad, group_lens=group_lens, pad_to=K.GEMM_K_ALIGN, kchunk=kc)
        if isinstance(b, QuantizedTensor):
            if b.axis != -1 or b.tensor_scale_inv is None:
                raise ValueError("the forward weight copy must be a tensor-wise scaled copy quantised along axis=-1")
            w_row, w_ru, w_si = _cached_codes(b, kc), _cached_scales(b, kc), b.tensor_scale_inv
            w_col = w_cu = None
            bt = False
            if need_dgrad:
                if b_t is not None:
                    w_col, w_cu = _cached_codes(b_t, kc), _cached_scales(b_t, kc)
                else:
                    w_col, w_cu = _transposed_cache(b, kc)
        else:
            # one scale per tensor: the transposed copy would be the row-wise codes transposed, so on the ring kernel
            # dgrad reads the row-wise codes through its transposing LDS reads and no second copy is written
            bt = (need_dgrad and _dgrad_reads_rowwise and kc == K.LAYOUT_KSTEP and fwd_fmt == _lib.FMT_E4M3
                  and b.shape[-2] % K.GEMM_K_ALIGN == 0 and b.shape[-1] % K.GEMM_K_ALIGN == 0)
            w_row, w_ru, w_col, w_cu, w_si = K.quantize_weight_tensorwise_impl(
                b.detach(), fwd_fmt, rowwise=True, colwise=need_dgrad and not bt, pad_to=K.GEMM_K_ALIGN, kchunk=kc)
            if bt:
                w_col, w_cu = w_row, w_ru
        y = K.gemm_tw_nt_impl(a_row, a_ru, a_si, w_row, w_ru, w_si, group_lens, kchunk=kc)
        ctx.save_for_backward(a_col, a_cu, a_si, w_col, w_cu, w_si, group_lens)
        ctx.cfg = (bwd_fmt, a.shape[0], need_dgrad, need_wgrad, tuple(b.shape), kc)
        ctx.b_transposed = bt
        ctx.accum = accum
        return y

    @staticmethod
    def backward(ctx, dy):
        a_col, a_cu, a_si, w_col, w_cu, w_si, group_lens = ctx.saved_tensors
        bwd_fmt, total_m, need_dgrad, need_wgrad, w_shape, kc = ctx.cfg
        dy = dy.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        d_row, d_ru, d_col, d_cu, d_si = K.quantize_tensorwise_impl(
            dy, bwd_fmt, rowwise=need_dgrad, colwise=need_wgrad, group_lens=group_lens, pad_to=K.GEMM_K_ALIGN, kchunk=kc)
        grad_a = grad_b = None
        overlap = _wgrad_overlap and need_dgrad and need_wgrad
        if overlap:
            main = torch.cuda.current_stream(dy.device)
            side = _side_stream(dy.device)
            side.wait_stream(main)
        if need_dgrad:
            grad_a = K.gemm_tw_nt_impl(d_row, d_ru, d_si, w_col, w_cu, w_si, group_lens, kchunk=kc,
                                       b_transposed_n=w_shape[-1] if ctx.b_transposed else None)
        if need_wgrad:
            target = ctx.accum[0] if ctx.accum is not None else None
            fused = _fusable(target) and kc != K.LAYOUT_ROWMAJOR

            def wgrad():
                return K.gemm_tw_wgrad_impl(d_col, d_cu, d_si, a_col, a_cu, a_si, group_lens, total_m, kchunk=kc,
                                            accum_into=target if fused else None)

            if overlap:
                with torch.cuda.stream(side):
                    grad_b = wgrad()
                for t in (d_col, d_cu, d_si, a_col, a_cu, a_si, grad_b):
                    t.record_stream(side)
                grad_b.record_stream(main)
                main.wait_stream(side)
            else:
                grad_b = wgrad()
            grad_b = _finish_wgrad(grad_b, ctx.accum, fused, w_shape)
        return grad_a, grad_b, None, None, None, None, None


class _BWLinearFunction(torch.autograd.Function):
    """Y = X . W^T under the 128-blockwise FP8 recipe, dense (FP8LinearBlockwiseFunction,
    primus_turbo_float8_local.py:993-1089) or grouped (zbpp_gemm.py:590-640, :757-800): X in 1 x 128 blocks, W in
    128 x 128 blocks, forward format; like the reference the backward starts from the bf16 tensors again and quantises
    dY (both axes), X (along the tokens, blocks restarting at every group) and W in the backward format (E5M2 for
    Format.HYBRID).  Every GEMM is NT on the transposed copies the quantisers write."""

    @staticmethod
    def forward(ctx, a, b, group_lens, fwd_fmt, bwd_fmt, accum=None):
        a_row, a_s, _, _ = K.quantize_blockwise_impl(a, fwd_fmt, rowwise=True, colwise=False)
        w_row, w_s, _, _ = K.quantize_blockwise_weight_impl(b.detach(), fwd_fmt, rowwise=True, colwise=False)
        y = K.gemm_blockwise_nt_impl(a_row, a_s, w_row, w_s, group_lens, b_rows_per_scale=None if group_lens is not None else 128)
        ctx.save_for_backward(a, b, group_lens)
        ctx.cfg = (bwd_fmt, a.requires_grad, b.requires_grad)
        ctx.accum = accum
        return y

    @staticmethod
    def backward(ctx, dy):
        a, b, group_lens = ctx.saved_tensors
        bwd_fmt, need_dgrad, need_wgrad = ctx.cfg
        dy = dy.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        d_row, d_s, d_col, d_cs = K.quantize_blockwise_impl(dy, bwd_fmt, rowwise=need_dgrad, colwise=need_wgrad,
                                                            group_lens=group_lens)
        grad_a = grad_b = None
        if need_dgrad:
            _, _, w_col, w_cs = K.quantize_blockwise_weight_impl(b.detach(), bwd_fmt, rowwise=False, colwise=True)
            grad_a = K.gemm_blockwise_nt_impl(d_row, d_s, w_col, w_cs, group_lens, b_rows_per_scale=None if group_lens is not None else 128)
        if need_wgrad:
            _, _, a_col, a_cs = K.quantize_blockwise_impl(a.detach(), bwd_fmt, rowwise=False, colwise=True, group_lens=group_lens)
            if group_lens is None:
                grad_b = K.gemm_blockwise_nt_impl(d_col, d_cs, a_col, a_cs, b_rows_per_scale=1)
            else:
                grad_b = K.grouped_gemm_blockwise_wgrad_impl(d_col, d_cs, a_col, a_cs, group_lens, a.shape[0])
            grad_b = _finish_wgrad(grad_b, ctx.accum, False, tuple(b.shape))
        return grad_a, grad_b, None, None, None, None


def _tensorwise_formats(config):
    """(forward, backward) code formats of the tensor-wise recipe (_get_fp8_dtype,
    primus_turbo_float8_local.py:146-154)."""
    if config.format == Format.E4M3:
        return _lib.FMT_E4M3, _lib.FMT_E4M3
    if config.format == Format.HYBRID:
        return _lib.FMT_E4M3, _lib.FMT_E5M2
    raise NotImplementedError(f"tensor-wise scaling is defined for Format.E4M3 and Format.HYBRID (got {config.format})")


def _formats(config, fp4: bool):
    if fp4:
        if not isinstance(config, Float4QuantConfig):
            raise TypeError("gemm_fp4 / grouped_gemm_fp4 expect a Float4QuantConfig")
        return fmt_code(config.activation_format), _lib.FMT_E2M1
    if not isinstance(config, Float8QuantConfig):
        raise TypeError("gemm_fp8 / grouped_gemm_fp8 expect a Float8QuantConfig")
    if config.granularity != ScalingGranularity.MX_BLOCKWISE:
        raise NotImplementedError(
            f"only the MX_BLOCKWISE recipe has kernels in this build (got {config.granularity})"
        )
    if config.format == Format.E5M2:
        raise NotImplementedError("the MXFP8 recipe uses E4M3 for every operand (primus_turbo.py:481-487)")
    f = fmt_code(config.format)
    return f, f


def _run(a, b, group_lens, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern, fp4, glu=None, norm=None):
    if trans_a or not trans_b:
        raise ValueError("the MX linear path is NT only: trans_a=False, trans_b=True (primus_turbo.py:1095-1103)")
    if out_dtype not in (None, torch.bfloat16):
        raise ValueError("the MX GEMMs produce bfloat16 output")
    if config is None:
        raise ValueError("config (Float8QuantConfig / Float4QuantConfig) is required")
    tensorwise = (not fp4) and isinstance(config, Float8QuantConfig) and config.granularity == ScalingGranularity.TENSORWISE
    blockwise = (not fp4) and isinstance(config, Float8QuantConfig) and config.granularity == ScalingGranularity.BLOCKWISE
    if blockwise:
        if glu is not None or norm is not None or not torch.is_tensor(b):
            raise NotImplementedError("the 128-blockwise recipe runs on a bfloat16 weight, without the fused prologues")
        if config.block_size not in (None, 128):
            raise NotImplementedError(f"blockwise scaling is built for block_size 128 (got {config.block_size})")
    if tensorwise or blockwise:
        fwd_fmt, bwd_fmt = _tensorwise_formats(config)
        act_fmt = w_fmt = fwd_fmt
    else:
        act_fmt, w_fmt = _formats(config, fp4)
    if a.dim() != 2 or a.dtype != torch.bfloat16:
        raise ValueError("activations must be a 2-D bfloat16 tensor (callers flatten to [tokens, K])")
    if not a.is_contiguous():
        raise ValueError("activations must be contiguous")
    b_t = None
    if isinstance(b, QuantizedTensorPair):
        b, b_t = b.data, b.data_t
        if b.fmt != w_fmt:
            raise ValueError("cached weight format does not match the op")
    elif isinstance(b, QuantizedTensor):
        pass
    else:
        if b.dtype != torch.bfloat16:
            raise ValueError("weights must be bfloat16 or a QuantizedTensorPair")
        if not b.is_contiguous():
            raise ValueError("weights must be contiguous")
    want_dims = 2 if group_lens is None else 3
    if b.dim() != want_dims:
        raise ValueError(f"weights must have {want_dims} dims ([N, K] dense, [G, N, K] grouped)")
    k_act = a.shape[-1] // 2 if glu is not None else a.shape[-1]
    if b.shape[-1] != k_act:
        raise ValueError(f"contraction dims differ: activations K={k_act}, weights K={b.shape[-1]}")
    if group_lens is not None and group_lens.numel() != b.shape[0]:
        raise ValueError("group_lens must have one entry per expert weight")
    # the reference sets the pattern for tensor-wise FP8 only (primus_turbo.py:243-275); the wgrad kernel here
    # accumulates for every recipe
    accum = _accum_from(b, fuse_bgrad_accum_pattern)
    if blockwise:
        if a.shape[-1] % 128 != 0 or b.shape[-2] % 128 != 0:
            raise ValueError("the 128-blockwise recipe needs K and N to be multiples of 128")
        return _BWLinearFunction.apply(a, b, group_lens, fwd_fmt, bwd_fmt, accum)
    if tensorwise:
        if glu is not None or norm is not None:
            raise NotImplementedError("the activation / normalisation prologues exist for the MX recipes only")
        return _TWLinearFunction.apply(a, b, b_t, group_lens, fwd_fmt, bwd_fmt, accum)
    # stochastic rounding applies to E2M1 gradients; with E4M3 activations the gradients are MXFP8
    grad_sr = bool(fp4 and config.use_gradient_sr and act_fmt == _lib.FMT_E2M1)
    rht = getattr(config, "colwise_rht_signs", None) if fp4 and act_fmt == _lib.FMT_E2M1 else None
    if norm is not None:
        if rht is not None or group_lens is not None:
            raise NotImplementedError("the normalisation prologue exists for the dense linear without the Hadamard transform")
        norm_weight, eps = norm
        if norm_weight.dtype != torch.bfloat16 or tuple(norm_weight.shape) != (a.shape[-1],):
            raise ValueError("the norm weight must be a bfloat16 vector of the contraction length")
        return _MXLinearFunction.apply(a, b, b_t, None, act_fmt, w_fmt, config.scale_mode.value,
                                       None, None, None, grad_sr, None, norm_weight.contiguous(), float(eps), accum)
    if glu is None:
        return _MXLinearFunction.apply(a, b, b_t, group_lens, act_fmt, w_fmt, config.scale_mode.value,
                                       None, None, None, grad_sr, rht, None, 0.0, accum)
    if rht is not None:
        raise NotImplementedError("the activation prologue and the Hadamard transform cannot be combined")
    probs, row_mask, activation = glu
    if activation not in ("silu", "gelu"):
        raise ValueError(f"activation must be 'silu' or 'gelu', got {activation!r}")
    if probs.dim() != 1 or probs.shape[0] != a.shape[0]:
        raise ValueError("probs must be 1-D with one entry per row of the activations")
    return _MXLinearFunction.apply(a, b, b_t, group_lens, act_fmt, w_fmt, config.scale_mode.value,
                                   probs.contiguous(), row_mask, activation, grad_sr, None, None, 0.0, accum)


def gemm_fp8(a, b, trans_a: bool = False, trans_b: bool = True, out_dtype: Optional[torch.dtype] = None,
             config: Optional[Float8QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    """``a[M, K] @ b[N, K]^T`` with MXFP8 operands; ``b`` is a bf16 weight or a
    ``QuantizedTensorPair`` of cached copies.  Differentiable in ``a`` and ``b``."""
    return _run(a, b, None, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern, fp4=False)


def gemm_fp4(a, b, trans_a: bool = False, trans_b: bool = True, out_dtype: Optional[torch.dtype] = None,
             config: Optional[Float4QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    """Same with MXFP4 weights (activations per ``config.activation_format``)."""
    return _run(a, b, None, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern, fp4=True)


class _RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        w = weight.detach().contiguous()
        y, rstd = K.rmsnorm_fwd_impl(x2, w, eps)
        ctx.save_for_backward(x2, w, rstd)
        ctx.shape = shape
        return y.view(shape)

    @staticmethod
    def backward(ctx, dy):
        x2, w, rstd = ctx.saved_tensors
        dy2 = dy.reshape(x2.shape)
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        dx, dw = K.rmsnorm_bwd_impl(dy2.contiguous(), x2, w, rstd)
        return dx.view(ctx.shape), dw, None


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``(x / sqrt(mean(x^2, -1) + eps)) * weight`` over the last dim, bf16 in and out, fp32 arithmetic with one
    rounding; differentiable in ``x`` and ``weight``.  Call site of the reference: ``rmsnorm(x,
    self.layer_norm_weight, self.eps)`` in front of the column-parallel linear (primus_turbo.py:1689-1700)."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError("rmsnorm expects bfloat16 input and weight")
    return _RMSNormFunction.apply(x, weight, float(eps))


def rmsnorm_gemm_fp8(x, norm_weight, eps: float, b, trans_a: bool = False, trans_b: bool = True,
                     out_dtype: Optional[torch.dtype] = None, config: Optional[Float8QuantConfig] = None,
                     fuse_bgrad_accum_pattern: Optional[str] = None):
    """``gemm_fp8(rmsnorm(x, norm_weight, eps), b)`` for 2-D ``x`` with the normalisation folded into the
    quantiser of the GEMM's input: same values bit for bit, forward and backward, without the normalised
    tensor being written or re-read.  Differentiable in ``x``, ``norm_weight`` and ``b``.  The reference runs
    the two operators one after the other (primus_turbo.py:1689-1741)."""
    return _run(x, b, None, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern, fp4=False,
                norm=(norm_weight, eps))


def rmsnorm_gemm_fp4(x, norm_weight, eps: float, b, trans_a: bool = False, trans_b: bool = True,
                     out_dtype: Optional[torch.dtype] = None, config: Optional[Float4QuantConfig] = None,
                     fuse_bgrad_accum_pattern: Optional[str] = None):
    return _run(x, b, None, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern, fp4=True,
                norm=(norm_weight, eps))


def _lens(group_lens: torch.Tensor) -> torch.Tensor:
    if group_lens is None:
        raise ValueError("group_lens (tokens per expert) is required")
    if group_lens.dtype != torch.int64:
        group_lens = group_lens.to(torch.int64)
    return group_lens.contiguous()


def grouped_gemm_fp8(a, b, group_lens: torch.Tensor, trans_b: bool = True,
                     config: Optional[Float8QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    """Per expert g: ``a[rows of g] @ b[g]^T``; ``group_lens`` is tokens per
    expert (int64, on the device of ``a``, zeros allowed) and is never read
    back to the host."""
    return _run(a, b, _lens(group_lens), False, trans_b, None, config, fuse_bgrad_accum_pattern, fp4=False)


def grouped_gemm_fp4(a, b, group_lens: torch.Tensor, trans_b: bool = True,
                     config: Optional[Float4QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    return _run(a, b, _lens(group_lens), False, trans_b, None, config, fuse_bgrad_accum_pattern, fp4=True)


def glu_grouped_gemm_fp8(x, probs, b, group_lens: torch.Tensor, activation: str = "silu",
                         row_mask: Optional[torch.Tensor] = None, trans_b: bool = True,
                         config: Optional[Float8QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    """fc2 of the expert MLP with the gated activation folded into its quantiser:
    ``grouped_gemm_fp8(swiglu_with_probs(x, probs, row_mask), b, group_lens)`` (``geglu`` for
    ``activation="gelu"``) for ``x [tokens, 2F]`` = fc1's output, same values bit for bit, forward and
    backward, without the activated tensor ``[tokens, F]`` being written or re-read.  Differentiable
    in ``x``, ``probs`` and ``b``.  The reference runs the two operators separately
    (primus/backends/megatron/core/transformer/experts.py:120-165, then :2122-2129 of
    extensions/primus_turbo.py)."""
    return _run(x, b, _lens(group_lens), False, trans_b, None, config, fuse_bgrad_accum_pattern, fp4=False,
                glu=(probs, row_mask, activation))


def glu_grouped_gemm_fp4(x, probs, b, group_lens: torch.Tensor, activation: str = "silu",
                         row_mask: Optional[torch.Tensor] = None, trans_b: bool = True,
                         config: Optional[Float4QuantConfig] = None, fuse_bgrad_accum_pattern: Optional[str] = None):
    return _run(x, b, _lens(group_lens), False, trans_b, None, config, fuse_bgrad_accum_pattern, fp4=True,
                glu=(probs, row_mask, activation))


# ---------------------------------------------------------------------------
# Unquantised operators.  The reference's modules fall back to them outside a
# low-precision autocast (primus_turbo.py:1180-1188, :2210-2216).  The grouped
# one has its own kernels (csrc/mx_gemm_bf16.hip): tokens per expert stay on
# the device, as in the quantised operators.  The dense one is the library GEMM
# behind ``torch.matmul``.
# ---------------------------------------------------------------------------
class _PlainLinearAccum(torch.autograd.Function):
    """Unquantised dense ``a . b^T`` whose weight gradient is added to ``b.main_grad``."""

    @staticmethod
    def forward(ctx, a, b, accum):
        ctx.save_for_backward(a, b)
        ctx.accum = accum
        return torch.matmul(a, b.transpose(-2, -1))

    @staticmethod
    def backward(ctx, dy):
        a, b = ctx.saved_tensors
        target, _ = ctx.accum
        grad_a = torch.matmul(dy, b)
        target.add_(torch.matmul(dy.transpose(-2, -1), a))
        return grad_a, _finish_wgrad(None, ctx.accum, True, tuple(b.shape)), None


class _GroupedLinearBf16(torch.autograd.Function):
    """``a[rows of g] . b[g]^T`` (``trans_b``) or ``a[rows of g] . b[g]`` on bf16 operands through the grouped bf16
    kernels; ``group_lens`` is a device tensor and is never read on the host.  With ``accum`` the weight gradient is
    added to the float32 ``main_grad`` inside the wgrad GEMM."""

    @staticmethod
    def forward(ctx, a, b, group_lens, trans_b, accum):
        ctx.save_for_backward(a, b, group_lens)
        ctx.trans_b, ctx.accum = trans_b, accum
        return K.grouped_gemm_bf16_impl(a, b, group_lens, b_kn=not trans_b)

    @staticmethod
    def backward(ctx, dy):
        a, b, group_lens = ctx.saved_tensors
        dy = dy.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        grad_a = grad_b = None
        if ctx.needs_input_grad[0]:
            # b [G, n, k]: dx = dy . b_g contracts over n, which is b's slow dim; b [G, k, n]: dx = dy . b_g^T
            grad_a = K.grouped_gemm_bf16_impl(dy, b, group_lens, b_kn=ctx.trans_b)
        if ctx.needs_input_grad[1]:
            p, q = (dy, a) if ctx.trans_b else (a, dy)      # dW [n, k] = dy^T x;  dW [k, n] = x^T dy
            fused = ctx.accum is not None and _fusable(ctx.accum[0])
            gb = K.grouped_gemm_bf16_wgrad_impl(p, q, group_lens, accum_into=ctx.accum[0] if fused else None)
            grad_b = _finish_wgrad(None if fused else gb, ctx.accum, fused, tuple(b.shape))
        return grad_a, grad_b, None, None, None


def gemm(a, b, trans_a: bool = False, trans_b: bool = True, out_dtype: Optional[torch.dtype] = None,
         fuse_bgrad_accum_pattern: Optional[str] = None):
    accum = _accum_from(b, fuse_bgrad_accum_pattern)
    if accum is not None:
        if trans_a or not trans_b or a.dim() != 2:
            raise ValueError("fuse_bgrad_accum_pattern is defined for the NT linear on 2-D activations")
        out = _PlainLinearAccum.apply(a, b, accum)
        return out if out_dtype is None else out.to(out_dtype)
    a2 = a.transpose(-2, -1) if trans_a else a
    b2 = b.transpose(-2, -1) if trans_b else b
    out = torch.matmul(a2, b2)
    return out if out_dtype is None else out.to(out_dtype)


class _GroupedLinearLibrary(torch.autograd.Function):
    """The same operator for operands the bf16 kernels do not take -- float32 / float16, or tensors in host memory, as
    the host-side module tests use them: a loop of the library GEMM behind ``torch.matmul`` per expert, which reads
    the counts on the host.  bf16 operands on the GPU never come here."""

    @staticmethod
    def forward(ctx, a, b, lens, trans_b, accum):
        ctx.save_for_backward(a, b)
        ctx.lens, ctx.trans_b, ctx.accum = lens, trans_b, accum
        parts = [torch.matmul(rows, b[g].transpose(-2, -1) if trans_b else b[g]) for g, rows in enumerate(torch.split(a, lens, dim=0))]
        return torch.cat(parts, dim=0)

    @staticmethod
    def backward(ctx, dy):
        a, b = ctx.saved_tensors
        parts, grads = [], []
        for g, (d, rows) in enumerate(zip(torch.split(dy, ctx.lens, dim=0), torch.split(a, ctx.lens, dim=0))):
            parts.append(torch.matmul(d, b[g] if ctx.trans_b else b[g].transpose(-2, -1)))
            grads.append(torch.matmul(d.transpose(-2, -1), rows) if ctx.trans_b else torch.matmul(rows.transpose(-2, -1), d))
        grad_b = torch.stack(grads, dim=0).to(b.dtype)
        return torch.cat(parts, dim=0), _finish_wgrad(grad_b, ctx.accum, False, tuple(b.shape)), None, None, None


def grouped_gemm(a, b, group_lens: torch.Tensor, trans_b: bool = True,
                 fuse_bgrad_accum_pattern: Optional[str] = None):
    """Per expert g: ``a[rows of g] @ b[g]^T`` (``trans_b``; ``b [G, n, k]``) or ``a[rows of g] @ b[g]`` (``b [G, k, n]``)
    (primus/backends/megatron/core/extensions/primus_turbo.py:2210-2216).  bf16 operands on the GPU -- what the
    reference's modules pass -- run on the grouped bf16 kernels: ``group_lens`` (int64, on the device) is consumed by
    the kernels, no host read, so the call can be captured in a graph; rows of ``a`` the counts do not cover are left
    unwritten; contraction length and output width in multiples of 32 (anything else raises: there is no second path
    for bf16).  Other dtypes, and tensors in host memory, go through a per-expert loop of the library GEMM."""
    accum = _accum_from(b, fuse_bgrad_accum_pattern)
    if accum is not None and not trans_b:
        raise ValueError("fuse_bgrad_accum_pattern is defined for the NT linear")
    if a.is_cuda and a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16:
        if a.shape[-1] % 32 != 0 or b.shape[-1] % 32 != 0 or b.shape[-2] % 32 != 0:
            raise ValueError("the bf16 grouped GEMM needs k and n in multiples of 32 (forward and dgrad contract over them)")
        return _GroupedLinearBf16.apply(a.contiguous(), b.contiguous(), _lens(group_lens), bool(trans_b), accum)
    lens = [int(v) for v in _lens(group_lens).tolist()]
    if sum(lens) != a.shape[0]:
        raise ValueError("group_lens must sum to the number of rows of a")
    return _GroupedLinearLibrary.apply(a, b, lens, bool(trans_b), accum)


# ---------------------------------------------------------------------------
# Gated activation fused with the router probability and the row mask: the three operators the
# reference's fused_bias_act_with_probs calls (primus_turbo.py:1954-1980).
# ---------------------------------------------------------------------------
def tokens_per_expert_to_mask(tokens_per_expert: torch.Tensor, num_tokens: int) -> torch.Tensor:
    """``mask[i] = i < sum(tokens_per_expert)``: the live rows of a buffer sized for the worst case.
    Stays on the device (no host read of the counts)."""
    total = tokens_per_expert.sum()
    return torch.arange(num_tokens, device=tokens_per_expert.device) < total


class _GluWithProbs(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, probs, row_mask, activation):
        ctx.save_for_backward(x, probs, row_mask)
        ctx.activation = activation
        return K.glu_with_probs_fwd_impl(x, probs, row_mask, activation)

    @staticmethod
    def backward(ctx, dy):
        x, probs, row_mask = ctx.saved_tensors
        dy = dy.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        dx, dp = K.glu_with_probs_bwd_impl(dy, x, probs, row_mask, ctx.activation)
        return dx, dp.to(probs.dtype), None, None


def _glu_with_probs(x, probs, row_mask, activation):
    if not x.is_contiguous():
        x = x.contiguous()
    return _GluWithProbs.apply(x, probs.contiguous(), row_mask, activation)


def swiglu_with_probs(x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(x[:, :F]) * x[:, F:] * probs[:, None]`` for bf16 ``x [tokens, 2F]``; rows whose mask is
    False give zeros.  Differentiable in ``x`` and ``probs``."""
    return _glu_with_probs(x, probs, row_mask, "silu")


def geglu_with_probs(x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Same with the (erf) GELU as the gate activation."""
    return _glu_with_probs(x, probs, row_mask, "gelu")


class _PadGroups(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, group_lens, align):
        out, padded_lens = K.pad_groups_impl(x.contiguous(), group_lens, align)
        ctx.save_for_backward(group_lens)
        ctx.align, ctx.rows = align, x.shape[0]
        ctx.mark_non_differentiable(padded_lens)
        return out, padded_lens

    @staticmethod
    def backward(ctx, dout, _):
        (group_lens,) = ctx.saved_tensors
        return K.unpad_groups_impl(dout.contiguous(), group_lens, ctx.align, ctx.rows), None, None


class _UnpadGroups(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, group_lens, align, rows):
        ctx.save_for_backward(group_lens)
        ctx.align, ctx.padded_rows = align, y.shape[0]
        return K.unpad_groups_impl(y.contiguous(), group_lens, align, rows)

    @staticmethod
    def backward(ctx, dout):
        (group_lens,) = ctx.saved_tensors
        dy, _ = K.pad_groups_impl(dout.contiguous(), group_lens, ctx.align)
        assert dy.shape[0] == ctx.padded_rows, "unpad_groups takes the buffer pad_groups made for the same counts"
        return dy, None, None, None


def pad_groups(x: torch.Tensor, group_lens: torch.Tensor, align: int):
    """``(padded, padded_lens)``: the rows of every expert followed by zero rows up to a multiple of ``align``,
    with the counts staying on the device (the reference reads them back and concatenates per expert,
    experts.py:196-209).  ``padded`` is sized for the worst case, ``(rows + G * (align - 1)) // align * align`` rows;
    the zero rows behind the last expert's padding count into ``padded_lens[-1]``, so ``padded_lens`` always
    describes the whole buffer.  Differentiable in ``x``."""
    return _PadGroups.apply(x, group_lens, int(align))


def unpad_groups(y: torch.Tensor, group_lens: torch.Tensor, align: int, rows: int) -> torch.Tensor:
    """The ``rows`` live rows of a buffer made by ``pad_groups`` for the same counts (experts.py:262-264).
    Differentiable in ``y``: padding rows get a zero gradient."""
    return _UnpadGroups.apply(y, group_lens, int(align), int(rows))
