"""QuantizedTensor / QuantizedTensorPair / create_quantized_weight.

Host-side mirror of the objects the reference imports from
``primus_turbo.pytorch.core`` and uses to cache quantised weights
(primus/backends/megatron/core/extensions/primus_turbo.py:215-237 the pair,
:278-358 building the row-wise and the transposed col-wise copy,
weight_deosc.py:155-168 quantize -> dequantize round trip).

A ``QuantizedTensor`` is a wrapper tensor: to autograd it looks like a tensor
of the original dtype and of the *logical* shape of what it holds, so a
weight gradient can flow to it (primus_turbo.py:194-213), while the payload
is MX codes plus E8M0 scales.
"""

from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from ... import _lib
from .. import kernels as K
from .low_precision import (
    Float4QuantConfig,
    Float8QuantConfig,
    Format,
    MXScalingRecipe,
    ScaleMode,
    ScalingGranularity,
    dtype_to_fmt_code,
    float8_e4m3,
)

_PASS_THROUGH = None  # filled lazily: aten ops that only re-wrap the payload


def _pass_through_ops():
    global _PASS_THROUGH
    if _PASS_THROUGH is None:
        aten = torch.ops.aten
        _PASS_THROUGH = {aten.detach.default, aten.alias.default, aten.clone.default, aten.view_as.default}
    return _PASS_THROUGH


class QuantizedTensor(torch.Tensor):
    """MX codes + E8M0 scales behind a tensor of the original dtype.

    ``axis=-1``: blocks of 32 along the last dim, payload in the orientation of
    the source.  ``axis=-2``: blocks along the second-to-last dim and the
    payload (and therefore the logical shape) TRANSPOSED
    (primus_turbo.py:346-354).  ``segment_lens`` marks a transposed activation
    copy whose blocks restart at expert boundaries and whose token dim is
    padded per expert.  ``kchunk`` marks a payload stored K-chunk-major
    (``codes[ld/128, rows, 128 elements]``, the layout the GEMMs load fastest);
    the scales have the same shape in both layouts.
    """

    @staticmethod
    def __new__(cls, codes, scales, *, logical_shape, orig_dtype=torch.bfloat16, axis=-1, use_2d_block=False,
                scale_mode=ScaleMode.OCP_FLOOR, segment_lens=None, total_rows=None, requires_grad=False, kchunk=False,
                tensor_scale_inv=None):
        return torch.Tensor._make_wrapper_subclass(
            cls, tuple(logical_shape), dtype=orig_dtype, device=codes.device, requires_grad=requires_grad
        )

    def __init__(self, codes, scales, *, logical_shape, orig_dtype=torch.bfloat16, axis=-1, use_2d_block=False,
                 scale_mode=ScaleMode.OCP_FLOOR, segment_lens=None, total_rows=None, requires_grad=False, kchunk=False,
                 tensor_scale_inv=None):
        # tensor-wise scaled payload: float32 reciprocal scale of the whole tensor (one element, on the device);
        # ``scales`` then holds unit E8M0 bytes, which only make the codes acceptable to the GEMM kernels
        self._tensor_scale_inv = tensor_scale_inv
        self._kchunk = K._layout(kchunk)
        self._codes = codes
        self._scales = scales
        self._axis = axis
        self._use_2d_block = use_2d_block
        self._scale_mode = scale_mode
        self._segment_lens = segment_lens
        self._total_rows = total_rows

    # -- payload accessors -------------------------------------------------
    @property
    def codes(self) -> torch.Tensor:
        return self._codes

    @property
    def scales(self) -> torch.Tensor:
        return self._scales

    @property
    def axis(self) -> int:
        return self._axis

    @property
    def use_2d_block(self) -> bool:
        return self._use_2d_block

    @property
    def kchunk(self) -> int:
        """Storage layout: 0 row-major, 1 K-chunk-major codes, 2 K-step-major codes and scales."""
        return self._kchunk

    @property
    def tensor_scale_inv(self) -> Optional[torch.Tensor]:
        return self._tensor_scale_inv

    def rowmajor_codes(self) -> torch.Tensor:
        """The payload as ``[..., rows, ld]`` whatever layout it is stored in (a copy if K-chunk-major)."""
        if not self._kchunk:
            return self._codes
        flat = K.unchunk(self._codes)
        return flat.view(tuple(self.shape[:-1]) + (flat.shape[-1],))

    def rowmajor_scales(self) -> torch.Tensor:
        """The scales as ``[..., rows, ld / 32]`` whatever layout they are stored in (a copy if K-step-major)."""
        if self._kchunk < K.LAYOUT_KSTEP:
            return self._scales
        if self._segment_lens is not None:
            raise NotImplementedError("row-major scales of a K-step-major copy that is split into groups")
        per = 2 if self.fmt == _lib.FMT_E2M1 else 1   # elements per code byte
        blocks = self._codes.shape[0] * self._codes.shape[2] * per // _lib.BLOCK
        flat = K.unpanel(self._scales.view(torch.uint8), blocks).view(self._scales.dtype)
        return flat.view(tuple(self.shape[:-1]) + (blocks,))

    def preshuffled_codes(self) -> torch.Tensor:
        """The payload of a 2-D MXFP4 tensor in the pre-shuffled byte order of the reference's FP4 GEMM back end
        (``shuffle_out`` of the scaling recipe, primus_turbo.py:305-311): a copy."""
        if self.fmt != _lib.FMT_E2M1 or self.dim() != 2:
            raise ValueError("the pre-shuffled layout is defined for 2-D MXFP4 tensors")
        return K.shuffle_codes_impl(self.rowmajor_codes())

    def preshuffled_scales(self) -> torch.Tensor:
        """The scales of a 2-D tensor in the pre-shuffled order (``shuffle_scale``), padded to 256 rows x 8 blocks."""
        if self.dim() != 2 or self._tensor_scale_inv is not None:
            raise ValueError("the pre-shuffled scale layout is defined for 2-D MX tensors")
        return K.shuffle_scales_impl(self.rowmajor_scales())

    @property
    def fmt(self) -> int:
        return dtype_to_fmt_code(self._codes.dtype)

    def _rewrap(self) -> "QuantizedTensor":
        return QuantizedTensor(
            self._codes, self._scales, logical_shape=self.shape, orig_dtype=self.dtype, axis=self._axis,
            use_2d_block=self._use_2d_block, scale_mode=self._scale_mode, segment_lens=self._segment_lens,
            total_rows=self._total_rows, kchunk=self._kchunk, tensor_scale_inv=self._tensor_scale_inv,
        )

    def __repr__(self):  # noqa: D105
        return (f"QuantizedTensor(shape={tuple(self.shape)}, codes={self._codes.dtype}, axis={self._axis}, "
                f"use_2d_block={self._use_2d_block})")

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        if func in _pass_through_ops():
            return args[0]._rewrap()
        if func is torch.ops.aten.view.default and tuple(args[1]) == tuple(args[0].shape):
            # autograd aliases a tensor that a Function returns unchanged with a same-shape view
            return args[0]._rewrap()
        raise NotImplementedError(
            f"{func} is not defined on a QuantizedTensor; call .dequantize() first or hand it to a gemm op"
        )

    # -- construction --------------------------------------------------------
    @classmethod
    def quantize(
        cls,
        x: torch.Tensor,
        dest_dtype: torch.dtype = float8_e4m3,
        granularity: ScalingGranularity = ScalingGranularity.MX_BLOCKWISE,
        block_size: Optional[int] = 32,
        scaling_recipe: Optional[MXScalingRecipe] = None,
        axis: int = -1,
    ) -> "QuantizedTensor":
        """Signature of the reference's call sites (primus_turbo.py:321-354)."""
        if granularity not in (ScalingGranularity.MX_BLOCKWISE, ScalingGranularity.TENSORWISE):
            raise NotImplementedError("only MX_BLOCKWISE and TENSORWISE scaling have kernels in this build")
        if axis not in (-1, -2):
            raise ValueError("axis must be -1 (row-wise) or -2 (column-wise, transposed result)")
        if granularity == ScalingGranularity.TENSORWISE:
            # one scale for the whole tensor; axis=-2 gives the transposed payload like the MX copies do
            fmt = dtype_to_fmt_code(dest_dtype)
            x = x.detach()
            if x.dtype != torch.bfloat16 or x.dim() not in (2, 3):
                raise ValueError("quantize expects a 2-D or 3-D bfloat16 tensor")
            if x.dim() == 3:
                q_row, s_row, q_col, s_col, si = K.quantize_weight_tensorwise_impl(
                    x.contiguous(), fmt, rowwise=(axis == -1), colwise=(axis == -2))
            else:
                q_row, s_row, q_col, s_col, si = K.quantize_tensorwise_impl(
                    x.contiguous(), fmt, rowwise=(axis == -1), colwise=(axis == -2))
            if axis == -1:
                return cls(q_row, s_row, logical_shape=x.shape, orig_dtype=x.dtype, axis=-1, tensor_scale_inv=si)
            shape = tuple(x.shape[:-2]) + (x.shape[-1], x.shape[-2])
            return cls(q_col, s_col, logical_shape=shape, orig_dtype=x.dtype, axis=-2, tensor_scale_inv=si,
                       total_rows=x.shape[-2])
        if block_size not in (None, _lib.BLOCK):
            raise ValueError(f"MX block size must be {_lib.BLOCK}")
        recipe = scaling_recipe or MXScalingRecipe()
        fmt = dtype_to_fmt_code(dest_dtype)
        x = x.detach()
        if x.dtype != torch.bfloat16:
            raise ValueError("quantize expects a bfloat16 tensor")
        if recipe.use_2d_block:
            if x.dim() not in (2, 3):
                raise ValueError("2-D block quantisation expects [n, k] or [G, n, k]")
            q_row, s_row, q_col, s_col = K.quantize_mx_weight_2d_impl(
                x.contiguous(), fmt, recipe.scale_mode.value, rowwise=(axis == -1), colwise=(axis == -2)
            )
            if axis == -1:
                return cls(q_row, s_row, logical_shape=x.shape, orig_dtype=x.dtype, axis=-1, use_2d_block=True,
                           scale_mode=recipe.scale_mode)
            shape = tuple(x.shape[:-2]) + (x.shape[-1], x.shape[-2])
            return cls(q_col, s_col, logical_shape=shape, orig_dtype=x.dtype, axis=-2, use_2d_block=True,
                       scale_mode=recipe.scale_mode)
        if x.dim() < 2:
            raise ValueError("quantize expects at least 2 dims")
        lead = tuple(x.shape[:-2])
        if axis == -1:
            x2 = x.contiguous().view(-1, x.shape[-1])
            q, s, _, _ = K.quantize_mx_impl(x2, fmt, recipe.scale_mode.value, rowwise=True, colwise=False)
            per = 2 if fmt == _lib.FMT_E2M1 else 1
            q = q.view(tuple(x.shape[:-1]) + (x.shape[-1] // per,))
            s = s.view(tuple(x.shape[:-1]) + (x.shape[-1] // _lib.BLOCK,))
            return cls(q, s, logical_shape=x.shape, orig_dtype=x.dtype, axis=-1, scale_mode=recipe.scale_mode)
        if lead:
            raise ValueError("column-wise 1-D block quantisation is defined for 2-D tensors")
        rows = x.shape[0]
        _, _, q, s = K.quantize_mx_impl(x.contiguous(), fmt, recipe.scale_mode.value, rowwise=False, colwise=True)
        return cls(q, s, logical_shape=(x.shape[1], rows), orig_dtype=x.dtype, axis=-2, scale_mode=recipe.scale_mode,
                   total_rows=rows)

    def dequantize(self) -> torch.Tensor:
        """Back to the original dtype in the payload's orientation.  For a
        transposed copy of ``rows`` tokens the padding columns are dropped."""
        out = K.dequantize_mx_impl(self.rowmajor_codes(), self.rowmajor_scales(), self.dtype)
        if self._tensor_scale_inv is not None:
            out = (out.float() * self._tensor_scale_inv).to(self.dtype)   # FP8 values are exact in bf16: one rounding
        if self._axis == -2 and not self._use_2d_block and self._segment_lens is not None:
            raise NotImplementedError("dequantize of a segment-padded activation copy")
        # drop the padding of the contraction dim (GEMM granularity / token padding)
        return out[..., : self.shape[-1]]

    def transpose(self, dim0: int, dim1: int):  # noqa: D102
        raise NotImplementedError(
            "an MX-quantised tensor cannot be transposed (its blocks run along one axis); "
            "quantise with axis=-2 to get the transposed copy (primus_turbo.py:346-354)"
        )


class QuantizedTensorPair:
    """Row-wise weight copy plus its optional transposed copy
    (primus_turbo.py:215-237): ``data`` feeds the forward GEMM and receives the
    weight gradient, ``data_t`` feeds dgrad."""

    def __init__(self, data: QuantizedTensor, data_t: Optional[QuantizedTensor] = None):
        self.data = data
        self.data_t = data_t

    def __repr__(self):  # noqa: D105
        return f"QuantizedTensorPair(data={self.data!r}, data_t={self.data_t!r})"


def create_quantized_weight(
    weight: torch.Tensor,
    dest_dtype: torch.dtype,
    quant_config: Union[Float8QuantConfig, Float4QuantConfig],
    need_weight_transpose_cache: bool = True,
    kchunk: Optional[bool] = None,
) -> Tuple[QuantizedTensor, Optional[QuantizedTensor]]:
    """``(rowwise, colwise_or_None)`` for a weight ``[n, k]`` or ``[G, n, k]``
    (primus_turbo.py:295-301).  Weights use 2-D 32x32 blocks
    (primus_turbo.py:313-317), so both copies come out of one pass over the
    weight and hold the same codes.  ``kchunk`` picks the storage layout of the
    codes (default: K-chunk-major whenever the GEMMs accept it for this size)."""
    if quant_config.granularity not in (ScalingGranularity.MX_BLOCKWISE, ScalingGranularity.TENSORWISE):
        raise NotImplementedError("only MX_BLOCKWISE and TENSORWISE scaling have kernels in this build")
    fmt = dtype_to_fmt_code(dest_dtype)
    w = weight.detach()
    if w.dtype != torch.bfloat16:
        raise ValueError("create_quantized_weight expects a bfloat16 weight")
    mode = quant_config.scale_mode
    if quant_config.granularity == ScalingGranularity.TENSORWISE:
        if kchunk is None:
            kchunk = K.pick_layout(w.numel() // (w.shape[-1] * w.shape[-2]) if w.dim() > 2 else 1, w.shape[-2], w.shape[-1], fp8=True)
        q_row, s_row, q_col, s_col, si = K.quantize_weight_tensorwise_impl(
            w.contiguous(), fmt, rowwise=True, colwise=need_weight_transpose_cache, pad_to=K.GEMM_K_ALIGN, kchunk=kchunk)
        row = QuantizedTensor(q_row, s_row, logical_shape=w.shape, orig_dtype=w.dtype, axis=-1, kchunk=kchunk,
                              tensor_scale_inv=si)
        col = None
        if need_weight_transpose_cache:
            shape = tuple(w.shape[:-2]) + (w.shape[-1], w.shape[-2])
            col = QuantizedTensor(q_col, s_col, logical_shape=shape, orig_dtype=w.dtype, axis=-2, kchunk=kchunk,
                                  tensor_scale_inv=si)
        return row, col
    if kchunk is None:
        kchunk = K.pick_layout(w.numel() // (w.shape[-1] * w.shape[-2]) if w.dim() > 2 else 1, w.shape[-2], w.shape[-1],
                               fp8=fmt != _lib.FMT_E2M1 or getattr(quant_config, "activation_format", None) == Format.E4M3,
                               fp4=fmt == _lib.FMT_E2M1 and getattr(quant_config, "activation_format", None) == Format.E2M1_X2)
    q_row, s_row, q_col, s_col = K.quantize_mx_weight_2d_impl(
        w.contiguous(), fmt, mode.value, rowwise=True, colwise=need_weight_transpose_cache, pad_to=K.GEMM_K_ALIGN,
        kchunk=kchunk,
    )
    row = QuantizedTensor(q_row, s_row, logical_shape=w.shape, orig_dtype=w.dtype, axis=-1, use_2d_block=True,
                          scale_mode=mode, kchunk=kchunk)
    col = None
    if need_weight_transpose_cache:
        shape = tuple(w.shape[:-2]) + (w.shape[-1], w.shape[-2])
        col = QuantizedTensor(q_col, s_col, logical_shape=shape, orig_dtype=w.dtype, axis=-2, use_2d_block=True,
                              scale_mode=mode, kchunk=kchunk)
    return row, col
