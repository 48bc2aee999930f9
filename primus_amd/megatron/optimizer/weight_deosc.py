"""The weight quantisation grid as the optimizer sees it
(primus/backends/megatron/core/optimizer/weight_deosc.py:136-174 ``qdq_mxfp4``,
:177-251 the local-shard tiling).

``Q(w) = dequantise(quantise(w))`` must use the grid of the forward GEMM's
weight operand: MX blocks of 32 with E8M0 scales, ``float4_e2m1fn_x2``
elements, 2-D 32x32 tiles, quantised along the last axis; every expert of a
``[G, out, in]`` weight is an independent 2-D matrix.  So ``Q(w)[i, j]``
depends on the whole 32x32 tile around ``(i, j)``, in the coordinates of the
full weight -- which is what the shard function below reconstructs for a flat
slice of a distributed optimizer's parameter.
"""

from __future__ import annotations

from typing import Tuple

import torch

from ...pytorch.core.low_precision import MXScalingRecipe, ScalingGranularity, float4_e2m1fn_x2
from ...pytorch.core.quantized_tensor import QuantizedTensor

MXFP4_SCALING_BLOCK_SIZE = 32


@torch.no_grad()
def qdq_mxfp4(weight: torch.Tensor) -> torch.Tensor:
    """Quantise-dequantise ``weight`` ([out, in] or [G, out, in]) on the forward grid."""
    if weight.ndim not in (2, 3):
        raise ValueError(f"qdq_mxfp4 expects a 2D or 3D weight, got {weight.ndim}D")
    src = weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)
    # the 2-D block kernel batches over the leading dim, so a grouped weight is one call
    qt = QuantizedTensor.quantize(
        src, dest_dtype=float4_e2m1fn_x2, granularity=ScalingGranularity.MX_BLOCKWISE,
        block_size=MXFP4_SCALING_BLOCK_SIZE, scaling_recipe=MXScalingRecipe(use_2d_block=True), axis=-1,
    )
    out = qt.dequantize()
    if out.shape != weight.shape:
        out = out[tuple(slice(0, s) for s in weight.shape)].contiguous()
    return out.to(weight.dtype)


@torch.no_grad()
def qdq_mxfp4_local_shard(shard_main_param: torch.Tensor, full_shape: Tuple[int, ...], start: int, end: int,
                          model_dtype: torch.dtype) -> torch.Tensor:
    """``Q`` of the flat slice ``[start, end)`` of a weight of shape
    ``full_shape``, without gathering the rest: for each matrix the slice
    touches, the band of 32-row tile rows it covers is rebuilt at its original
    coordinates (elements outside the slice are zero), quantised, and the
    slice's part copied back.  Tiles entirely inside the slice come out exact;
    the two boundary tile rows see zeros where other ranks' data would be."""
    shape = tuple(int(d) for d in full_shape)
    if len(shape) not in (2, 3):
        raise ValueError(f"local MXFP4 QDQ expects a 2D or 3D full shape, got {shape}")
    if min(shape) <= 0:
        raise ValueError(f"local MXFP4 QDQ requires positive dimensions, got {shape}")
    numel = 1
    for d in shape:
        numel *= d
    if not 0 <= start <= end <= numel:
        raise ValueError(f"invalid local shard range [{start}, {end}) for shape {shape}")
    flat = shard_main_param.detach().reshape(-1)
    if flat.numel() != end - start:
        raise ValueError(f"local shard has {flat.numel()} elements, expected {end - start} for range [{start}, {end})")
    # the forward quantises the model-dtype weight, not the fp32 master
    local = flat.to(dtype=model_dtype)
    if local.numel() == 0:
        return local
    out = torch.empty_like(local)
    rows, cols = shape[-2:]
    per_matrix = rows * cols
    blk = MXFP4_SCALING_BLOCK_SIZE
    for m in range(start // per_matrix, (end - 1) // per_matrix + 1):
        lo = max(start, m * per_matrix) - m * per_matrix       # slice within matrix m
        hi = min(end, (m + 1) * per_matrix) - m * per_matrix
        band_lo = (lo // cols) // blk * blk                     # first row of the covering tile rows
        band_hi = ((hi - 1) // cols // blk + 1) * blk
        band = torch.zeros((band_hi - band_lo, cols), device=local.device, dtype=model_dtype)
        b0, b1 = lo - band_lo * cols, hi - band_lo * cols       # slice within the band
        s0, s1 = lo + m * per_matrix - start, hi + m * per_matrix - start   # slice within the shard
        band.view(-1)[b0:b1].copy_(local[s0:s1])
        out[s0:s1].copy_(qdq_mxfp4(band).reshape(-1)[b0:b1])
    return out
