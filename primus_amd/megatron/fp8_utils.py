"""Model config -> FP8 quant config and the per-layer FP8 context
(primus/backends/megatron/core/fp8_utils.py:130-253).

``config`` is any object with Megatron's ``TransformerConfig`` field names
(``fp8``, ``fp8_recipe``, ``fp8_param``, ``first_last_layers_bf16``,
``num_layers_at_start_in_bf16``, ``num_layers_at_end_in_bf16``,
``num_layers``).  There is no Transformer Engine underneath, so the context
only drives the state the Primus-Turbo modules read (``enabled`` stays False)."""

from __future__ import annotations

import warnings
from contextlib import nullcontext

from ..pytorch.core.low_precision import Format, ScaleDtype, ScalingGranularity
from .enums import Fp8Recipe
from .extensions.primus_turbo import (
    MXFP8_SCALING_BLOCK_SIZE,
    SCALING_BLOCK_SIZE,
    PrimusTurboQuantConfig,
    primus_turbo_fp8_autocast,
)

WARN_ONCE = True

_FORMATS = {"e4m3": Format.E4M3, "hybrid": Format.HYBRID}


def is_first_last_bf16_layer(config, layer_no: int) -> bool:
    """Whether global layer ``layer_no`` stays in bf16: the first
    ``num_layers_at_start_in_bf16`` and last ``num_layers_at_end_in_bf16``
    layers do when ``first_last_layers_bf16`` is set (Megatron's rule, used at
    fp8_utils.py:190; the same arithmetic is spelled out at fp4_utils.py:153-164)."""
    if layer_no < 0 or not getattr(config, "first_last_layers_bf16", False):
        return False
    at_start = int(getattr(config, "num_layers_at_start_in_bf16", 0) or 0)
    at_end = int(getattr(config, "num_layers_at_end_in_bf16", 0) or 0)
    return layer_no < at_start or layer_no >= int(config.num_layers) - at_end


def get_fp8_quant_config(config):
    """``(PrimusTurboQuantConfig | None, reason_if_none)`` (fp8_utils.py:130-170)."""
    if config.fp8 not in _FORMATS:
        raise ValueError("E4M3 and HYBRID are the only supported FP8 formats.")
    fmt = _FORMATS[config.fp8]
    recipe = config.fp8_recipe
    if recipe == Fp8Recipe.delayed:
        return None, "Primus-Turbo not support delayed scaling."
    if recipe == Fp8Recipe.tensorwise:
        return PrimusTurboQuantConfig(granularity=ScalingGranularity.TENSORWISE, format=fmt), ""
    if recipe == Fp8Recipe.blockwise:
        return PrimusTurboQuantConfig(granularity=ScalingGranularity.BLOCKWISE, format=fmt,
                                      block_size=SCALING_BLOCK_SIZE), ""
    if recipe == Fp8Recipe.mxfp8:
        return PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=fmt,
                                      block_size=MXFP8_SCALING_BLOCK_SIZE, scale_dtype=ScaleDtype.E8M0), ""
    return None, ""


def get_fp8_context(config, layer_no: int = -1, is_init: bool = False):
    """Context manager for one layer's forward: ``nullcontext`` for bf16
    training and for the bf16 first/last layers, else the Primus-Turbo FP8
    autocast with the recipe's quant config (fp8_utils.py:172-253).
    ``layer_no < 0`` means "every layer"."""
    need = config.fp8 if not is_init else getattr(config, "fp8_param", False)
    if not need or is_first_last_bf16_layer(config, layer_no):
        return nullcontext()
    quant_config, why = get_fp8_quant_config(config)
    global WARN_ONCE
    if WARN_ONCE:
        if quant_config is None:
            warnings.warn(f"Primus-Turbo FP8 {config.fp8_recipe} not work since {why}")
        if is_init:
            warnings.warn(f"Primus-Turbo FP8 {config.fp8_recipe} not work since Primus-Turbo not support fp8 model init.")
        WARN_ONCE = False
    if is_init:
        # quantised parameter initialisation belongs to Transformer Engine; nothing to enter here
        return nullcontext()
    return primus_turbo_fp8_autocast(
        enabled=False, fp8_recipe=None, fp8_group=None,
        enabled_turbo=quant_config is not None, turbo_quant_config=quant_config,
    )
