"""Model config -> FP4 quant config and the per-layer FP4 context
(primus/backends/megatron/core/fp4_utils.py:59-243)."""

from __future__ import annotations

import warnings
from contextlib import nullcontext

from ..pytorch.core.low_precision import Format, ScaleDtype, ScalingGranularity
from . import runtime
from .enums import Fp4Recipe
from .extensions.primus_turbo import (
    MXFP4_SCALING_BLOCK_SIZE,
    PrimusTurboQuantConfig,
    primus_turbo_fp4_autocast,
)

WARN_ONCE = True
_UNSET = object()


def _primus_turbo_enabled() -> bool:
    """fp4_utils.py:43-54: the Turbo FP4 path is used exactly when the global
    arguments enable Primus-Turbo."""
    try:
        return bool(getattr(runtime.get_args(), "enable_primus_turbo", False))
    except Exception:
        return False


def _mxfp4_gradient_sr_enabled(config) -> bool:
    """Stochastic rounding of gradients: an explicit config field wins, else
    the global argument, else off (fp4_utils.py:59-76)."""
    value = getattr(config, "mxfp4_gradient_stochastic_rounding", _UNSET)
    if value is not _UNSET:
        return bool(value)
    try:
        return bool(getattr(runtime.get_args(), "mxfp4_gradient_stochastic_rounding", False))
    except Exception:
        return False


def get_fp4_quant_config(config):
    """``(PrimusTurboQuantConfig | None, reason_if_none)`` (fp4_utils.py:120-151)."""
    if config.fp4_recipe != Fp4Recipe.mxfp4:
        return None, "Only MXFP4 is supported in Primus-Turbo."
    quant_config = PrimusTurboQuantConfig(
        granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E2M1_X2, block_size=MXFP4_SCALING_BLOCK_SIZE,
        scale_dtype=ScaleDtype.E8M0, use_gradient_sr=_mxfp4_gradient_sr_enabled(config),
    )
    return quant_config, ""


def get_fp4_context(config, layer_no: int = -1, is_init: bool = False):
    """fp4_utils.py:153-243: bf16 for the configured first/last layers, nothing
    for the "local" transformer implementation (it quantises inside its own
    modules), else the Primus-Turbo FP4 autocast."""
    bf16_ends = bool(getattr(config, "first_last_layers_bf16", False))
    at_start = int(getattr(config, "num_layers_at_start_in_bf16", 0) or 0) if bf16_ends else 0
    at_end = int(getattr(config, "num_layers_at_end_in_bf16", 0) or 0) if bf16_ends else 0
    need = config.fp4 if not is_init else getattr(config, "fp4_param", False)
    if not need:
        return nullcontext()
    if layer_no >= 0 and bf16_ends and (layer_no < at_start or layer_no >= int(config.num_layers) - at_end):
        return nullcontext()
    if getattr(config, "transformer_impl", "transformer_engine") == "local":
        return nullcontext()
    global WARN_ONCE
    if is_init:
        if WARN_ONCE:
            warnings.warn(f"Primus-Turbo FP4 {config.fp4_recipe} not work since Primus-Turbo not support fp4 model init.")
            WARN_ONCE = False
        return nullcontext()
    if not (_primus_turbo_enabled() and not getattr(config, "fp4_use_native_te_autocast", False)):
        raise RuntimeError(
            "the FP4 context without Primus-Turbo is Transformer Engine's own autocast, which is not part of "
            "this package; set enable_primus_turbo=True and fp4_use_native_te_autocast=False"
        )
    quant_config, why = get_fp4_quant_config(config)
    if quant_config is None and WARN_ONCE:
        warnings.warn(f"Primus-Turbo FP4 {config.fp4_recipe} not work since {why}")
        WARN_ONCE = False
    return primus_turbo_fp4_autocast(
        enabled=False, fp4_recipe=None, fp4_group=None,
        enabled_turbo=quant_config is not None, turbo_quant_config=quant_config,
    )
