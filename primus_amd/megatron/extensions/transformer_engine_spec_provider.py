"""Which module class implements each slot of a transformer-layer spec
(primus/backends/megatron/core/extensions/transformer_engine_spec_provider.py:
120-152, 195-212, 233-285).

The reference picks between its Primus-Turbo classes and Transformer Engine's
by two switches, ``use_turbo_gemm`` and ``use_turbo_grouped_gemm``.  The
Transformer Engine side is not part of this package: ``fallback`` is the
provider to delegate to when a switch is off (inside Megatron, an instance of
its ``TESpecProvider``); without one, asking for a non-Turbo class raises."""

from __future__ import annotations

from typing import Optional

from .. import runtime
from ..transformer.experts import GroupedMLPSubmodules, PrimusGroupedMLP
from .primus_turbo import (
    PrimusTurboColumnParallelGroupedLinear,
    PrimusTurboColumnParallelLinear,
    PrimusTurboLayerNormColumnParallelLinear,
    PrimusTurboLinear,
    PrimusTurboRowParallelGroupedLinear,
    PrimusTurboRowParallelLinear,
)


class PrimusTurboSpecProvider:
    def __init__(self, fallback=None, fallback_to_eager_attn: bool = False):
        self.cfg = runtime.get_args()
        self.fallback = fallback
        self.fallback_to_eager_attn = fallback_to_eager_attn

    def _other(self, slot: str, *args, **kwargs):
        if self.fallback is None:
            raise RuntimeError(
                f"'{slot}' was requested with its Primus-Turbo switch off and no fallback spec provider is set"
            )
        return getattr(self.fallback, slot)(*args, **kwargs)

    def linear(self) -> type:
        return PrimusTurboLinear if self.cfg.use_turbo_gemm else self._other("linear")

    def column_parallel_linear(self) -> type:
        return PrimusTurboColumnParallelLinear if self.cfg.use_turbo_gemm else self._other("column_parallel_linear")

    def row_parallel_linear(self) -> type:
        return PrimusTurboRowParallelLinear if self.cfg.use_turbo_gemm else self._other("row_parallel_linear")

    def fuse_layernorm_and_linear(self) -> bool:
        return True

    def column_parallel_layer_norm_linear(self) -> Optional[type]:
        if self.cfg.use_turbo_gemm:
            return PrimusTurboLayerNormColumnParallelLinear
        return self._other("column_parallel_layer_norm_linear")

    def grouped_mlp_modules(self, moe_use_grouped_gemm: bool, moe_use_legacy_grouped_gemm: Optional[bool] = None):
        """``(mlp_class, submodules)`` for the experts."""
        if moe_use_legacy_grouped_gemm is None:
            moe_use_legacy_grouped_gemm = getattr(self.cfg, "moe_use_legacy_grouped_gemm", False)
        use_turbo_grouped_gemm = self.cfg.use_turbo_grouped_gemm
        assert not (moe_use_legacy_grouped_gemm and use_turbo_grouped_gemm), (
            "moe_use_legacy_grouped_gemm and use_turbo_grouped_gemm are not compatible."
        )
        if moe_use_grouped_gemm and not moe_use_legacy_grouped_gemm and use_turbo_grouped_gemm:
            return PrimusGroupedMLP, GroupedMLPSubmodules(
                linear_fc1=PrimusTurboColumnParallelGroupedLinear,
                linear_fc2=PrimusTurboRowParallelGroupedLinear,
            )
        return self._other("grouped_mlp_modules", moe_use_grouped_gemm, moe_use_legacy_grouped_gemm)
