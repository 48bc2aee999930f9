"""``from primus_turbo.pytorch.ops.normalization import rmsnorm`` -- the import the reference's
LayerNormColumnParallelLinear makes (primus/backends/megatron/core/extensions/primus_turbo.py:1696-1698)."""

from . import rmsnorm  # noqa: F401

__all__ = ["rmsnorm"]
