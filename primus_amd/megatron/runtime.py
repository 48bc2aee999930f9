"""The two process-wide values the reference reads from Megatron while running
the linear path: the parsed arguments (``get_args()``,
primus/backends/megatron/core/extensions/primus_turbo.py:1017,2005,2331 and
core/transformer/experts.py:38) and the number of microbatches per step
(``get_num_microbatches()``, primus_turbo.py:1094,2121), which decides whether
quantised weight copies are cached across microbatches.

Inside Megatron, bind them once::

    from megatron.training.global_vars import get_args
    from megatron.core.num_microbatches_calculator import get_num_microbatches
    runtime.bind(get_args=get_args, get_num_microbatches=get_num_microbatches)

Stand-alone use sets plain values with ``set_args`` / ``set_num_microbatches``.
"""

from __future__ import annotations

from types import SimpleNamespace
from typing import Callable, Optional

# The options this path reads, with the reference's defaults
# (primus/configs/modules/megatron/primus_turbo.yaml:3,42-51: everything off).
_DEFAULT_ARGS = dict(
    enable_primus_turbo=False,
    use_turbo_gemm=False,
    use_turbo_grouped_gemm=False,
    use_turbo_attention=False,
    use_turbo_fused_act_with_probs=False,
    moe_router_padding_for_quantization=False,
    turbo_grouped_gemm_without_padding=False,
    moe_use_legacy_grouped_gemm=False,
    offload=False,
    offload_ops=(),
    patch_zero_bubble=False,
    enable_zero_bubble=False,
    mxfp4_gradient_stochastic_rounding=False,
)

_args = SimpleNamespace(**_DEFAULT_ARGS)
_num_microbatches = 1
_get_args_fn: Optional[Callable] = None
_get_num_microbatches_fn: Optional[Callable] = None


def bind(get_args: Optional[Callable] = None, get_num_microbatches: Optional[Callable] = None) -> None:
    """Route the getters to a host framework's own functions (None restores the local values)."""
    global _get_args_fn, _get_num_microbatches_fn
    _get_args_fn = get_args
    _get_num_microbatches_fn = get_num_microbatches


def default_args(**overrides) -> SimpleNamespace:
    values = dict(_DEFAULT_ARGS)
    values.update(overrides)
    return SimpleNamespace(**values)


def set_args(args=None, **overrides) -> None:
    """Install an argument namespace (or the defaults plus ``overrides``)."""
    global _args
    if args is None:
        args = default_args(**overrides)
    else:
        for key, value in overrides.items():
            setattr(args, key, value)
    _args = args


def get_args():
    return _get_args_fn() if _get_args_fn is not None else _args


def set_num_microbatches(n: int) -> None:
    global _num_microbatches
    if n < 1:
        raise ValueError("number of microbatches must be >= 1")
    _num_microbatches = int(n)


def get_num_microbatches() -> int:
    return _get_num_microbatches_fn() if _get_num_microbatches_fn is not None else _num_microbatches
