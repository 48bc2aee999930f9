"""Host-side logic of the MX linear path as the reference wires it into
Megatron-LM (primus/backends/megatron/...): recipe selection, autocast state,
cached quantised weights, the linear / grouped-linear / grouped-MLP modules,
spec-provider selection, patch gating and argument validation.

Megatron-LM and Transformer Engine are not dependencies: the modules here are
plain ``torch.nn.Module`` classes with Megatron's constructor and forward
conventions (``[s, b, h]`` activations, ``(output, bias)`` return pairs,
``main_grad`` gradient accumulation), and the two Megatron globals the
reference reads (``get_args`` and ``get_num_microbatches``) are provided by
``runtime`` and can be pointed at Megatron's own.
"""

from . import enums, runtime  # noqa: F401
