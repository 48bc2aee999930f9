"""Expert MLP over grouped GEMMs: fc1 -> activation (x router probability) ->
fc2 (primus/backends/megatron/core/transformer/experts.py:24-268).

Tokens arrive permuted so that each local expert's rows are contiguous;
``tokens_per_expert`` stays on the device.  Whether rows are padded per expert
before quantisation is the reference's policy (:54-60): never when the router
already padded, never when the grouped GEMM takes ragged groups
(``turbo_grouped_gemm_without_padding``), otherwise yes -- and that fallback
costs a device-to-host read of ``tokens_per_expert`` (:196-209)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch
import torch.nn.functional as F

from .. import runtime
from ..extensions.primus_turbo import (
    PrimusTurboGroupedLinear,
    PrimusTurboColumnParallelGroupedLinear,
    PrimusTurboRowParallelGroupedLinear,
)


@dataclass
class GroupedMLPSubmodules:
    """Which classes implement fc1 and fc2 (Megatron's ``TEGroupedMLPSubmodules``)."""

    linear_fc1: type = PrimusTurboColumnParallelGroupedLinear
    linear_fc2: type = PrimusTurboRowParallelGroupedLinear


def get_align_size_for_quantization(config) -> int:
    """Rows per expert are padded to a multiple of this before quantisation:
    32 for the MX recipes (one scale block), 16 for the other FP8 recipes."""
    if getattr(config, "fp4", None):
        return 32
    if getattr(config, "fp8", None):
        return 32 if getattr(config, "fp8_recipe", None) == "mxfp8" else 16
    return 16


class PrimusGroupedMLP(torch.nn.Module):
    def __init__(self, num_local_experts: int, config, submodules: Optional[GroupedMLPSubmodules] = None,
                 pg_collection=None):
        super().__init__()
        args = runtime.get_args()
        submodules = submodules or GroupedMLPSubmodules()
        self.config = config
        self.num_local_experts = int(num_local_experts)
        self.input_size = int(config.hidden_size)
        ffn = int(getattr(config, "moe_ffn_hidden_size", None) or config.ffn_hidden_size)
        self.gated = bool(getattr(config, "gated_linear_unit", False))
        self.activation_func: Callable = getattr(config, "activation_func", F.silu if self.gated else F.gelu)
        init = getattr(config, "init_method", None)
        out_init = getattr(config, "output_layer_init_method", None) or init
        add_bias = bool(getattr(config, "add_bias_linear", False))
        self.linear_fc1 = submodules.linear_fc1(
            self.num_local_experts, self.input_size, ffn * (2 if self.gated else 1), config=config,
            init_method=init, bias=add_bias, skip_bias_add=False, is_expert=True, tp_comm_buffer_name="fc1",
            pg_collection=pg_collection,
        )
        self.linear_fc2 = submodules.linear_fc2(
            self.num_local_experts, ffn, self.input_size, config=config, init_method=out_init, bias=add_bias,
            skip_bias_add=True, is_expert=True, tp_comm_buffer_name="fc2", pg_collection=pg_collection,
        )
        # use_turbo_fused_act_with_probs has priority over the other activation fusions (experts.py:46-48)
        self.use_turbo_fused_act_with_probs = bool(getattr(args, "use_turbo_fused_act_with_probs", False))
        self.moe_router_padding_for_quantization = bool(getattr(args, "moe_router_padding_for_quantization", False))
        self.turbo_grouped_gemm_without_padding = bool(getattr(args, "turbo_grouped_gemm_without_padding", False))
        # with the fused activation, fc2 can take fc1's output directly and apply the activation inside its
        # quantiser (same values; the activated tensor is never stored).  Not a reference flag: default on.
        self.fuse_act_into_fc2 = bool(getattr(args, "turbo_fuse_act_into_fc2_quantize", True))

    # -- padding policy (experts.py:54-60) ------------------------------------
    def _use_explicit_quantization_padding(self) -> bool:
        """Whether this forward must pad expert groups before quantization."""
        if not (self.config.fp8 or self.config.fp4):
            return False
        if self.moe_router_padding_for_quantization:
            return False
        return not self.turbo_grouped_gemm_without_padding

    def quantization_padding(self, hidden: torch.Tensor, tokens_per_expert: List[int]):
        """Zero rows appended to every expert's segment up to the alignment."""
        align = get_align_size_for_quantization(self.config)
        padded = [(n + align - 1) // align * align for n in tokens_per_expert]
        pieces = []
        for seg, n, m in zip(torch.split(hidden, tokens_per_expert, dim=0), tokens_per_expert, padded):
            pieces.append(seg)
            if m > n:
                pieces.append(seg.new_zeros((m - n,) + tuple(seg.shape[1:])))
        return torch.cat(pieces, dim=0), padded

    def quantization_unpadding(self, hidden: torch.Tensor, tokens_per_expert: List[int]) -> torch.Tensor:
        align = get_align_size_for_quantization(self.config)
        padded = [(n + align - 1) // align * align for n in tokens_per_expert]
        kept = [seg[:n] for seg, n in zip(torch.split(hidden, padded, dim=0), tokens_per_expert)]
        return torch.cat(kept, dim=0)

    # -- activation (experts.py:62-118, the unfused branch) ---------------------
    def bias_act_func(self, intermediate, bias, permuted_probs):
        if bias is not None:
            intermediate = intermediate + bias
        if self.gated:
            glu, linear = torch.chunk(intermediate, 2, dim=-1)
            clamp = getattr(self.config, "activation_func_clamp_value", None)
            if clamp is not None:
                glu = glu.clamp(min=None, max=clamp)
                linear = linear.clamp(min=-clamp, max=clamp)
            intermediate = self.activation_func(glu) * (linear + getattr(self.config, "glu_linear_offset", 0.0))
        else:
            intermediate = self.activation_func(intermediate)
        dtype = intermediate.dtype
        return (intermediate * permuted_probs).to(dtype)

    def bias_act_func_with_mask(self, intermediate, bias, permuted_probs, tokens_per_experts=None):
        """experts.py:120-165: the fused kernel when ``use_turbo_fused_act_with_probs`` is set (gated
        SiLU / GELU only, no clamp, no linear offset), else the unfused arithmetic."""
        if not self.use_turbo_fused_act_with_probs:
            return self.bias_act_func(intermediate, bias, permuted_probs)
        from ..extensions.primus_turbo import fused_bias_act_with_probs

        assert tokens_per_experts is not None, (
            "tokens_per_experts is required when `use_turbo_fused_act_with_probs` is True."
        )
        assert getattr(self.config, "activation_func_clamp_value", None) is None, (
            "`use_turbo_fused_act_with_probs` does not support activation_func_clamp_value."
        )
        assert getattr(self.config, "glu_linear_offset", 0.0) == 0.0, (
            "`use_turbo_fused_act_with_probs` does not support a non-zero glu_linear_offset."
        )
        assert not getattr(self.config, "activation_func_fp8_input_store", False), (
            "`use_turbo_fused_act_with_probs` does not support activation_func_fp8_input_store."
        )
        activation = self._fused_activation_name()
        # forward() hands the probabilities over as [tokens, 1]; the kernel takes them 1-D
        probs_1d = permuted_probs.squeeze(-1) if permuted_probs.dim() == 2 else permuted_probs
        return fused_bias_act_with_probs(intermediate, bias, probs_1d, tokens_per_experts, activation)

    def _fused_activation_name(self) -> str:
        if self.activation_func == F.silu and self.gated:
            return "silu"
        if self.activation_func == F.gelu and self.gated:
            return "gelu"
        raise ValueError(
            "Only support fusion of swiglu and gelu in PrimusGroupedMLP when `use_turbo_fused_act_with_probs` is True."
        )

    def _can_fuse_act_into_fc2(self, bias) -> bool:
        """fc2 applies the activation in its own quantiser: needs the fused-activation flag, no fc1
        bias, none of the options the fused kernel rejects, and an fc2 that takes the prologue."""
        cfg = self.config
        return (self.use_turbo_fused_act_with_probs and self.fuse_act_into_fc2 and bias is None and self.gated
                and self.activation_func in (F.silu, F.gelu)
                and getattr(cfg, "activation_func_clamp_value", None) is None
                and getattr(cfg, "glu_linear_offset", 0.0) == 0.0
                and not getattr(cfg, "activation_func_fp8_input_store", False)
                and isinstance(self.linear_fc2, PrimusTurboGroupedLinear))

    def forward(self, permuted_local_hidden_states: torch.Tensor, tokens_per_expert: torch.Tensor,
                permuted_probs: torch.Tensor) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        pad = self._use_explicit_quantization_padding()
        on_device = pad and tokens_per_expert.is_cuda
        if on_device:
            # the counts stay on the device: both tensors go into buffers sized for the worst case, whose zero rows
            # behind the last expert's padding count as that expert's (no host read-back, unlike the reference)
            from ...pytorch import ops

            actual_rows = permuted_local_hidden_states.shape[0]
            actual = tokens_per_expert.to(torch.int64).contiguous()
            align = get_align_size_for_quantization(self.config)
            permuted_local_hidden_states, tokens_per_expert = ops.pad_groups(permuted_local_hidden_states, actual, align)
            permuted_probs, _ = ops.pad_groups(permuted_probs.unsqueeze(-1), actual, align)
        elif pad:
            # counts that already live on the host: the reference's sequence as it stands
            actual: List[int] = [int(v) for v in tokens_per_expert.tolist()]
            permuted_local_hidden_states, padded = self.quantization_padding(permuted_local_hidden_states, actual)
            permuted_probs, _ = self.quantization_padding(permuted_probs.unsqueeze(-1), actual)
            tokens_per_expert = torch.tensor(padded, device=permuted_local_hidden_states.device)
        else:
            permuted_probs = permuted_probs.unsqueeze(-1)

        if getattr(self.config, "moe_apply_probs_on_input", False):
            assert self.config.moe_router_topk == 1, "`moe_apply_probs_on_input` only works with `moe_router_topk`=1."
            dtype = permuted_local_hidden_states.dtype
            permuted_local_hidden_states = (permuted_probs * permuted_local_hidden_states).to(dtype)
            permuted_probs = torch.ones_like(permuted_probs)

        fc1_output, bias1 = self.linear_fc1(permuted_local_hidden_states, tokens_per_expert)
        if self._can_fuse_act_into_fc2(bias1):
            from ...pytorch import ops

            row_mask = ops.tokens_per_expert_to_mask(tokens_per_expert, fc1_output.shape[0])
            output, _ = self.linear_fc2(fc1_output, tokens_per_expert,
                                        glu=(permuted_probs.squeeze(-1), row_mask, self._fused_activation_name()))
        else:
            act = self.bias_act_func_with_mask(fc1_output, bias1, permuted_probs, tokens_per_expert)
            output, _ = self.linear_fc2(act, tokens_per_expert)
        if on_device:
            output = ops.unpad_groups(output, actual, align, actual_rows)
        elif pad:
            output = self.quantization_unpadding(output, actual)
        return output, None
