"""Argument validation of the low-precision path on ROCm
(primus/backends/megatron/patches/args/rocm_arg_validation.py:100-108,142-178)."""

from __future__ import annotations

import os

SUPPORTED_FP8_RECIPES = ("tensorwise", "blockwise", "mxfp8")
SUPPORTED_FP4_RECIPES = ("mxfp4",)


def validate_turbo_grouped_gemm_without_padding(args) -> None:
    """The ragged (no padding) grouped-GEMM path needs the Turbo grouped GEMM
    and must not be combined with router-side padding."""
    option = "turbo_grouped_gemm_without_padding"
    if not getattr(args, option, False):
        return
    if not getattr(args, "enable_primus_turbo", False) or not getattr(args, "use_turbo_grouped_gemm", False):
        raise ValueError(f"{option}=True requires enable_primus_turbo=True and use_turbo_grouped_gemm=True.")
    if getattr(args, "moe_router_padding_for_quantization", False):
        raise ValueError(f"{option}=True requires moe_router_padding_for_quantization=False.")


def validate_args_on_rocm(args) -> None:
    """The FP8 / FP4 part of the reference's validation."""
    assert not getattr(args, "use_turbo_parallel_linear", False), (
        "use_turbo_parallel_linear has been removed; please use use_turbo_gemm instead."
    )
    use_turbo_gemm = getattr(args, "use_turbo_gemm", False)
    if getattr(args, "fp8", None) and use_turbo_gemm:
        assert args.fp8_recipe in SUPPORTED_FP8_RECIPES, (
            f"{args.fp8_recipe} recipe is not support when enable `use_turbo_gemm`."
        )
    if getattr(args, "fp4", None) and use_turbo_gemm:
        assert args.fp4_recipe in SUPPORTED_FP4_RECIPES, (
            f"{args.fp4_recipe} recipe is not support when enable `use_turbo_gemm`."
        )
    if (
        getattr(args, "fp4", None)
        and use_turbo_gemm
        and getattr(args, "fp4_use_native_te_autocast", False)
        and getattr(args, "transformer_impl", "transformer_engine") != "local"
    ):
        raise ValueError(
            "fp4_use_native_te_autocast=True is incompatible with use_turbo_gemm=True: the native autocast does "
            "not set the Primus-Turbo FP4 state the Turbo linears read, so they would silently run in BF16. "
            "Set use_turbo_gemm=false or fp4_use_native_te_autocast=false."
        )
    if getattr(args, "fp8_recipe", None) == "mxfp8":
        assert os.getenv("NVTE_ROCM_ENABLE_MXFP8", "0") == "1", (
            "Please set `NVTE_ROCM_ENABLE_MXFP8=1` to enable `mxfp8` recipe."
        )
    validate_turbo_grouped_gemm_without_padding(args)
