"""Patches that install this path into Megatron-LM modules
(primus/backends/megatron/patches/turbo/fp8_patches.py:26-65,
fp4_patches.py:29-83, te_spec_provider_patches.py:36-104, utils.py:14-35).

A patch is ``(id, condition(ctx), apply(ctx))``.  ``apply_patches`` runs, in
priority order, every patch whose condition holds.  The targets are Megatron
modules, imported only inside ``apply`` -- without Megatron installed the
conditions and the gating can still be evaluated (and are tested), and
``apply_patches(..., targets=...)`` can patch stand-in module objects."""

from __future__ import annotations

import importlib
import importlib.util
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

_FP_CONTEXT_TARGETS = (
    "megatron.core.transformer.transformer_block",
    "megatron.core.ssm.mamba_block",
    "megatron.core.transformer.multi_token_prediction",
)
_SPEC_PROVIDER_TARGETS = (
    "megatron.core.extensions.transformer_engine_spec_provider",
    "megatron.core.models.gpt.gpt_layer_specs",
    "megatron.core.models.gpt.moe_module_specs",
    "megatron.core.transformer.multi_token_prediction",
)


@dataclass
class PatchContext:
    args: object
    backend: str = "megatron"
    phase: str = "before_train"
    # module path -> module object; lets a caller (or a test) supply the objects to patch
    targets: Dict[str, object] = field(default_factory=dict)
    log: List[str] = field(default_factory=list)

    def module(self, path: str):
        if path in self.targets:
            return self.targets[path]
        return importlib.import_module(path)


@dataclass
class _Patch:
    patch_id: str
    condition: Callable[[PatchContext], bool]
    apply: Callable[[PatchContext], None]
    priority: int = 50
    description: str = ""


_REGISTRY: List[_Patch] = []


def register_patch(patch_id: str, *, condition: Callable[[PatchContext], bool], priority: int = 50,
                   description: str = ""):
    def deco(fn):
        _REGISTRY.append(_Patch(patch_id, condition, fn, priority, description))
        return fn

    return deco


def registered_patches() -> List[str]:
    return [p.patch_id for p in sorted(_REGISTRY, key=lambda p: p.priority)]


def is_primus_turbo_can_patch(ctx: PatchContext, package: str = "primus_amd") -> bool:
    """Turbo patches apply when ``enable_primus_turbo`` is set and the kernel
    package can be found.  Tensor parallelism is deliberately not part of the
    gate: only the linear classes need TP = 1 and they check it themselves
    (utils.py:14-35)."""
    if not bool(getattr(ctx.args, "enable_primus_turbo", False)):
        return False
    if importlib.util.find_spec(package) is None:
        ctx.log.append(f"[Patch:megatron.turbo] {package} not found, use TE backend...")
        return False
    return True


def _fp8_can_patch(ctx: PatchContext) -> bool:
    return bool(getattr(ctx.args, "fp8", False)) and is_primus_turbo_can_patch(ctx)


def _fp4_enabled(ctx: PatchContext) -> bool:
    return bool(getattr(ctx.args, "fp4", False))


@register_patch(
    "megatron.fp8.context",
    condition=lambda ctx: _fp8_can_patch(ctx) and not getattr(ctx.args, "disable_fp8_context_patches", False),
    description="get_fp8_context -> the Primus-Turbo FP8 autocast",
)
def patch_fp8_context(ctx: PatchContext) -> None:
    from ..fp8_utils import get_fp8_context

    for path in _FP_CONTEXT_TARGETS + ("megatron.core.fp8_utils",):
        ctx.module(path).get_fp8_context = get_fp8_context
        ctx.log.append(f"[Patch:megatron.fp8.context] patched {path}.get_fp8_context")


@register_patch("megatron.core.enums", condition=_fp4_enabled, description="Fp4Recipe with the mxfp4 member")
def patch_enums(ctx: PatchContext) -> None:
    from ..enums import Fp4Recipe

    ctx.module("megatron.core.enums").Fp4Recipe = Fp4Recipe
    ctx.log.append("[Patch:megatron.core.enums] patched megatron.core.enums.Fp4Recipe")


@register_patch("megatron.core.fp4_utils", condition=_fp4_enabled,
                description="get_fp4_context -> the Primus-Turbo FP4 autocast")
def patch_fp4_context(ctx: PatchContext) -> None:
    from ..fp4_utils import get_fp4_context

    for path in _FP_CONTEXT_TARGETS + ("megatron.core.fp4_utils",):
        ctx.module(path).get_fp4_context = get_fp4_context
        ctx.log.append(f"[Patch:megatron.fp4.context] patched {path}.get_fp4_context")


def _needs_primus_spec_provider(ctx: PatchContext) -> bool:
    if bool(getattr(ctx.args, "moe_use_legacy_grouped_gemm", False)):
        return True
    return is_primus_turbo_can_patch(ctx)


@register_patch("megatron.turbo.te_spec_provider", condition=_needs_primus_spec_provider, priority=41,
                description="TESpecProvider -> PrimusTurboSpecProvider")
def patch_te_spec_provider(ctx: PatchContext) -> None:
    from ..extensions.transformer_engine_spec_provider import PrimusTurboSpecProvider

    for path in _SPEC_PROVIDER_TARGETS:
        ctx.module(path).TESpecProvider = PrimusTurboSpecProvider
        ctx.log.append(f"[Patch:megatron.turbo.te_spec_provider] patched {path}.TESpecProvider")


def apply_patches(args, targets: Optional[Dict[str, object]] = None) -> PatchContext:
    """Apply every registered patch whose condition holds; returns the context
    (``ctx.log`` lists what was done)."""
    ctx = PatchContext(args=args, targets=dict(targets or {}))
    for patch in sorted(_REGISTRY, key=lambda p: p.priority):
        if patch.condition(ctx):
            patch.apply(ctx)
    return ctx
