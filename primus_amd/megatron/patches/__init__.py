"""Installation of the Primus-Turbo classes into a host framework and the
argument checks that go with it."""

from .args import validate_args_on_rocm, validate_turbo_grouped_gemm_without_padding  # noqa: F401
from .turbo import (  # noqa: F401
    PatchContext,
    apply_patches,
    is_primus_turbo_can_patch,
    registered_patches,
)
