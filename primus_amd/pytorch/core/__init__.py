"""``core`` namespace of the operator surface (primus_turbo.py:48-82)."""

from . import low_precision, quantized_tensor  # noqa: F401
from .low_precision import (  # noqa: F401
    Float4QuantConfig,
    Float8QuantConfig,
    Format,
    MXScalingRecipe,
    ScaleDtype,
    ScaleMode,
    ScalingGranularity,
    ScalingRecipe,
    ScalingStrategy,
    check_fp8_support,
    check_mxfp4_support,
    check_mxfp8_support,
    float4_e2m1fn_x2,
    float8_e4m3,
    float8_e5m2,
)
from .quantized_tensor import QuantizedTensor, QuantizedTensorPair, create_quantized_weight  # noqa: F401
