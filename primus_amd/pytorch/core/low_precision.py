"""Quantisation recipe objects of the low-precision linear path.

Mirrors the names the reference imports from
``primus_turbo.pytorch.core.low_precision``
(primus/backends/megatron/core/extensions/primus_turbo.py:57-82) and the way
it constructs them (:425-495, fp8_utils.py:162-168, fp4_utils.py:144-150).
Only the MX (microscaling) granularity has kernels here; the other enum
members exist so that recipe-selection code keeps working and are rejected,
with a clear error, where a kernel would be needed.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto
from typing import Optional, Tuple

import torch

from ... import _lib

# dtype aliases (primus_turbo.py:80-81)
float8_e4m3 = torch.float8_e4m3fn
float8_e5m2 = torch.float8_e5m2
float4_e2m1fn_x2 = torch.float4_e2m1fn_x2
float8_e8m0 = torch.float8_e8m0fnu

MX_BLOCK_SIZE = 32


class Format(Enum):
    E4M3 = auto()
    E5M2 = auto()
    HYBRID = auto()  # E4M3 forward, E5M2 gradients
    E2M1_X2 = auto()  # two FP4 values per byte


class ScaleDtype(Enum):
    FP32 = auto()
    E8M0 = auto()


class ScalingGranularity(Enum):
    TENSORWISE = auto()
    ROWWISE = auto()
    BLOCKWISE = auto()
    MX_BLOCKWISE = auto()


class ScalingStrategy(Enum):
    DYNAMIC = auto()


class ScaleMode(Enum):
    """How the E8M0 block scale is derived from the block's largest magnitude.

    The reference's kernel library is not part of its tree, so the rule is an
    explicit recipe field here: OCP MX v1.0 floor rule (default), round-up
    (``2^ceil(log2(amax / max_normal))``) and the AITER / Quark "even" rule
    (round amax to the element's mantissa width first)."""

    OCP_FLOOR = _lib.SCALE_OCP_FLOOR
    RCEIL = _lib.SCALE_RCEIL
    EVEN = _lib.SCALE_EVEN


@dataclass
class MXScalingRecipe:
    """Per-operand options of MX quantisation (primus_turbo.py:305-319)."""

    use_2d_block: bool = False  # one scale per 32x32 tile (weights)
    # Pre-shuffled scale / data layouts (primus_turbo.py:305-311).  In the reference they ask the quantiser for the
    # byte order its FP4 GEMM back end wants.  Here the storage of a QuantizedTensor is private to the library (its
    # GEMMs read the K-chunk-major layout the quantisers write directly), so the flags are accepted and change
    # nothing an operator computes; the pre-shuffled byte orders themselves are available through
    # ``QuantizedTensor.preshuffled_codes()`` / ``preshuffled_scales()`` and the flags of ``quantize_mxfp4_dual``.
    shuffle_scale: bool = False
    shuffle_out: bool = False
    scale_mode: ScaleMode = ScaleMode.OCP_FLOOR


# older name of the same class (primus_turbo.py:57-62)
ScalingRecipe = MXScalingRecipe


@dataclass
class Float8QuantConfig:
    format: Format = Format.E4M3
    granularity: ScalingGranularity = ScalingGranularity.TENSORWISE
    strategy: ScalingStrategy = ScalingStrategy.DYNAMIC
    scale_dtype: ScaleDtype = ScaleDtype.FP32
    block_size: Optional[int] = None
    scale_mode: ScaleMode = ScaleMode.OCP_FLOOR

    def __post_init__(self):
        if self.granularity == ScalingGranularity.MX_BLOCKWISE:
            if self.block_size is None:
                self.block_size = MX_BLOCK_SIZE
            if self.block_size != MX_BLOCK_SIZE:
                raise ValueError(f"MX block size must be {MX_BLOCK_SIZE}, got {self.block_size}")
            if self.scale_dtype != ScaleDtype.E8M0:
                raise ValueError("MX_BLOCKWISE requires scale_dtype=ScaleDtype.E8M0")


@dataclass
class Float4QuantConfig:
    format: Format = Format.E2M1_X2
    granularity: ScalingGranularity = ScalingGranularity.MX_BLOCKWISE
    strategy: ScalingStrategy = ScalingStrategy.DYNAMIC
    scale_dtype: ScaleDtype = ScaleDtype.E8M0
    block_size: Optional[int] = MX_BLOCK_SIZE
    use_gradient_sr: bool = False  # stochastic rounding of E2M1 gradients
    # Accepted for the reference's configs (primus_turbo.py:304-311): the operators already keep FP4 weights in the
    # layout their GEMM reads fastest, so the switch changes no result here (see MXScalingRecipe).
    use_preshuffle: bool = False
    scale_mode: ScaleMode = ScaleMode.OCP_FLOOR
    # Element format of activations and gradients.  E2M1_X2 is plain MXFP4;
    # E4M3 gives MXFP4 weights with MXFP8 activations (GPT-OSS style).
    activation_format: Format = Format.E2M1_X2
    # Randomised Hadamard transform (16 tokens) of the transposed copies of activations and gradients,
    # i.e. of both wgrad operands: None = off, else the 16 sign bits.  E2M1 activations only.
    colwise_rht_signs: Optional[int] = None

    def __post_init__(self):
        if self.format != Format.E2M1_X2:
            raise ValueError("Float4QuantConfig only supports Format.E2M1_X2")
        if self.granularity != ScalingGranularity.MX_BLOCKWISE or self.scale_dtype != ScaleDtype.E8M0:
            raise ValueError("FP4 requires MX_BLOCKWISE granularity with E8M0 scales")
        if self.block_size is None:
            self.block_size = MX_BLOCK_SIZE
        if self.block_size != MX_BLOCK_SIZE:
            raise ValueError(f"MX block size must be {MX_BLOCK_SIZE}, got {self.block_size}")
        if self.activation_format not in (Format.E2M1_X2, Format.E4M3):
            raise ValueError("activation_format must be E2M1_X2 or E4M3")


def _gfx950_reason() -> Tuple[bool, str]:
    if not torch.cuda.is_available():
        return False, "no GPU is visible to PyTorch"
    name = torch.cuda.get_device_properties(torch.cuda.current_device()).gcnArchName
    if "gfx950" not in name:
        return False, f"the MX kernels are built for gfx950 only, found {name}"
    try:
        _lib.load()
    except Exception as exc:  # missing or unloadable extension
        return False, str(exc)
    return True, ""


def check_fp8_support() -> Tuple[bool, str]:
    """(available, reason) like the reference's probe (primus_turbo.py:549-550)."""
    return _gfx950_reason()


def check_mxfp8_support() -> Tuple[bool, str]:
    return _gfx950_reason()


def check_mxfp4_support() -> Tuple[bool, str]:
    return _gfx950_reason()


def fmt_code(fmt: Format) -> int:
    """Element-format enum of the C ABI for a recipe format."""
    if fmt in (Format.E4M3, Format.HYBRID):
        # the MX recipe of the reference is E4M3 for every operand (primus_turbo.py:481-487)
        return _lib.FMT_E4M3
    if fmt == Format.E2M1_X2:
        return _lib.FMT_E2M1
    raise ValueError(f"no MX kernel for element format {fmt}")


def dtype_to_fmt_code(dtype: torch.dtype) -> int:
    if dtype == float8_e4m3:
        return _lib.FMT_E4M3
    if dtype == float4_e2m1fn_x2:
        return _lib.FMT_E2M1
    if dtype == float8_e5m2:
        return _lib.FMT_E5M2
    raise ValueError(f"no MX kernel for dest_dtype {dtype}")


def fmt_code_to_dtype(code: int) -> torch.dtype:
    return {_lib.FMT_E4M3: float8_e4m3, _lib.FMT_E2M1: float4_e2m1fn_x2, _lib.FMT_E5M2: float8_e5m2}[code]
