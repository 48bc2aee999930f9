"""Recipe names (primus/backends/megatron/core/enums.py:10-14 for FP4; the
FP8 names are Megatron's ``megatron.core.enums.Fp8Recipe`` as used at
primus/backends/megatron/core/fp8_utils.py:148-168).  ``str`` enums, so a
plain string from a YAML config compares equal."""

import enum


class Fp8Recipe(str, enum.Enum):
    delayed = "delayed"
    tensorwise = "tensorwise"
    mxfp8 = "mxfp8"
    blockwise = "blockwise"
    custom = "custom"


class Fp4Recipe(str, enum.Enum):
    nvfp4 = "nvfp4"
    mxfp4 = "mxfp4"
    custom = "custom"
