"""MI355X-native MX (microscaling) low-precision linear path.

``primus_amd.pytorch`` mirrors the operator surface the reference's Megatron
modules import (``core``, ``ops``, ``kernels``); ``primus_amd.megatron`` holds
the host-side module / recipe logic that calls it.  All arithmetic runs in the
HIP extension behind ``include/mxlinear.h``.
"""

__version__ = "0.1.0"
