"""Environment variable names the reference publishes its backend choice into
(primus/backends/megatron/core/extensions/primus_turbo.py:69,104-122).
This implementation has exactly one backend (hand-written gfx950 kernels); the
variables are accepted and ignored."""

ENV_GEMM_BACKEND = "PRIMUS_TURBO_GEMM_BACKEND"
ENV_GROUPED_GEMM_BACKEND = "PRIMUS_TURBO_GROUPED_GEMM_BACKEND"
ENV_AUTO_TUNE = "PRIMUS_TURBO_AUTO_TUNE"
