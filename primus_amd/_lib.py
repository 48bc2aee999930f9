"""ctypes binding of the C-ABI extension (include/mxlinear.h).

The extension is the only compute path: if the shared library is missing or a
call fails, an exception is raised -- there is no CPU or PyTorch fallback.
"""

from __future__ import annotations

import ctypes
import os
import threading

from . import build as _build

_lock = threading.Lock()
_lib = None

FMT_E4M3 = 0
FMT_E2M1 = 1
FMT_E5M2 = 2   # tensor-wise scaled operands only
SCALE_OCP_FLOOR = 0
SCALE_RCEIL = 1
SCALE_EVEN = 2
BLOCK = 32
SEG_ALIGN = 128
GEMM_K_ALIGN = 128  # the GEMM kernels take the contraction dim in multiples of this
MAX_GROUPS = 1024
ACT_SILU, ACT_GELU = 0, 1
PROBS_F32, PROBS_BF16 = 0, 1
QF_SR, QF_RHT_COL, QF_KCHUNK, QF_KSTEP, QF_KSTEP128 = 1, 2, 4, 8, 16   # flags of mxl_quantize_ex
GF_KCHUNK = 1                               # flag of the GEMM _ex entry points: operands are K-chunk-major
GF_KSTEP = 4                                # ... K-step-major codes and scales (ring kernel)
GF_ACCUM_F32 = 2                            # wgrad: the output is float32 and the result is added to it
GF_B_SHUFFLED = 16                          # forward / dgrad, row-major E2M1: b's codes are in the pre-shuffled byte order
GF_B_TRANSPOSED = 8                         # forward / dgrad: b's codes are those of the transposed matrices (row-wise weight copy)
BF_B_KN, BF_ACCUM_F32, BF_TILE_128, BF_TILE_256 = 1, 2, 4, 8    # flags of the bf16 grouped GEMMs

EXPORTS = (
    "mxl_version",
    "mxl_error_string",
    "mxl_padded_width",
    "mxl_quantize",
    "mxl_quantize_ex",
    "mxl_quantize_weight_2d_ex",
    "mxl_quantize_weight_2d",
    "mxl_dequantize",
    "mxl_gemm_nt",
    "mxl_grouped_gemm_nt",
    "mxl_grouped_gemm_wgrad",
    "mxl_grouped_gemm_nt_ex",
    "mxl_grouped_gemm_wgrad_ex",
    "mxl_grouped_gemm_bf16",
    "mxl_grouped_gemm_bf16_wgrad",
    "mxl_glu_probs_fwd",
    "mxl_glu_probs_bwd",
    "mxl_glu_probs_quantize",
    "mxl_rmsnorm_fwd",
    "mxl_rmsnorm_bwd",
    "mxl_rmsnorm_bwd_workspace_bytes",
    "mxl_rmsnorm_bwd_noalloc",
    "mxl_rmsnorm_bwd_noalloc_max_bytes",
    "mxl_rmsnorm_bwd_noalloc_bind",
    "mxl_rmsnorm_quantize",
    "mxl_amax",
    "mxl_quantize_tensorwise",
    "mxl_quantize_weight_tensorwise",
    "mxl_grouped_gemm_nt_scaled",
    "mxl_grouped_gemm_wgrad_scaled",
    "mxl_padded_rows_bound",
    "mxl_pad_groups",
    "mxl_unpad_groups",
    "mxl_quantize_blockwise",
    "mxl_quantize_blockwise_weight",
    "mxl_gemm_nt_blockwise",
    "mxl_grouped_gemm_nt_blockwise",
    "mxl_grouped_gemm_wgrad_blockwise",
    "mxl_blockwise_gemm_tile",
    "mxl_blockwise_gemm_plan",
    "mxl_shuffle_codes",
    "mxl_shuffle_scales",
    "mxl_calibrate_mfma",
    "mxl_calibrate_mfma_flops",
    "mxl_calibrate_mfma_bf16",
    "mxl_calibrate_mfma_bf16_flops",
    "mxl_calibrate_tile_copy",
    "mxl_calibrate_range_check",
)


class MXLinearError(RuntimeError):
    pass


def lib_path() -> str:
    """The in-tree library, or the one ``MXL_LIBRARY`` names (an alternative build of the same ABI)."""
    return os.environ.get("MXL_LIBRARY") or _build.LIB_PATH


def load() -> ctypes.CDLL:
    """Load libmxlinear.so (built in-tree by ``primus_amd.build``)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = lib_path()
        if not os.path.exists(path):
            raise MXLinearError(
                f"{path} is missing: build the HIP extension first (python -m primus_amd.build). "
                "The MX linear path has no fallback implementation."
            )
        lib = ctypes.CDLL(path)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        lib.mxl_version.restype = i32
        lib.mxl_error_string.restype = ctypes.c_char_p
        lib.mxl_error_string.argtypes = [i32]
        lib.mxl_padded_width.restype = i64
        lib.mxl_padded_width.argtypes = [i64, i32]
        lib.mxl_quantize.restype = i32
        lib.mxl_quantize.argtypes = [vp, i64, i64, i64, i32, i32, vp, i32, vp, vp, vp, vp, vp]
        u32 = ctypes.c_uint32
        lib.mxl_quantize_ex.restype = i32
        lib.mxl_quantize_ex.argtypes = [vp, i64, i64, i64, i32, i32, vp, i32, vp, vp, vp, vp, u32, ctypes.c_uint64, u32, vp]
        lib.mxl_quantize_weight_2d_ex.restype = i32
        lib.mxl_quantize_weight_2d_ex.argtypes = [vp, i64, i64, i64, i64, i64, i32, i32, vp, vp, vp, vp, u32, vp]
        lib.mxl_quantize_weight_2d.restype = i32
        lib.mxl_quantize_weight_2d.argtypes = [vp, i64, i64, i64, i64, i64, i32, i32, vp, vp, vp, vp, vp]
        lib.mxl_dequantize.restype = i32
        lib.mxl_dequantize.argtypes = [vp, vp, i64, i64, i32, vp, vp]
        lib.mxl_gemm_nt.restype = i32
        lib.mxl_gemm_nt.argtypes = [vp, vp, i32, vp, vp, i32, vp, i64, i64, i64, vp]
        lib.mxl_grouped_gemm_nt_ex.restype = i32
        lib.mxl_grouped_gemm_nt_ex.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, ctypes.c_uint32, vp]
        lib.mxl_grouped_gemm_wgrad_ex.restype = i32
        lib.mxl_grouped_gemm_wgrad_ex.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, ctypes.c_uint32, vp]
        lib.mxl_grouped_gemm_nt.restype = i32
        lib.mxl_grouped_gemm_nt.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp]
        lib.mxl_grouped_gemm_wgrad.restype = i32
        lib.mxl_grouped_gemm_wgrad.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp]
        lib.mxl_grouped_gemm_bf16.restype = i32
        lib.mxl_grouped_gemm_bf16.argtypes = [vp, vp, vp, vp, i32, i64, i64, i64, u32, vp]
        lib.mxl_grouped_gemm_bf16_wgrad.restype = i32
        lib.mxl_grouped_gemm_bf16_wgrad.argtypes = [vp, vp, vp, vp, i32, i64, i64, i64, u32, vp]
        lib.mxl_glu_probs_fwd.restype = i32
        lib.mxl_glu_probs_fwd.argtypes = [vp, vp, i32, vp, i64, i64, i32, vp, vp]
        lib.mxl_glu_probs_bwd.restype = i32
        lib.mxl_glu_probs_bwd.argtypes = [vp, vp, vp, i32, vp, i64, i64, i32, vp, vp, vp]
        lib.mxl_glu_probs_quantize.restype = i32
        lib.mxl_glu_probs_quantize.argtypes = [vp, vp, i32, vp, i64, i64, i64, i32, i32, i32, vp, i32, vp, vp, vp, vp,
                                               ctypes.c_uint32, vp]
        lib.mxl_rmsnorm_fwd.restype = i32
        lib.mxl_rmsnorm_fwd.argtypes = [vp, vp, ctypes.c_float, i64, i64, vp, vp, vp]
        lib.mxl_rmsnorm_bwd_workspace_bytes.restype = i64
        lib.mxl_rmsnorm_bwd_workspace_bytes.argtypes = [i64, i64]
        lib.mxl_rmsnorm_bwd.restype = i32
        lib.mxl_rmsnorm_bwd.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, i64, vp]
        lib.mxl_rmsnorm_bwd_noalloc.restype = i32
        lib.mxl_rmsnorm_bwd_noalloc.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp]
        lib.mxl_rmsnorm_bwd_noalloc_max_bytes.restype = i64
        lib.mxl_rmsnorm_bwd_noalloc_max_bytes.argtypes = []
        lib.mxl_rmsnorm_bwd_noalloc_bind.restype = i32
        lib.mxl_rmsnorm_bwd_noalloc_bind.argtypes = [vp]
        lib.mxl_rmsnorm_quantize.restype = i32
        lib.mxl_rmsnorm_quantize.argtypes = [vp, vp, vp, i64, i64, i64, i32, i32, vp, i32, vp, vp, vp, vp, u32, vp]
        lib.mxl_amax.restype = i32
        lib.mxl_amax.argtypes = [vp, i64, vp, vp]
        lib.mxl_quantize_tensorwise.restype = i32
        lib.mxl_quantize_tensorwise.argtypes = [vp, i64, i64, i64, i32, vp, vp, i32, vp, vp, vp, vp, vp, u32, vp]
        lib.mxl_quantize_weight_tensorwise.restype = i32
        lib.mxl_quantize_weight_tensorwise.argtypes = [vp, i64, i64, i64, i64, i64, i32, vp, vp, vp, vp, vp, vp, u32, vp]
        lib.mxl_grouped_gemm_nt_scaled.restype = i32
        lib.mxl_grouped_gemm_nt_scaled.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp, vp, u32, vp]
        lib.mxl_grouped_gemm_wgrad_scaled.restype = i32
        lib.mxl_grouped_gemm_wgrad_scaled.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp, vp, u32, vp]
        lib.mxl_padded_rows_bound.restype = i64
        lib.mxl_padded_rows_bound.argtypes = [i64, i32, i32]
        lib.mxl_pad_groups.restype = i32
        lib.mxl_pad_groups.argtypes = [vp, i64, i64, vp, i32, i32, vp, i64, vp, vp]
        lib.mxl_unpad_groups.restype = i32
        lib.mxl_unpad_groups.argtypes = [vp, i64, i64, vp, i32, i32, vp, i64, vp]
        lib.mxl_quantize_blockwise.restype = i32
        lib.mxl_quantize_blockwise.argtypes = [vp, i64, i64, i32, vp, i32, vp, vp, vp, vp, vp]
        lib.mxl_quantize_blockwise_weight.restype = i32
        lib.mxl_quantize_blockwise_weight.argtypes = [vp, i64, i64, i64, i32, vp, vp, vp, vp, vp]
        lib.mxl_grouped_gemm_nt_blockwise.restype = i32
        lib.mxl_grouped_gemm_nt_blockwise.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp]
        lib.mxl_grouped_gemm_wgrad_blockwise.restype = i32
        lib.mxl_grouped_gemm_wgrad_blockwise.argtypes = [vp, vp, i32, vp, vp, i32, vp, vp, i32, i64, i64, i64, vp]
        lib.mxl_shuffle_codes.restype = i32
        lib.mxl_shuffle_codes.argtypes = [vp, i64, i64, vp, i32, vp]
        lib.mxl_shuffle_scales.restype = i32
        lib.mxl_shuffle_scales.argtypes = [vp, i64, i64, vp, i32, vp]
        lib.mxl_calibrate_mfma.restype = i32
        lib.mxl_calibrate_mfma.argtypes = [i32, i32, i64, vp]
        lib.mxl_calibrate_tile_copy.restype = i32
        lib.mxl_calibrate_tile_copy.argtypes = [vp, i64, i64, vp, vp, vp]
        lib.mxl_calibrate_range_check.restype = i32
        lib.mxl_calibrate_range_check.argtypes = [vp, i64, vp, i32, vp, i64, vp]
        lib.mxl_calibrate_mfma_flops.restype = i64
        lib.mxl_calibrate_mfma_flops.argtypes = [i64]
        lib.mxl_calibrate_mfma_bf16.restype = i32
        lib.mxl_calibrate_mfma_bf16.argtypes = [i64, vp]
        lib.mxl_calibrate_mfma_bf16_flops.restype = i64
        lib.mxl_calibrate_mfma_bf16_flops.argtypes = [i64]
        lib.mxl_gemm_nt_blockwise.restype = i32
        lib.mxl_gemm_nt_blockwise.argtypes = [vp, vp, i32, vp, vp, i32, i32, vp, i64, i64, i64, vp]
        lib.mxl_blockwise_gemm_tile.restype = i32
        lib.mxl_blockwise_gemm_tile.argtypes = [i32]
        lib.mxl_blockwise_gemm_plan.restype = i32
        lib.mxl_blockwise_gemm_plan.argtypes = [i64, i64, i32, i32, vp, vp]
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mxl_error_string(rc).decode()
        raise MXLinearError(f"{what} failed: {msg} (code {rc})")


def padded_width(total_rows: int, num_groups: int) -> int:
    return int(load().mxl_padded_width(int(total_rows), int(num_groups)))
