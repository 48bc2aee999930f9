"""The C-ABI library: loads, exports every symbol include/mxlinear.h declares, and its host-only
entry points answer (no kernel is launched here)."""

import ctypes
import os
import re

import pytest

from oracle import mx_oracle as o
from primus_amd import _lib, build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mxlinear.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.lib_path()):
        build.build()   # hipcc cross-compiles without a GPU
    return _lib.load()


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mxl_\w+)\s*\(", text)))


def test_header_and_loader_agree():
    assert _declared() == sorted(_lib.EXPORTS)


def test_every_declared_symbol_is_exported(lib):
    raw = ctypes.CDLL(_lib.lib_path())
    for name in _declared():
        assert hasattr(raw, name), name


def test_host_only_entry_points(lib):
    assert lib.mxl_version() >= 1
    for code in (0, -1, -2, -3, -99):
        assert lib.mxl_error_string(code).decode()
    for rows, groups in [(0, 0), (1, 1), (128, 1), (129, 1), (32768, 8), (65536, 128), (5, 0)]:
        assert _lib.padded_width(rows, groups) == o.padded_width(rows, groups)
    # the calibration loop: 256 workgroups x 4 waves x iters x 16 MFMAs of 2 * 32 * 32 * 64 flops
    assert lib.mxl_calibrate_mfma_flops(1) == 256 * 4 * 16 * 2 * 32 * 32 * 64
    assert lib.mxl_calibrate_mfma_flops(4096) == 4096 * lib.mxl_calibrate_mfma_flops(1)
    assert lib.mxl_calibrate_mfma_flops(-1) == -1
    assert lib.mxl_calibrate_mfma(_lib.FMT_E4M3, _lib.FMT_E4M3, 0, None) == -1      # no iterations
    assert lib.mxl_calibrate_mfma(7, _lib.FMT_E4M3, 16, None) == -1                 # unknown format
    assert lib.mxl_calibrate_tile_copy(None, 128, 128, None, None, None) == -1      # no input
    assert lib.mxl_calibrate_tile_copy(ctypes.c_void_p(4096), 100, 128, None, None, None) == -1   # rows % 128


def test_constants_match_the_header():
    text = open(HEADER).read()
    defs = dict(re.findall(r"#define\s+(MXL_\w+)\s+\(?(-?\d+)u?\)?", text))
    assert int(defs["MXL_BLOCK"]) == _lib.BLOCK == o.BLOCK
    assert int(defs["MXL_SEG_ALIGN"]) == _lib.SEG_ALIGN == o.SEG_ALIGN
    assert int(defs["MXL_MAX_GROUPS"]) == _lib.MAX_GROUPS
    assert (int(defs["MXL_FMT_E4M3"]), int(defs["MXL_FMT_E2M1"])) == (_lib.FMT_E4M3, _lib.FMT_E2M1) == (o.FMT_E4M3, o.FMT_E2M1)
    assert (int(defs["MXL_SCALE_OCP_FLOOR"]), int(defs["MXL_SCALE_RCEIL"]), int(defs["MXL_SCALE_EVEN"])) == (
        o.SCALE_OCP_FLOOR, o.SCALE_RCEIL, o.SCALE_EVEN)
    assert (int(defs["MXL_ACT_SILU"]), int(defs["MXL_ACT_GELU"])) == (_lib.ACT_SILU, _lib.ACT_GELU)
    assert (int(defs["MXL_QF_SR"]), int(defs["MXL_QF_RHT_COL"]), int(defs["MXL_QF_KCHUNK"])) == (
        _lib.QF_SR, _lib.QF_RHT_COL, _lib.QF_KCHUNK)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "lib_path", lambda: str(tmp_path / "nope.so"))
    with pytest.raises(_lib.MXLinearError, match="no fallback"):
        _lib.load()


def test_without_a_gfx950_device_the_entry_points_refuse(lib):
    """On a machine without a GPU a well-formed call returns MXL_ENODEV before anything is launched
    (bad arguments are still reported as such first)."""
    import torch

    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present: this call would be a real launch")
    buf = ctypes.create_string_buffer(128 * 128 * 2)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.mxl_quantize(p, 128, 128, 128, _lib.FMT_E4M3, 0, None, 0, p, p, None, None, None) == -3
    assert lib.mxl_quantize(p, 128, 100, 128, _lib.FMT_E4M3, 0, None, 0, p, p, None, None, None) == -1   # cols % 32
    assert lib.mxl_gemm_nt(p, p, 0, p, p, 0, p, 128, 128, 128, None) == -3
    assert lib.mxl_gemm_nt(p, p, 0, p, p, 0, p, 128, 128, 100, None) == -1                                 # k % 128
    assert lib.mxl_glu_probs_fwd(p, p, 0, None, 4, 32, 0, p, None) == -3
    assert lib.mxl_error_string(-3).decode().startswith("device")


def test_newer_entry_points_validate_before_they_touch_the_device(lib):
    """RMSNorm, tensor-wise scaling and the accumulating wgrad: malformed calls are MXL_EINVAL (-1), well-formed ones
    MXL_ENODEV (-3) on a machine without a GPU."""
    import torch

    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present: the well-formed calls would be real launches")
    buf = ctypes.create_string_buffer(256 * 256 * 4)
    p = ctypes.cast(buf, ctypes.c_void_p)
    f32 = ctypes.c_float
    # RMSNorm
    assert lib.mxl_rmsnorm_fwd(p, p, f32(1e-5), 4, 256, p, p, None) == -3
    assert lib.mxl_rmsnorm_fwd(p, p, f32(1e-5), 4, 100, p, p, None) == -1            # k % 8
    assert lib.mxl_rmsnorm_fwd(p, p, f32(1e-5), 4, 32768, p, p, None) == -1          # k > 16384
    assert lib.mxl_rmsnorm_fwd(p, p, f32(-1.0), 4, 256, p, p, None) == -1            # eps < 0
    assert lib.mxl_rmsnorm_fwd(p, None, f32(1e-5), 4, 256, p, p, None) == -1         # y without a weight
    assert lib.mxl_rmsnorm_fwd(p, None, f32(1e-5), 0, 256, None, None, None) == 0    # no rows: nothing to do
    assert lib.mxl_rmsnorm_bwd_workspace_bytes(4, 256) == 4 * 256 * 4
    assert lib.mxl_rmsnorm_bwd_workspace_bytes(100000, 4096) == 1024 * 4096 * 4     # capped number of partial rows
    assert lib.mxl_rmsnorm_bwd_workspace_bytes(4, 100) == -1
    assert lib.mxl_rmsnorm_bwd(p, p, p, p, 4, 256, p, None, p, 4096, None) == -1     # no dw
    assert lib.mxl_rmsnorm_quantize(p, None, p, 4, 256, 256, 0, 0, None, 0, p, p, None, None, 0, None) == -1   # no weight
    assert lib.mxl_rmsnorm_quantize(p, p, p, 4, 256, 256, 0, 0, None, 0, p, p, None, None, 64, None) == -1     # unknown flag
    assert lib.mxl_rmsnorm_quantize(p, p, p, 4, 256, 256, 0, 0, None, 0, p, p, None, None, 0, None) == -3
    # tensor-wise scaling
    assert lib.mxl_amax(p, -1, p, None) == -1
    assert lib.mxl_amax(p, 64, None, None) == -1
    assert lib.mxl_amax(p, 64, p, None) == -3
    assert lib.mxl_quantize_tensorwise(p, 128, 128, 128, _lib.FMT_E2M1, p, None, 0, p, p, None, None, p, 0, None) == -1   # FP8 only
    assert lib.mxl_quantize_tensorwise(p, 128, 128, 128, _lib.FMT_E5M2, None, None, 0, p, p, None, None, p, 0, None) == -1  # no amax
    assert lib.mxl_quantize_tensorwise(p, 128, 128, 128, _lib.FMT_E5M2, p, None, 0, p, p, None, None, p, 0, None) == -3
    assert lib.mxl_quantize_weight_tensorwise(p, 1, 128, 128, 128, 128, 7, p, p, p, None, None, p, 0, None) == -1
    # scaled GEMMs and the accumulating wgrad
    assert lib.mxl_grouped_gemm_nt_scaled(p, p, 0, p, p, 0, p, None, 1, 128, 128, 128, None, p, 0, None) == -1    # one factor missing
    assert lib.mxl_grouped_gemm_nt_scaled(p, p, 0, p, p, 0, p, None, 1, 128, 128, 128, p, p, 0, None) == -3
    assert lib.mxl_grouped_gemm_nt_ex(p, p, _lib.FMT_E5M2, p, p, 0, p, None, 1, 128, 128, 128, 0, None) in (-1, -3)
    assert lib.mxl_grouped_gemm_wgrad_ex(p, p, 0, p, p, 0, p, None, 0, 128, 128, 128, _lib.GF_ACCUM_F32, None) == -1   # needs KCHUNK
    assert lib.mxl_grouped_gemm_wgrad_ex(p, p, 0, p, p, 0, p, None, 0, 128, 128, 128, 64, None) == -1                   # unknown flag
    assert lib.mxl_grouped_gemm_wgrad_ex(p, p, 0, p, p, 0, p, None, 0, 128, 128, 128, _lib.GF_ACCUM_F32 | _lib.GF_KCHUNK, None) == -3


def test_blockwise_gemm_plan(lib):
    """The tile-height choice of the blockwise GEMMs is a host calculation: the Llama-3-8B MLP's three GEMMs at 8192
    tokens, a problem too small for 256-row tiles, grouped shapes, the override and the argument checks."""
    def plan(m, n, mode=0, groups=0):
        rows, cols = ctypes.c_int64(-1), ctypes.c_int64(-1)
        rc = lib.mxl_blockwise_gemm_plan(m, n, mode, groups, ctypes.byref(rows), ctypes.byref(cols))
        return rc, rows.value, cols.value

    assert plan(8192, 14336) == (0, 8192, 14336)          # forward: 32 x 56 tiles = 7 rounds, all on 256-row tiles
    assert plan(8192, 4096) == (0, 8192, 4096)            # dgrad: 2 rounds
    assert plan(14336, 4096) == (0, 12288, 4096)          # wgrad of fc1: 3 whole rounds, the last 2048 rows on 128-row tiles
    assert plan(4096, 14336) == (0, 4096, 12288)          # wgrad of fc2: the last 8 column tiles
    assert plan(2048, 4096) == (0, 0, 0)                  # half a round of 256-row tiles: 128-row tiles fill the chip
    assert plan(1, 128) == (0, 0, 0)
    assert plan(32768, 28672, 1, 8) == (0, 32768, 28672)  # grouped forward, 4096 rows per group
    assert plan(4096, 1024, 1, 64) == (0, 0, 0)           # 64 rows per group: the ragged last tiles would be mostly padding
    assert plan(28672, 4096, 2, 8) == (0, 28672, 4096)    # grouped weight gradient
    assert lib.mxl_blockwise_gemm_tile(128) == 0 and plan(8192, 14336) == (0, 0, 0)
    assert lib.mxl_blockwise_gemm_tile(256) == 0 and plan(2048, 4096) == (0, 2048, 4096)
    assert lib.mxl_blockwise_gemm_tile(0) == 0 and plan(8192, 14336) == (0, 8192, 14336)
    assert lib.mxl_blockwise_gemm_tile(64) != 0
    assert plan(0, 128)[0] != 0 and plan(128, 100)[0] != 0 and plan(128, 128, 3)[0] != 0 and plan(128, 128, 1, 0)[0] != 0
