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
