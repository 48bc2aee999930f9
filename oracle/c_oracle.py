"""ctypes loader of oracle/libmxoracle.so (the C restatement of the oracle).
TEST INFRASTRUCTURE ONLY -- see the header of mx_oracle.py."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

from . import mx_oracle as o

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmxoracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-B", "-C", HERE, "libmxoracle.so"], check=True)
    return LIB


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def quantize_rowwise(xb: np.ndarray, fmt: int, mode: int = 0):
    xb = np.ascontiguousarray(xb, dtype=np.uint16)
    rows, cols = xb.shape
    per = 2 if fmt == o.FMT_E2M1 else 1
    codes = np.empty((rows, cols // per), np.uint8)
    scales = np.empty((rows, cols // 32), np.uint8)
    load().mxo_quantize_rowwise(_p(xb), ctypes.c_int64(rows), ctypes.c_int64(cols), fmt, mode, _p(codes), _p(scales))
    return codes, scales


def quantize_colwise_segmented(xb: np.ndarray, group_lens, fmt: int, mode: int = 0):
    xb = np.ascontiguousarray(xb, dtype=np.uint16)
    rows, cols = xb.shape
    offs, poffs = o.segment_layout(group_lens)
    offs = np.ascontiguousarray(offs, np.int64)
    poffs = np.ascontiguousarray(poffs, np.int64)
    W = o.padded_width(rows, len(group_lens))
    per = 2 if fmt == o.FMT_E2M1 else 1
    codes = np.empty((cols, W // per), np.uint8)
    scales = np.empty((cols, W // 32), np.uint8)
    load().mxo_quantize_colwise_segmented(
        _p(xb), ctypes.c_int64(rows), ctypes.c_int64(cols), fmt, mode, _p(offs), _p(poffs), len(group_lens), ctypes.c_int64(W), _p(codes), _p(scales)
    )
    return codes, scales


def quantize_2d(wb: np.ndarray, fmt: int, mode: int = 0, row: bool = True, col: bool = True):
    wb = np.ascontiguousarray(wb, dtype=np.uint16)
    lead = wb.shape[:-2]
    batch = int(np.prod(lead)) if lead else 1
    n, k = wb.shape[-2:]
    per = 2 if fmt == o.FMT_E2M1 else 1
    q_row = np.empty(lead + (n, k // per), np.uint8) if row else None
    s_row = np.empty(lead + (n, k // 32), np.uint8) if row else None
    q_col = np.empty(lead + (k, n // per), np.uint8) if col else None
    s_col = np.empty(lead + (k, n // 32), np.uint8) if col else None
    load().mxo_quantize_2d(_p(wb), ctypes.c_int64(batch), ctypes.c_int64(n), ctypes.c_int64(k), fmt, mode, _p(q_row), _p(s_row), _p(q_col), _p(s_col))
    return q_row, s_row, q_col, s_col


def dequantize(codes: np.ndarray, scales: np.ndarray, fmt: int) -> np.ndarray:
    codes = np.ascontiguousarray(codes)
    scales = np.ascontiguousarray(scales)
    per = 2 if fmt == o.FMT_E2M1 else 1
    k = codes.shape[-1] * per
    rows = codes.size // codes.shape[-1]
    out = np.empty(codes.shape[:-1] + (k,), np.float32)
    load().mxo_dequantize(_p(codes), _p(scales), ctypes.c_int64(rows), ctypes.c_int64(k), fmt, _p(out))
    return out


def matmul_nt_bf16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), np.uint16)
    load().mxo_matmul_nt_bf16(_p(a), _p(b), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), _p(c))
    return c
