"""Writes tests/golden/*.npz from the CPU oracle (oracle/mx_oracle.py).

The reference tree holds no golden vectors for this path (its arithmetic lives
in an un-vendored package), so these fixtures are produced here, by the oracle
that tests/test_oracle_pinning.py pins against PyTorch's float8 cast, brute
force and closed forms.  Run from the repo root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import mx_oracle as o  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def exhaustive():
    """Every bf16 bit pattern, 32 consecutive patterns per MX block, so each
    block has a different amax and every value is cast under many scales."""
    x = np.arange(65536, dtype=np.uint16).reshape(2048, 32)
    # second arrangement: value v sits in a block whose amax is a fixed large number -> tests small-value rounding
    y = np.arange(65536, dtype=np.uint16).reshape(2048, 32).copy()
    y[:, 0] = 0x4380  # 256.0
    data = {"x": x, "y": y}
    for fmt, fn in ((o.FMT_E4M3, "e4m3"), (o.FMT_E2M1, "e2m1")):
        for mode, mn in ((0, "floor"), (1, "rceil"), (2, "even")):
            for name, arr in (("x", x), ("y", y)):
                q, s = o.quantize_mx_rowwise(arr, fmt, mode)
                data[f"{name}_{fn}_{mn}_q"] = q
                data[f"{name}_{fn}_{mn}_s"] = s
    np.savez_compressed(os.path.join(HERE, "exhaustive_bf16.npz"), **data)


def matrices():
    data = {}
    g = torch.Generator().manual_seed(1234)
    mats = {
        "normal": torch.randn(64, 96, generator=g),
        "weight": torch.randn(64, 96, generator=g) * 0.02,
        "outlier": torch.randn(64, 96, generator=g),
    }
    mask = torch.rand(64, 96, generator=g) < 0.01
    mats["outlier"] = torch.where(mask, mats["outlier"] * 50, mats["outlier"])
    for name, m in mats.items():
        xb = o.to_bf16_bits(m.bfloat16())
        data[f"{name}_x"] = xb
        for fmt, fn in ((o.FMT_E4M3, "e4m3"), (o.FMT_E2M1, "e2m1")):
            q, s = o.quantize_mx_rowwise(xb, fmt)
            qc, sc = o.quantize_mx_colwise_segmented(xb, [64], fmt)
            q2, s2, q2t, s2t = o.quantize_mx_2d(xb, fmt)
            for k, v in (("row_q", q), ("row_s", s), ("col_q", qc), ("col_s", sc), ("2d_q", q2), ("2d_s", s2), ("2d_qt", q2t), ("2d_st", s2t)):
                data[f"{name}_{fn}_{k}"] = v
    np.savez_compressed(os.path.join(HERE, "matrices.npz"), **data)


def ragged_gemm():
    g = torch.Generator().manual_seed(4321)
    lens = [0, 33, 1, 64]
    m, k, n = sum(lens), 160, 96
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(4, n, k, generator=g) * 0.05).bfloat16()
    dy = torch.randn(m, n, generator=g).bfloat16()
    xq, xs = o.quantize_mx_rowwise(x)
    wq, ws, wqt, wst = o.quantize_mx_2d(w)
    y = o.grouped_gemm_nt_ref(xq, xs, wq, ws, lens)
    dx, dw = o.linear_bwd_ref(x, w, dy, group_lens=lens)
    np.savez_compressed(
        os.path.join(HERE, "ragged_gemm.npz"),
        lens=np.array(lens, dtype=np.int64), x=o.to_bf16_bits(x), w=o.to_bf16_bits(w), dy=o.to_bf16_bits(dy),
        xq=xq, xs=xs, wq=wq, ws=ws, wqt=wqt, wst=wst, y=y, dx=dx, dw=dw,
    )


if __name__ == "__main__":
    exhaustive()
    matrices()
    ragged_gemm()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))
