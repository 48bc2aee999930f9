"""Pins the oracle's 128-blockwise FP8 quantisers and GEMM: the per-block formula (the one the reference restates for
its tensor-wise quantiser, primus_turbo_float8_local.py:194-207, applied to the blocks of :1019-1061) evaluated with
torch ops on reshaped blocks and torch's float8 casts (library routines); a tensor that is one block equals the
tensor-wise quantiser; blocks are independent; the GEMM against float64 arithmetic on the decoded operands."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

FMTS = [(o.FMT_E4M3, torch.float8_e4m3fn, 448.0), (o.FMT_E5M2, torch.float8_e5m2, 57344.0)]


def _x(seed, rows, cols, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, cols, generator=g) * spread * torch.logspace(-2, 1, cols)[None, :]).bfloat16()


@pytest.mark.parametrize("fmt,dt,fmax", FMTS)
@pytest.mark.parametrize("rows,cols", [(5, 128), (64, 384), (200, 256)])
def test_rowwise_blocks_match_the_formula_in_torch(fmt, dt, fmax, rows, cols):
    x = _x(rows + cols + fmt, rows, cols)
    codes, sinv = o.quantize_blockwise(x, fmt, axis=-1)
    blocks = x.float().reshape(rows, cols // 128, 128)
    amax = blocks.abs().amax(dim=2, keepdim=True)
    scale = torch.full_like(amax, fmax) / amax.clamp(min=1e-12)      # tensor / tensor: an IEEE division (scalar / tensor is not)
    want = (blocks * scale).clamp(-fmax, fmax).to(dt).view(torch.uint8).reshape(rows, cols).numpy()
    assert codes.shape == (rows, cols) and np.array_equal(codes, want)
    assert sinv.shape == (rows, cols // 128) and sinv.dtype == np.float32
    assert np.allclose(sinv, (amax.double() / fmax).reshape(rows, cols // 128).numpy(), rtol=2.5e-7, atol=0)
    # every block's largest element lands on the largest code
    top = (np.abs(o.decode_fp8(codes, fmt)).reshape(rows, cols // 128, 128).max(axis=2))
    assert np.all(top == fmax)


@pytest.mark.parametrize("fmt,dt,fmax", FMTS)
@pytest.mark.parametrize("rows", [128, 200, 1])
def test_blocks_along_the_rows_come_back_transposed_and_padded(fmt, dt, fmax, rows):
    cols = 256
    x = _x(rows + fmt, rows, cols, 3.0)
    codes_t, sinv_t = o.quantize_blockwise(x, fmt, axis=0)
    rows_pad = -(-rows // 128) * 128
    assert codes_t.shape == (cols, rows_pad) and sinv_t.shape == (cols, rows_pad // 128)
    xp = torch.zeros(rows_pad, cols)
    xp[:rows] = x.float()
    blocks = xp.reshape(rows_pad // 128, 128, cols)
    amax = blocks.abs().amax(dim=1, keepdim=True)
    scale = torch.full_like(amax, fmax) / amax.clamp(min=1e-12)      # tensor / tensor: an IEEE division (scalar / tensor is not)
    want = (blocks * scale).clamp(-fmax, fmax).to(dt).view(torch.uint8).reshape(rows_pad, cols).numpy()
    assert np.array_equal(codes_t, want.T)
    assert not codes_t[:, rows:].any()
    assert np.allclose(sinv_t, (amax.double() / fmax).reshape(rows_pad // 128, cols).numpy().T, rtol=2.5e-7, atol=0)
    # the same thing through the row-wise quantiser on the transposed tensor
    xt = o.f32_to_bf16_bits(xp.numpy().T.copy())
    c2, s2 = o.quantize_blockwise(xt, fmt, axis=-1)
    assert np.array_equal(c2, codes_t) and np.array_equal(s2, sinv_t)


@pytest.mark.parametrize("fmt,dt,fmax", FMTS)
def test_2d_blocks_and_the_single_block_case(fmt, dt, fmax):
    w = (_x(3 + fmt, 256, 384) * 0.02).bfloat16()
    codes, sinv, codes_t, sinv_t = o.quantize_blockwise_2d(w, fmt)
    tiles = w.float().reshape(2, 128, 3, 128)
    amax = tiles.abs().amax(dim=(1, 3), keepdim=True)
    scale = torch.full_like(amax, fmax) / amax.clamp(min=1e-12)      # tensor / tensor: an IEEE division (scalar / tensor is not)
    want = (tiles * scale).clamp(-fmax, fmax).to(dt).view(torch.uint8).reshape(256, 384).numpy()
    assert np.array_equal(codes, want) and np.array_equal(codes_t, want.T)
    assert sinv.shape == (2, 3) and np.array_equal(sinv_t, sinv.T)
    # one 128 x 128 tile is a tensor with a single scale: the tensor-wise quantiser
    one = w[:128, :128].contiguous()
    c1, s1, _, _ = o.quantize_blockwise_2d(one, fmt)
    ct, st = o.quantize_tensorwise(one, fmt)
    assert np.array_equal(c1, ct) and s1.shape == (1, 1) and s1[0, 0] == st
    # blocks are independent: changing one tile leaves the codes and scales of the others alone
    w2 = w.clone()
    w2[130:140, 5:9] = 100.0
    d, ds, _, _ = o.quantize_blockwise_2d(w2, fmt)
    keep = np.ones((256, 384), bool)
    keep[128:, :128] = False
    assert np.array_equal(d[keep], codes[keep]) and ds[0].tolist() == sinv[0].tolist() and ds[1, 1:].tolist() == sinv[1, 1:].tolist()
    assert ds[1, 0] != sinv[1, 0]


def test_zero_and_nonfinite_blocks():
    x = torch.zeros(4, 256).bfloat16()
    x[1, 130] = float("inf")
    x[2, 5] = 3.0
    codes, sinv = o.quantize_blockwise(x, o.FMT_E4M3)
    assert not codes[0].any() and np.all(np.isfinite(sinv[0])) and sinv[0, 0] == np.float32(1.0) / (np.float32(448.0) / np.float32(1e-12))
    assert np.all(codes[1, 128:] == 0x7F) and not codes[1, :128].any()
    assert codes[2, 5] == 0x7E and sinv[2, 0] == np.float32(1.0) / (np.float32(448.0) / np.float32(3.0))


@pytest.mark.parametrize("per_row", [False, True])
def test_gemm_reference_against_float64(per_row):
    x = _x(11, 70, 384)
    w = (_x(12, 256, 384) * 0.05).bfloat16()
    a, sa = o.quantize_blockwise(x, o.FMT_E4M3)
    if per_row:
        b, sb = o.quantize_blockwise(w, o.FMT_E5M2)
        bf = o.FMT_E5M2
    else:
        b, sb, _, _ = o.quantize_blockwise_2d(w, o.FMT_E4M3)
        bf = o.FMT_E4M3
    got = o.blockwise_gemm_nt_ref(a, sa, b, sb, o.FMT_E4M3, bf, out_bf16=False)
    da = o.decode_fp8(a, o.FMT_E4M3).astype(np.float64) * np.repeat(sa.astype(np.float64), 128, axis=1)
    sbr = sb if per_row else np.repeat(sb, 128, axis=0)
    db = o.decode_fp8(b, bf).astype(np.float64) * np.repeat(sbr.astype(np.float64), 128, axis=1)
    want = da @ db.T
    scale = np.abs(da) @ np.abs(db).T
    assert np.all(np.abs(got - want) <= 400 * 2.0 ** -24 * scale + 1e-30)
    # and the dequantised operands are the input to FP8 precision, so the product is the bf16 product to ~2^-3 of |x||w|
    ref = x.double().numpy() @ w.double().numpy().T
    assert np.abs(got - ref).max() <= 0.08 * (np.abs(x.double().numpy()) @ np.abs(w.double().numpy()).T).max()


def test_segmented_copy_is_the_groups_side_by_side():
    lens = [5, 0, 130, 64]
    x = _x(21, sum(lens), 256, 2.0)
    codes, sinv = o.quantize_blockwise_segmented(x, lens, o.FMT_E4M3)
    assert codes.shape == (256, o.padded_width(sum(lens), 4, 128)) and sinv.shape == (256, codes.shape[1] // 128)
    pos = src = 0
    for n in lens:
        w = -(-n // 128) * 128
        if n:
            c, s = o.quantize_blockwise(x[src:src + n], o.FMT_E4M3, axis=0)
            assert np.array_equal(codes[:, pos:pos + w], c) and np.array_equal(sinv[:, pos // 128:(pos + w) // 128], s)
        pos += w
        src += n
    assert not codes[:, pos:].any()
    # the wgrad reference over the segments equals per-group products of the dequantised pieces
    dy = _x(22, sum(lens), 128)
    at, sat = o.quantize_blockwise_segmented(dy, lens, o.FMT_E4M3)
    got = o.grouped_blockwise_wgrad_ref(at, sat, codes, sinv, lens, out_bf16=False)
    assert got.shape == (4, 128, 256) and not got[1].any()
    da = o.decode_fp8(at, o.FMT_E4M3).astype(np.float64) * np.repeat(sat.astype(np.float64), 128, axis=1)
    db = o.decode_fp8(codes, o.FMT_E4M3).astype(np.float64) * np.repeat(sinv.astype(np.float64), 128, axis=1)
    seg3 = slice(128 + 256, 128 + 256 + 128)
    ref = da[:, seg3] @ db[:, seg3].T
    assert np.allclose(got[3], ref, rtol=1e-5, atol=1e-5 * np.abs(ref).max())
