"""Pins the CPU oracle against things it did not compute itself: PyTorch's
float8 cast (a library routine), brute-force nearest-value search, closed
forms in exact rational arithmetic, and algebraic invariants.  CPU only."""

import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

ALL_BF16 = np.arange(65536, dtype=np.uint16)
ALL_F32 = o.bf16_bits_to_f32(ALL_BF16)
FINITE = np.isfinite(ALL_F32)

E4M3_TABLE = o.decode_e4m3(np.arange(128, dtype=np.uint8))[:127].astype(np.float64)  # 0x7F is NaN


def _nearest_even(values: np.ndarray, table: np.ndarray) -> np.ndarray:
    """Brute force: index of the nearest table entry, ties to the even index,
    saturating at the last entry.  `table` is ascending and starts at 0."""
    a = np.minimum(np.abs(values.astype(np.float64)), table[-1])  # saturation
    d = np.abs(a[:, None] - table[None, :])
    best = d.min(axis=1)
    out = np.empty(len(a), dtype=np.int64)
    for i in range(len(a)):
        cand = np.nonzero(d[i] == best[i])[0]
        if len(cand) == 1:
            out[i] = cand[0]
        else:  # exact tie between two neighbours
            out[i] = cand[0] if cand[0] % 2 == 0 else cand[1]
    return out


def test_e4m3_table_is_the_ocp_format():
    # known values of the OCP FP8 E4M3 format
    assert E4M3_TABLE[0] == 0.0
    assert E4M3_TABLE[1] == 2.0**-9  # smallest subnormal
    assert E4M3_TABLE[8] == 2.0**-6  # smallest normal
    assert E4M3_TABLE[0x38] == 1.0
    assert E4M3_TABLE[0x7E] == 448.0  # largest normal
    assert np.all(np.diff(E4M3_TABLE) > 0)
    assert np.isnan(o.decode_e4m3(np.array([0x7F, 0xFF], dtype=np.uint8))).all()
    t = torch.arange(127, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(t.astype(np.float64), E4M3_TABLE)


def test_cast_e4m3_matches_torch_on_every_bf16_and_scale():
    # the multiply by a power of two is exact, so this covers every reachable (x, scale) pair class
    for shift in range(-12, 13):
        with np.errstate(over="ignore"):
            v = (ALL_F32[FINITE] * np.float32(2.0**shift)).astype(np.float32)
        want = torch.from_numpy(v).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(o.cast_e4m3(v), want), shift


def test_cast_e4m3_matches_torch_on_random_fp32():
    rng = np.random.default_rng(11)
    v = (rng.standard_normal(1 << 20) * np.exp2(rng.integers(-16, 11, 1 << 20))).astype(np.float32)
    want = torch.from_numpy(v).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(o.cast_e4m3(v), want)


def test_cast_e4m3_brute_force_nearest_even():
    rng = np.random.default_rng(5)
    v = (rng.standard_normal(4000) * np.exp2(rng.integers(-12, 10, 4000))).astype(np.float32)
    # add exact ties and the saturation region
    ties = ((E4M3_TABLE[:-1] + E4M3_TABLE[1:]) / 2).astype(np.float32)
    v = np.concatenate([v, ties, -ties, np.float32([448, 449, 464, 465, 480, 1e9, -1e9, 0.0, -0.0])])
    code = o.cast_e4m3(v)
    want = _nearest_even(v, E4M3_TABLE)
    assert np.array_equal(code & 0x7F, want)
    assert np.array_equal(code >> 7, np.signbit(v).astype(np.uint8))


def test_cast_e2m1_brute_force_nearest_even_every_bf16():
    table = o.E2M1_VALUES.astype(np.float64)
    for shift in (-3, -1, 0, 1, 2):
        with np.errstate(over="ignore"):
            v = (ALL_F32[FINITE] * np.float32(2.0**shift)).astype(np.float32)
        # brute force is O(n*8): fine for 65k values
        a = np.minimum(np.abs(v.astype(np.float64)), 6.0)  # saturation
        d = np.abs(a[:, None] - table[None, :])
        idx = d.argmin(axis=1)  # first minimum = lower neighbour on ties
        tie = (d == d.min(axis=1, keepdims=True)).sum(axis=1) == 2
        idx = np.where(tie & (idx % 2 == 1), idx + 1, idx)
        code = o.cast_e2m1(v)
        assert np.array_equal(code & 7, idx), shift
        assert np.array_equal(code >> 3, np.signbit(v).astype(np.uint8))
    assert np.array_equal(o.decode_e2m1(np.arange(8, dtype=np.uint8)), o.E2M1_VALUES)


def _exact_log2_floor(fr: Fraction) -> int:
    e = 0
    while fr >= 2:
        fr /= 2
        e += 1
    while fr < 1:
        fr *= 2
        e -= 1
    return e


@pytest.mark.parametrize("fmt,emax,maxnorm,mbits", [(o.FMT_E4M3, 8, 448, 3), (o.FMT_E2M1, 2, 6, 1)])
def test_scale_byte_closed_forms_every_amax(fmt, emax, maxnorm, mbits):
    """OCP floor: floor(log2 amax) - emax.  RCEIL: ceil(log2(amax / max_normal)).
    EVEN: floor(log2(round-half-up of amax to (1+mbits) significant bits)) - emax.
    All clamped to [0, 254] after adding the bias 127; evaluated with exact
    rationals for every positive normal bf16 amax."""
    bits = np.arange(0x0080, 0x7F80, dtype=np.uint32)  # positive normal bf16
    got = {m: o.e8m0_scale_byte(bits << 16, fmt, m) for m in (o.SCALE_OCP_FLOOR, o.SCALE_RCEIL, o.SCALE_EVEN)}
    for i, b in enumerate(bits[::7]):  # every 7th value keeps the rational arithmetic fast; covers all exponents
        j = i * 7
        e = (int(b) >> 7) - 127
        man = Fraction(128 + (int(b) & 0x7F), 128)
        amax = man * Fraction(2) ** e
        fl = _exact_log2_floor(amax)
        assert fl == e
        want_floor = min(max(fl - emax + 127, 0), 254)
        q = amax / maxnorm
        ce = _exact_log2_floor(q)
        if Fraction(2) ** ce != q:
            ce += 1
        want_rceil = min(max(ce + 127, 0), 254)
        # EVEN: round the significand to mbits fractional bits, half up
        step = Fraction(1, 2**mbits)
        rounded = (man / step + Fraction(1, 2)).__floor__() * step * Fraction(2) ** e
        want_even = min(max(_exact_log2_floor(rounded) - emax + 127, 0), 254)
        assert got[o.SCALE_OCP_FLOOR][j] == want_floor, hex(b)
        assert got[o.SCALE_RCEIL][j] == want_rceil, hex(b)
        assert got[o.SCALE_EVEN][j] == want_even, hex(b)


def test_scale_byte_edges():
    for fmt in (o.FMT_E4M3, o.FMT_E2M1):
        for mode in (0, 1, 2):
            z = o.e8m0_scale_byte(np.array([0], dtype=np.uint32), fmt, mode)
            assert z[0] == 0  # amax == 0 -> 2^-127
            sub = o.e8m0_scale_byte(np.array([0x007F0000], dtype=np.uint32), fmt, mode)  # bf16 subnormal
            assert sub[0] == 0
            big = o.e8m0_scale_byte(np.array([0x7F7F0000], dtype=np.uint32), fmt, mode)  # largest finite bf16
            assert 240 <= big[0] <= 253


def test_rceil_never_saturates_and_floor_is_within_one():
    """With RCEIL no finite element exceeds the format's max after scaling;
    OCP floor may exceed it by < 2x and then saturates."""
    bits = np.arange(0x0800, 0x7F00, dtype=np.uint32) << 16
    amax = bits.view(np.float32).astype(np.float64)
    for fmt, mx in ((o.FMT_E4M3, 448.0), (o.FMT_E2M1, 6.0)):
        r = o.e8m0_scale_byte(bits, fmt, o.SCALE_RCEIL).astype(np.float64)
        f = o.e8m0_scale_byte(bits, fmt, o.SCALE_OCP_FLOOR).astype(np.float64)
        ok = (r > 0) & (r < 254)
        assert np.all(amax[ok] / np.exp2(r[ok] - 127) <= mx)
        assert np.all(amax[ok] / np.exp2(r[ok] - 127) > mx / 2)
        assert np.all((r - f >= 0) & (r - f <= 1))


def test_rowwise_roundtrip_error_bound():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 256, generator=g).bfloat16()
    xf = x.float().numpy()
    for mode in (0, 1, 2):
        q, s = o.quantize_mx_rowwise(x, o.FMT_E4M3, mode)
        dq = o.dequantize_mx(q, s, o.FMT_E4M3)
        blk_amax = np.abs(xf).reshape(64, 8, 32).max(-1).repeat(32, -1).reshape(64, 256)
        # E4M3 keeps 3 mantissa bits: relative step 2^-3, so error <= 2^-4 of the value's binade,
        # and never more than 1/8 of the block maximum (saturation under the floor rule is < 2x)
        assert np.all(np.abs(dq - xf) <= blk_amax * 0.125 + 1e-30), mode
        q4, s4 = o.quantize_mx_rowwise(x, o.FMT_E2M1, mode)
        dq4 = o.dequantize_mx(q4, s4, o.FMT_E2M1)
        assert np.all(np.abs(dq4 - xf) <= blk_amax * 0.5 + 1e-30), mode


def test_representable_values_survive_exactly():
    # values that are exactly code * 2^k must round-trip bit for bit
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 0x7F, size=(16, 64)).astype(np.uint8) | (rng.integers(0, 2, size=(16, 64)) << 7).astype(np.uint8)
    codes[:, 0] = 0x7E  # pin each block's amax at the top of the format so the scale is recovered exactly
    codes[:, 32] = 0x7E
    scales = rng.integers(100, 150, size=(16, 2)).astype(np.uint8)
    x = o.dequantize_mx(codes, scales, o.FMT_E4M3)
    xb = o.f32_to_bf16_bits(x)
    assert np.array_equal(o.bf16_bits_to_f32(xb), x)  # e4m3 * 2^k fits bf16
    q, s = o.quantize_mx_rowwise(xb, o.FMT_E4M3, o.SCALE_OCP_FLOOR)
    assert np.array_equal(s, scales)
    assert np.array_equal(q & 0x7F, codes & 0x7F)


def test_colwise_is_rowwise_of_the_transpose():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(96, 64, generator=g).bfloat16()
    for fmt in (o.FMT_E4M3, o.FMT_E2M1):
        qc, sc = o.quantize_mx_colwise(x, fmt)
        qr, sr = o.quantize_mx_rowwise(x.t().contiguous(), fmt)
        assert np.array_equal(qc, qr) and np.array_equal(sc, sr)


def test_2d_block_copies_are_byte_transposes_and_experts_independent():
    """Q_row(W)^T == Q_colT(W) byte for byte, scales shared by the 32x32 tile, and a
    3-D weight is quantised expert by expert in original tile coordinates
    (tests/unit_tests/backends/megatron/test_weight_deosc.py:82-127)."""
    g = torch.Generator().manual_seed(6)
    w = (torch.randn(3, 64, 96, generator=g) * 0.02).bfloat16()
    q, s, qt, st = o.quantize_mx_2d(w, o.FMT_E4M3)
    assert np.array_equal(np.swapaxes(q, -1, -2), qt)
    assert np.array_equal(s[:, ::32, :], np.swapaxes(st[:, ::32, :], -1, -2))
    assert np.all(s.reshape(3, 2, 32, 3) == s.reshape(3, 2, 32, 3)[:, :, :1, :])
    for e in range(3):
        qe, se, _, _ = o.quantize_mx_2d(w[e], o.FMT_E4M3)
        assert np.array_equal(qe, q[e]) and np.array_equal(se, s[e])
    # the tile scale is the row-wise rule applied to the tile's amax
    wb = o.to_bf16_bits(w)
    tile = wb[1, 32:64, 64:96]
    amax = (tile & 0x7FFF).max().astype(np.uint32) << 16
    assert s[1, 40, 2] == o.e8m0_scale_byte(np.array([amax]), o.FMT_E4M3)[0]
    q4, s4, q4t, s4t = o.quantize_mx_2d(w, o.FMT_E2M1)
    assert np.array_equal(np.swapaxes(o.unpack_fp4(q4), -1, -2), o.unpack_fp4(q4t))


def test_nonfinite_and_zero_blocks():
    x = torch.zeros(2, 64).bfloat16()
    x[0, 3] = float("inf")
    x[0, 5] = -2.0
    x[0, 40] = float("nan")
    x[1, 0] = -0.0
    q, s = o.quantize_mx_rowwise(x, o.FMT_E4M3)
    assert s[0, 0] == 255 and s[0, 1] == 255 and s[1, 0] == 0 and s[1, 1] == 0
    assert q[0, 3] == 0x7F and q[0, 40] == 0x7F and q[0, 5] == 0x80 and q[0, 6] == 0x00
    assert q[1, 0] == 0x80 and q[1, 1] == 0
    assert np.isnan(o.dequantize_mx(q, s)[0]).all()
    q4, s4 = o.quantize_mx_rowwise(x, o.FMT_E2M1)
    c = o.unpack_fp4(q4)
    assert s4[0, 0] == 255 and c[0, 3] == 0x7 and c[0, 40] == 0x7 and c[0, 5] == 0x8 and c[1, 0] == 0x8


def test_fp4_nibble_order():
    x = torch.zeros(1, 32).bfloat16()
    x[0, 0] = 6.0
    x[0, 1] = -1.0
    q, s = o.quantize_mx_rowwise(x, o.FMT_E2M1)
    assert s[0, 0] == 127  # floor(log2 6) - 2 = 0
    assert q[0, 0] == (0x7 | (0xA << 4))  # element 0 in bits 3:0, element 1 in bits 7:4


def test_segment_layout_and_padding():
    lens = [33, 0, 130, 1]
    offs, poffs = o.segment_layout(lens)
    assert list(offs) == [0, 33, 33, 163, 164] and list(poffs) == [0, 128, 128, 384, 512]
    assert o.padded_width(164, 4) >= poffs[-1]
    assert o.padded_width(256, 1) == 256 and o.padded_width(257, 1) == 384
    # worst case of the bound: every group one row over a multiple of 128
    assert o.padded_width(4 * 129, 4) == 4 * 256
    g = torch.Generator().manual_seed(8)
    x = torch.randn(164, 32, generator=g).bfloat16()
    q, s = o.quantize_mx_colwise_segmented(x, lens)
    W = o.padded_width(164, 4)
    assert q.shape == (32, W) and s.shape == (32, W // 32)
    # group 2 alone, quantised as its own matrix, lands at its padded offset
    # 130 is not a multiple of 32 -> pad by hand
    xp = torch.zeros(160, 32).bfloat16()
    xp[:130] = x[33:163]
    q2, s2 = o.quantize_mx_colwise(xp)
    assert np.array_equal(q[:, 128:288], q2) and np.array_equal(s[:, 4:9], s2)
    assert not q[:, 288:384].any() and not s[:, 9:12].any()  # padding: zero codes, byte 0


def _int_case(rng, m, n, k):
    """Operands whose products and sums are exact in fp32: small integers with
    power-of-two block scales."""
    vals = np.array([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=np.uint8)  # 0, 1, 2, 3, 4, -1, -2, -3
    a = vals[rng.integers(0, len(vals), size=(m, k))]
    b = vals[rng.integers(0, len(vals), size=(n, k))]
    sa = rng.integers(125, 130, size=(m, k // 32)).astype(np.uint8)
    sb = rng.integers(125, 130, size=(n, k // 32)).astype(np.uint8)
    return a, sa, b, sb


def test_gemm_oracle_exact_on_integer_operands():
    rng = np.random.default_rng(2)
    a, sa, b, sb = _int_case(rng, 8, 12, 64)
    ai = o.decode_e4m3(a).astype(np.int64)
    bi = o.decode_e4m3(b).astype(np.int64)
    # integer reference with the scales folded in as shifts (scale exponent in [-2, 2] -> multiply by 4 first)
    ea = np.repeat(sa.astype(np.int64) - 125, 32, axis=1)
    eb = np.repeat(sb.astype(np.int64) - 125, 32, axis=1)
    want = ((ai << ea) @ (bi << eb).T).astype(np.float64) / 16.0
    got = o.gemm_nt_ref(a, sa, b, sb, out_bf16=False)
    assert np.array_equal(got.astype(np.float64), want)


def test_grouped_gemm_oracle_invariants():
    rng = np.random.default_rng(3)
    k, n = 64, 32
    lens = [5, 0, 33, 1]
    a, sa, _, _ = _int_case(rng, sum(lens), 1, k)
    bs = [_int_case(rng, 1, n, k)[2:] for _ in lens]
    b = np.stack([x[0] for x in bs])
    sb = np.stack([x[1] for x in bs])
    y = o.grouped_gemm_nt_ref(a, sa, b, sb, lens, out_bf16=False)
    offs = np.concatenate([[0], np.cumsum(lens)])
    for g in range(4):  # each group equals the dense oracle on its rows
        sl = slice(offs[g], offs[g + 1])
        assert np.array_equal(y[sl], o.gemm_nt_ref(a[sl], sa[sl], b[g], sb[g], out_bf16=False))
    # G = 1 is the dense GEMM
    assert np.array_equal(
        o.grouped_gemm_nt_ref(a, sa, b[:1], sb[:1], [sum(lens)], out_bf16=False), o.gemm_nt_ref(a, sa, b[0], sb[0], out_bf16=False)
    )
    # permuting experts permutes row blocks
    perm = [2, 0, 3, 1]
    a_p = np.concatenate([a[offs[g] : offs[g + 1]] for g in perm])
    sa_p = np.concatenate([sa[offs[g] : offs[g + 1]] for g in perm])
    y_p = o.grouped_gemm_nt_ref(a_p, sa_p, b[perm], sb[perm], [lens[g] for g in perm], out_bf16=False)
    assert np.array_equal(y_p, np.concatenate([y[offs[g] : offs[g + 1]] for g in perm]))


def test_wgrad_oracle_matches_per_expert_dense_and_zero_fills():
    g = torch.Generator().manual_seed(9)
    lens = [0, 33, 1, 64]
    m = sum(lens)
    x = torch.randn(m, 64, generator=g).bfloat16()
    dy = torch.randn(m, 32, generator=g).bfloat16()
    dyT, dysT = o.quantize_mx_colwise_segmented(dy, lens)
    xT, xsT = o.quantize_mx_colwise_segmented(x, lens)
    dw = o.grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, lens, out_bf16=False)
    assert dw.shape == (4, 32, 64) and not dw[0].any()
    offs = np.concatenate([[0], np.cumsum(lens)])
    for e in (1, 2, 3):
        # per-expert: pad the expert's rows to a multiple of 32 with zeros, quantise col-wise, dense NT GEMM
        rows = lens[e]
        pad = (rows + 31) // 32 * 32
        xe = torch.zeros(pad, 64).bfloat16()
        de = torch.zeros(pad, 32).bfloat16()
        xe[:rows] = x[offs[e] : offs[e + 1]]
        de[:rows] = dy[offs[e] : offs[e + 1]]
        qa, sa = o.quantize_mx_colwise(de)
        qb, sb = o.quantize_mx_colwise(xe)
        want = o.gemm_nt_ref(qa, sa, qb, sb, out_bf16=False)
        np.testing.assert_allclose(dw[e], want, rtol=1e-6, atol=1e-6)
    # and the whole thing is close to the unquantised gradient (cosine, as the reference's MoE test does)
    true = torch.stack([dy[offs[e] : offs[e + 1]].float().t() @ x[offs[e] : offs[e + 1]].float() for e in range(4)]).numpy()
    cos = (dw * true).sum() / (np.linalg.norm(dw) * np.linalg.norm(true))
    assert cos > 0.99


def test_linear_oracle_close_to_bf16_truth():
    g = torch.Generator().manual_seed(10)
    x = torch.randn(64, 128, generator=g).bfloat16()
    w = (torch.randn(96, 128, generator=g) * 0.02).bfloat16()
    y = o.bf16_bits_to_f32(o.linear_fwd_ref(x, w))
    true = (x.float() @ w.float().t()).numpy()
    cos = (y * true).sum() / (np.linalg.norm(y) * np.linalg.norm(true))
    assert cos > 0.995
    y4 = o.bf16_bits_to_f32(o.linear_fwd_ref(x, w, o.FMT_E2M1, o.FMT_E2M1))
    snr = 10 * math.log10((true**2).sum() / ((y4 - true) ** 2).sum())
    assert snr > 10  # the reference's MXFP4 bar (test_primus_turbo_mxfp4_local.py:182-189)
