"""HIP MX GEMMs (through the C ABI) against the CPU oracle: dense, grouped
(ragged / empty experts), variable-K wgrad, FP8 and FP4 operands.

Tolerance: max |got - want| <= 1e-2 * max |want| with bf16 output (the bound
named for this path; the reference's own layout-agreement bar is 2e-2,
tests/unit_tests/backends/megatron/test_native_fp8_layout.py:141-151).
Operands whose products and sums are exact in fp32 must match bit for bit.
"""

import os

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = 1e-2


def _dt(fmt):
    return torch.float8_e4m3fn if fmt == o.FMT_E4M3 else torch.float4_e2m1fn_x2


def _dev(a, dev, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev).view(dtype)


def _bf16_np(t):
    return o.bf16_bits_to_f32(t.view(torch.int16).cpu().numpy().view(np.uint16))


def _check(got, want, tol=TOL):
    assert not np.isnan(got).any()
    scale = max(np.abs(want).max(), 1e-30)
    err = np.abs(got - want).max() / scale
    assert err <= tol, f"max err {err:.3e} > {tol}"


def _run_fwd(dev, x, w, lens, afmt, bfmt):
    """x[M,K] bf16, w[G,N,K] bf16 (CPU) -> (gpu result, oracle result) as float arrays."""
    from primus_amd.pytorch import kernels as K

    aq, as_ = o.quantize_mx_rowwise(x, afmt)
    bq, bs = o.quantize_mx_rowwise(w, bfmt)
    want = o.grouped_gemm_nt_ref(aq, as_, bq, bs, lens, afmt, bfmt, out_bf16=False)
    A, SA = _dev(aq, dev, _dt(afmt)), _dev(as_, dev, torch.float8_e8m0fnu)
    B, SB = _dev(bq, dev, _dt(bfmt)), _dev(bs, dev, torch.float8_e8m0fnu)
    if len(lens) == 1 and w.shape[0] == 1:
        got = K.gemm_mx_nt_impl(A, SA, B[0], SB[0])
    else:
        got = K.grouped_gemm_mx_nt_impl(A, SA, B, SB, torch.tensor(lens, dtype=torch.int64, device=dev))
    return _bf16_np(got), want


@pytest.mark.parametrize(
    "m,n,k",
    [(256, 256, 128), (256, 256, 512), (300, 320, 384), (512, 512, 2880), (1, 32, 32), (257, 288, 160), (64, 1024, 4096)],
)
def test_dense_fp8(gpu, m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(1, n, k, generator=g) * 0.05).bfloat16()
    got, want = _run_fwd(gpu, x, w, [m], o.FMT_E4M3, o.FMT_E4M3)
    _check(got, want)


@pytest.mark.parametrize("afmt,bfmt", [(0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k", [(300, 320, 384), (130, 64, 2880)])
def test_dense_fp4_mixes(gpu, afmt, bfmt, m, n, k):
    g = torch.Generator().manual_seed(afmt * 2 + bfmt + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(1, n, k, generator=g) * 0.05).bfloat16()
    got, want = _run_fwd(gpu, x, w, [m], afmt, bfmt)
    _check(got, want)


@pytest.mark.parametrize(
    "lens,n,k",
    [
        ([300, 0, 5, 695], 512, 256),
        ([0, 33, 1, 64], 96, 160),
        ([0, 0, 0, 7], 64, 64),
        ([256, 256], 256, 128),
        ([1] * 32, 64, 96),
        ([513, 0, 255, 257, 0, 1, 31, 1000], 320, 512),
    ],
)
@pytest.mark.parametrize("afmt,bfmt", [(0, 0), (0, 1)])
def test_grouped_ragged(gpu, lens, n, k, afmt, bfmt):
    m = sum(lens)
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(len(lens), n, k, generator=g) * 0.05).bfloat16()
    got, want = _run_fwd(gpu, x, w, lens, afmt, bfmt)
    _check(got, want)


def _int_operands(rng, rows, k):
    vals = np.array([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=np.uint8)  # 0, +-1, +-2, +-3, 4
    q = vals[rng.integers(0, len(vals), size=(rows, k))]
    s = rng.integers(125, 130, size=(rows, k // 32)).astype(np.uint8)
    return q, s


def test_exact_integer_products_bit_exact(gpu):
    """Small integers with power-of-two scales: every partial sum is exact in
    fp32, so the result must equal the oracle bit for bit, whatever the
    accumulation order."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(12)
    lens = [300, 0, 77, 135]
    m, n, k = sum(lens), 288, 384
    aq, as_ = _int_operands(rng, m, k)
    bq, bs = _int_operands(rng, 4 * n, k)
    bq, bs = bq.reshape(4, n, k), bs.reshape(4, n, k // 32)
    want = o.grouped_gemm_nt_ref(aq, as_, bq, bs, lens)
    got = K.grouped_gemm_mx_nt_impl(
        _dev(aq, gpu, torch.float8_e4m3fn), _dev(as_, gpu, torch.float8_e8m0fnu), _dev(bq, gpu, torch.float8_e4m3fn),
        _dev(bs, gpu, torch.float8_e8m0fnu), torch.tensor(lens, dtype=torch.int64, device=gpu),
    )
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want)


def _exact_operands(rng, rows, k, fmt):
    """Codes whose values are small multiples of 1/2 and scales within 2^-2..2^2: all products and all
    partial sums of a row of a few hundred of them are exact in fp32."""
    if fmt == o.FMT_E4M3:
        q, s = _int_operands(rng, rows, k)
        return q, s
    nib = rng.integers(0, 16, size=(rows, k)).astype(np.uint8)          # every E2M1 value is a multiple of 1/2
    return o.pack_fp4(nib), rng.integers(125, 130, size=(rows, k // 32)).astype(np.uint8)


@pytest.mark.parametrize("afmt,bfmt", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("lens,n,k", [([300, 0, 77, 135], 288, 384), ([513], 256, 128), ([1, 0, 255, 257, 31], 96, 512),
                                      ([40] * 12, 544, 256)])
def test_exact_products_bit_exact_all_formats(gpu, afmt, bfmt, lens, n, k):
    """Forward / dgrad kernel, every operand-format pair: bit-equal to the oracle on operands whose
    arithmetic is exact, i.e. independent of accumulation order -- every output element, not a norm."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(afmt * 7 + bfmt * 3 + n + k)
    m, G = sum(lens), len(lens)
    aq, as_ = _exact_operands(rng, m, k, afmt)
    bq, bs = _exact_operands(rng, G * n, k, bfmt)
    bq, bs = bq.reshape(G, n, -1), bs.reshape(G, n, k // 32)
    want = o.grouped_gemm_nt_ref(aq, as_, bq, bs, lens, afmt, bfmt)
    A, SA = _dev(aq, gpu, _dt(afmt)), _dev(as_, gpu, torch.float8_e8m0fnu)
    B, SB = _dev(bq, gpu, _dt(bfmt)), _dev(bs, gpu, torch.float8_e8m0fnu)
    if G == 1:
        got = K.gemm_mx_nt_impl(A, SA, B[0], SB[0])
    else:
        got = K.grouped_gemm_mx_nt_impl(A, SA, B, SB, torch.tensor(lens, dtype=torch.int64, device=gpu))
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want)


@pytest.mark.parametrize("afmt,bfmt", [(0, 0), (1, 1), (0, 1)])
@pytest.mark.parametrize("lens,n,k", [([300, 0, 77, 135], 288, 160), ([513], 256, 128), ([1, 0, 255, 257, 31], 96, 320)])
def test_wgrad_exact_products_bit_exact(gpu, afmt, bfmt, lens, n, k):
    """Variable-K wgrad kernel on exact operands in the segment-padded transposed layout (zero codes in
    the padding): bit-equal to the oracle, empty experts exactly zero."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(afmt * 5 + bfmt + n + k)
    m, G = sum(lens), len(lens)
    W = o.padded_width(m, G)
    _, poffs = o.segment_layout(lens)
    live = np.zeros(W, dtype=bool)
    for g, ln in enumerate(lens):
        live[poffs[g] : poffs[g] + ln] = True

    def operand(rows, fmt):
        q, s = _exact_operands(rng, rows, W, fmt)
        if fmt == o.FMT_E2M1:
            nib = o.unpack_fp4(q)
            nib[:, ~live] = 0
            q = o.pack_fp4(nib)
        else:
            q[:, ~live] = 0
        return q, s

    aq, as_ = operand(n, afmt)
    bq, bs = operand(k, bfmt)
    want = o.grouped_gemm_wgrad_ref(aq, as_, bq, bs, lens, afmt, bfmt)
    got = K.grouped_gemm_mx_wgrad_impl(_dev(aq, gpu, _dt(afmt)), _dev(as_, gpu, torch.float8_e8m0fnu),
                                       _dev(bq, gpu, _dt(bfmt)), _dev(bs, gpu, torch.float8_e8m0fnu),
                                       torch.tensor(lens, dtype=torch.int64, device=gpu), m)
    got = got.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, want)
    for g, ln in enumerate(lens):
        if ln == 0:
            assert not got[g].any()


@pytest.mark.parametrize(
    "lens,n,k",
    [([300, 0, 5, 695], 320, 288), ([128], 256, 256), ([0, 33, 1, 64], 96, 160), ([0, 0], 64, 32), ([200, 200, 200], 512, 96)],
)
@pytest.mark.parametrize("fmt", [0, 1])
def test_wgrad_variable_k(gpu, lens, n, k, fmt):
    from primus_amd.pytorch import kernels as K

    m = sum(lens)
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(max(m, 1), k, generator=g).bfloat16()[:m]
    dy = torch.randn(max(m, 1), n, generator=g).bfloat16()[:m]
    dyT, dysT = o.quantize_mx_colwise_segmented(dy, lens, fmt)
    xT, xsT = o.quantize_mx_colwise_segmented(x, lens, fmt)
    want = o.grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, lens, fmt, fmt, out_bf16=False)
    if dyT.shape[1] == 0:  # no tokens at all and G small enough that the padded width is 0
        pytest.skip("degenerate: empty padded layout")
    got = K.grouped_gemm_mx_wgrad_impl(
        _dev(dyT, gpu, _dt(fmt)), _dev(dysT, gpu, torch.float8_e8m0fnu), _dev(xT, gpu, _dt(fmt)),
        _dev(xsT, gpu, torch.float8_e8m0fnu), torch.tensor(lens, dtype=torch.int64, device=gpu), m,
    )
    got = _bf16_np(got)
    assert got.shape == want.shape
    for e, ln in enumerate(lens):
        if ln == 0:
            assert not got[e].any()  # an expert without tokens gets exactly zero
    _check(got, want)


def test_golden_ragged_case(gpu):
    """The committed 4-expert case {0, 33, 1, 64}: forward from the stored codes,
    then the whole linear (quantise + 3 GEMMs) from the stored bf16 tensors."""
    from primus_amd.pytorch import kernels as K

    r = np.load(os.path.join(GOLD, "ragged_gemm.npz"))
    lens = torch.tensor(r["lens"], dtype=torch.int64, device=gpu)
    e8 = torch.float8_e8m0fnu
    y = K.grouped_gemm_mx_nt_impl(
        _dev(r["xq"], gpu, torch.float8_e4m3fn), _dev(r["xs"], gpu, e8), _dev(r["wq"], gpu, torch.float8_e4m3fn), _dev(r["ws"], gpu, e8), lens
    )
    _check(_bf16_np(y), o.bf16_bits_to_f32(r["y"]))
    m = int(r["lens"].sum())
    dy = torch.from_numpy(r["dy"].view(np.int16)).to(gpu).view(torch.bfloat16)
    x = torch.from_numpy(r["x"].view(np.int16)).to(gpu).view(torch.bfloat16)
    d_row, d_rs, d_col, d_cs = K.quantize_mx_impl(dy, 0, 0, rowwise=True, colwise=True, group_lens=lens)
    _, _, x_col, x_cs = K.quantize_mx_impl(x, 0, 0, rowwise=False, colwise=True, group_lens=lens)
    dx = K.grouped_gemm_mx_nt_impl(d_row, d_rs, _dev(r["wqt"], gpu, torch.float8_e4m3fn), _dev(r["wst"], gpu, e8), lens)
    dw = K.grouped_gemm_mx_wgrad_impl(d_col, d_cs, x_col, x_cs, lens, m)
    _check(_bf16_np(dx), o.bf16_bits_to_f32(r["dx"]))
    _check(_bf16_np(dw), o.bf16_bits_to_f32(r["dw"]))
    assert not _bf16_np(dw)[0].any()


def test_full_size_against_torch_fp32(gpu):
    """Mixtral-shape fc2 slice at full K (14336) and N (4096) on 2048 ragged rows:
    checked against a plain PyTorch fp32 matmul of the dequantised operands
    (decoded with torch's own float8 view, not with this library)."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator(device=gpu).manual_seed(1003)
    lens_l = [700, 0, 1, 600, 300, 447, 0, 0]
    m, k, n, G = sum(lens_l), 14336, 4096, 8
    x = torch.randn(m, k, generator=g, device=gpu).bfloat16()
    w = (torch.randn(G, n, k, generator=g, device=gpu) * 0.02).bfloat16()
    lens = torch.tensor(lens_l, dtype=torch.int64, device=gpu)
    xq, xs, _, _ = K.quantize_mx_impl(x, 0, 0, rowwise=True, colwise=False)
    wq, ws, _, _ = K.quantize_mx_weight_2d_impl(w, 0, 0, colwise=False)
    y = K.grouped_gemm_mx_nt_impl(xq, xs, wq, ws, lens).float()

    def deq(q, s):
        sc = torch.exp2(s.view(torch.uint8).float() - 127.0).repeat_interleave(32, dim=-1)
        return q.float() * sc

    xd, wd = deq(xq, xs), deq(wq, ws)
    offs = [0]
    for ln in lens_l:
        offs.append(offs[-1] + ln)
    want = torch.cat([xd[offs[e] : offs[e + 1]] @ wd[e].t() for e in range(G)])
    err = (y - want).abs().max() / want.abs().max()
    assert float(err) <= TOL, float(err)


def test_bad_arguments_return_errors(gpu):
    from primus_amd.pytorch import kernels as K

    a = torch.zeros(4, 64, dtype=torch.uint8, device=gpu).view(torch.float8_e4m3fn)
    s = torch.zeros(4, 2, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)
    b = torch.zeros(32, 96, dtype=torch.uint8, device=gpu).view(torch.float8_e4m3fn)
    sb = torch.zeros(32, 3, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)
    with pytest.raises(ValueError):
        K.gemm_mx_nt_impl(a, s, b, sb)  # K mismatch
    with pytest.raises(ValueError):
        K.gemm_mx_nt_impl(a, s, b[:, :64].contiguous(), sb)  # scale shape mismatch
    with pytest.raises(ValueError):
        K.gemm_mx_nt_impl(a, s, b[:, :64].contiguous(), sb[:, :2].contiguous(), out_dtype=torch.float16)
    lens = torch.tensor([4], dtype=torch.int32, device=gpu)
    with pytest.raises(ValueError):
        K.grouped_gemm_mx_nt_impl(a, s, b[None, :, :64].contiguous(), sb[None, :, :2].contiguous(), lens)  # int32 lens


def test_one_thousand_experts(gpu):
    """The largest expert count the device-side tile tables hold (1024), most experts with 0-3 rows:
    forward and wgrad against the oracle; one more expert is refused with an error, not a fault."""
    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(1024)
    G, n, k = _lib.MAX_GROUPS, 64, 128
    lens = rng.integers(0, 4, size=G).tolist()
    lens[17] = 300
    m = sum(lens)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(G, n, k, generator=g) * 0.05).bfloat16()
    got, want = _run_fwd(gpu, x, w, lens, o.FMT_E4M3, o.FMT_E4M3)
    _check(got, want)
    dy = torch.randn(m, n, generator=g).bfloat16()
    dyT, dysT = o.quantize_mx_colwise_segmented(dy, lens, o.FMT_E4M3)
    xT, xsT = o.quantize_mx_colwise_segmented(x, lens, o.FMT_E4M3)
    want = o.grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, lens, out_bf16=False)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    dw = _bf16_np(K.grouped_gemm_mx_wgrad_impl(
        _dev(dyT, gpu, torch.float8_e4m3fn), _dev(dysT, gpu, torch.float8_e8m0fnu), _dev(xT, gpu, torch.float8_e4m3fn),
        _dev(xsT, gpu, torch.float8_e8m0fnu), gl, m))
    _check(dw, want)
    # the quantiser writes the same transposed layout for that many groups
    q = K.quantize_mx_impl(x.to(gpu), o.FMT_E4M3, rowwise=False, colwise=True, group_lens=gl)
    assert np.array_equal(q[2].view(torch.uint8).cpu().numpy(), xT) and np.array_equal(q[3].view(torch.uint8).cpu().numpy(), xsT)
    too_many = torch.zeros(G + 1, dtype=torch.int64, device=gpu)
    with pytest.raises(Exception):
        K.quantize_mx_impl(x.to(gpu), o.FMT_E4M3, rowwise=False, colwise=True, group_lens=too_many)


@pytest.mark.parametrize("bad,clamped", [([200, 300], [200, 56]), ([-5, 256, 9], [0, 256, 0]), ([1000, 1000], [256, 0])])
def test_group_lens_that_do_not_match_the_buffers_are_clamped(gpu, bad, clamped):
    """Token counts live on the device, so no host check can catch counts that disagree with the
    buffers (stale or corrupted counts).  The kernels clamp them -- negative to 0, the running sum to
    the rows that exist -- and so behave exactly as for the clamped counts instead of leaving the
    buffers."""
    from primus_amd.pytorch import kernels as K

    rows, k, n = 256, 128, 64
    g = torch.Generator().manual_seed(3)
    x = torch.randn(rows, k, generator=g).bfloat16().to(gpu)
    w = (torch.randn(len(bad), n, k, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(rows, n, generator=g).bfloat16().to(gpu)
    outs = []
    for lens in (bad, clamped):
        gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
        xq, xs, xqT, xsT = K.quantize_mx_impl(x, o.FMT_E4M3, rowwise=True, colwise=True, group_lens=gl, pad_to=128)
        _, _, dqT, dsT = K.quantize_mx_impl(dy, o.FMT_E4M3, rowwise=False, colwise=True, group_lens=gl)
        wq, ws, _, _ = K.quantize_mx_weight_2d_impl(w, o.FMT_E4M3, rowwise=True, colwise=False, pad_to=128)
        y = K.grouped_gemm_mx_nt_impl(xq, xs, wq, ws, gl)
        dw = K.grouped_gemm_mx_wgrad_impl(dqT, dsT, xqT, xsT, gl, rows)
        covered = sum(clamped)
        outs.append((xq.view(torch.uint8)[:covered], xs.view(torch.uint8)[:covered], xqT.view(torch.uint8),
                     xsT.view(torch.uint8), y[:covered], dw))
    torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("mode", ["fwd", "wgrad"])
def test_fp4_fp4_repeated_launches_are_identical(gpu, mode):
    """Two FP4 operands make the LDS ring slots half as large as with FP8; the epilogue's staging
    patches must still fit into one of them (they once reached into the scale panels behind the ring,
    which the prefetch for the next tile writes at the same time: a rare, timing-dependent corruption).
    Many launches on the same exactly representable operands: every result equals the oracle's."""
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(279)
    lens = [257, 255, 256, 256, 300, 0, 0, 0]
    m, G, n, k = sum(lens), len(lens), 512, 128
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    f4, e8 = torch.float4_e2m1fn_x2, torch.float8_e8m0fnu
    if mode == "fwd":
        aq, as_ = _exact_operands(rng, m, k, o.FMT_E2M1)
        bq, bs = _exact_operands(rng, G * n, k, o.FMT_E2M1)
        bq, bs = bq.reshape(G, n, -1), bs.reshape(G, n, k // 32)
        want = o.grouped_gemm_nt_ref(aq, as_, bq, bs, lens, o.FMT_E2M1, o.FMT_E2M1)
        args = (_dev(aq, gpu, f4), _dev(as_, gpu, e8), _dev(bq, gpu, f4), _dev(bs, gpu, e8), gl)
        launch = lambda: K.grouped_gemm_mx_nt_impl(*args)   # noqa: E731
    else:
        W = o.padded_width(m, G)
        _, poffs = o.segment_layout(lens)
        live = np.zeros(W, dtype=bool)
        for g, ln in enumerate(lens):
            live[poffs[g] : poffs[g] + ln] = True

        def operand(rows):
            q, s = _exact_operands(rng, rows, W, o.FMT_E2M1)
            nib = o.unpack_fp4(q)
            nib[:, ~live] = 0
            return o.pack_fp4(nib), s

        (aq, as_), (bq, bs) = operand(288), operand(256)
        want = o.grouped_gemm_wgrad_ref(aq, as_, bq, bs, lens, o.FMT_E2M1, o.FMT_E2M1)
        args = (_dev(aq, gpu, f4), _dev(as_, gpu, e8), _dev(bq, gpu, f4), _dev(bs, gpu, e8), gl, m)
        launch = lambda: K.grouped_gemm_mx_wgrad_impl(*args)   # noqa: E731
    want_t = torch.from_numpy(want.view(np.int16)).to(gpu)
    bad = 0
    for _ in range(400):
        bad += int(not torch.equal(launch().view(torch.int16), want_t))
    assert bad == 0, f"{bad} of 400 launches differ from the oracle"


def test_calibration_loop_runs_for_every_operand_mix():
    """The register-only MFMA loop of the benchmark's calibration launches and finishes for the four operand mixes."""
    from primus_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    for fa in (_lib.FMT_E4M3, _lib.FMT_E2M1):
        for fb in (_lib.FMT_E4M3, _lib.FMT_E2M1):
            assert lib.mxl_calibrate_mfma(fa, fb, 8, st) == 0
    torch.cuda.synchronize()


def test_quantizer_traffic_twin_runs_in_every_mode():
    """The tile-copy kernel of the benchmark's calibration: each output it is given receives one byte per element
    (every byte of both arrays is written), the input is untouched."""
    from primus_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    x = torch.randn(256, 384, device=dev).bfloat16()
    keep = x.clone()
    for want_row, want_col in ((True, True), (True, False), (False, True), (False, False)):
        o1 = torch.full((256, 384), 0xA5, dtype=torch.uint8, device=dev)
        o2 = torch.full((384, 256), 0xA5, dtype=torch.uint8, device=dev)
        rc = lib.mxl_calibrate_tile_copy(x.data_ptr(), 256, 384, o1.data_ptr() if want_row else None,
                                         o2.data_ptr() if want_col else None, st)
        assert rc == 0
        torch.cuda.synchronize()
        # XORs of random bf16 halves: practically never all 0xA5 in a written array, exactly 0xA5 in an untouched one
        assert bool((o1 != 0xA5).any()) == want_row and bool((o2 != 0xA5).any()) == want_col
    assert torch.equal(x, keep)
    assert lib.mxl_calibrate_tile_copy(x.data_ptr(), 256, 100, None, None, st) == -1
