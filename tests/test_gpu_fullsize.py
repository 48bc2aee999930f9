"""The benchmark configurations at their FULL shapes (Llama-3-8B MLP with outlier-injected
activations, Mixtral-8x7B, DeepSeek-V3 expert shard, GPT-OSS-120B with MXFP4 weights under
uniform and under skewed routing): same seeded routing, tensor shapes and per-tensor
distributions as bench.py.

A full CPU oracle run at these sizes would take hours, so each case checks
 (1) quantised bytes and scales BIT-EXACT against the oracle on sampled bands (the
     first and last rows of experts -- where blocks restart and padding begins -- and
     random interior rows; both the row-wise and the transposed copy),
 (2) forward, dgrad and wgrad outputs of the differentiable op at sampled output
     positions against the oracle's fp64 dot products of the dequantised operands
     (tolerance 1e-2 of the largest expected magnitude, 3e-2 with FP4 operands),
 (3) size-independent properties: an expert without tokens gets an all-zero weight
     gradient and no output rows; outputs are finite.
"""

import numpy as np
import pytest
import torch

import bench
from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu


def _u8(t):
    return t.view(torch.uint8)


def _deq_rows(codes_u8, scales_u8, fmt):
    """float64 [rows, K] from uint8 numpy codes / scales (row-wise layout)."""
    return o.dequantize_mx(codes_u8, scales_u8, fmt).astype(np.float64)


def _bf(t):
    return o.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)


def _elementwise_bound(want, absdot, k):
    """|got - want| allowed per element: bf16 rounding of the output (2^-8 relative) plus the accumulation error,
    (k + 1024) * 2^-23 * sum |a_i b_i|: k fp32 additions, and a floor of 2^-13 for the MFMA's 64-term dot product,
    whose products are aligned to a common exponent in a finite datapath (measured: at most 2^-16 of sum |a_i b_i|
    beyond the output rounding, at k = 128 as at k = 14336)."""
    return 2.0 ** -8 * np.abs(want) + (k + 1024) * 2.0 ** -23 * absdot + 1e-30


def _sample_rows(lens, rng, per_group=2):
    """Row indices: first and last row of every non-empty expert plus random interior rows."""
    rows, off = [], 0
    for n in lens:
        if n > 0:
            rows += [off, off + n - 1]
            rows += [off + int(v) for v in rng.integers(0, n, size=per_group)]
        off += n
    return sorted(set(rows))


def _group_of(row, lens):
    off = 0
    for g, n in enumerate(lens):
        if row < off + n:
            return g, off
        off += n
    raise AssertionError


CASES = [
    ("llama3_8b_mlp_mxfp8", 0),
    ("mixtral_8x7b_moe_mxfp8", 0),
    ("deepseek_v3_shard_mxfp8", 0),
    ("gpt_oss_120b_mxfp4", 0),
    ("gpt_oss_120b_mxfp4_skewed", 0),     # 16 experts without tokens, 11 with more than four times the mean
]


@pytest.mark.parametrize("workload,layer", [(w, l) for w, _ in CASES for l in (0, 1)])
def test_full_size_linear(gpu, workload, layer):
    import primus_amd.pytorch as pt
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    spec = bench.WORKLOADS[workload]
    lens = bench.route(spec)
    G, M = spec["G"], sum(lens)
    dense = spec["routing"] == "dense"
    k, n = ((spec["hidden"], spec["fc1_out"]), (spec["fc2_in"], spec["hidden"]))[layer]
    fp4 = spec["fp4"]
    a_fmt, w_fmt = o.FMT_E4M3, (o.FMT_E2M1 if fp4 else o.FMT_E4M3)
    tol = 3e-2 if fp4 else 1e-2
    if fp4:
        cfg = Float4QuantConfig(activation_format=Format.E4M3)
    else:
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
    rng = np.random.default_rng(spec["seed"] + layer)
    # the benchmark's own recipe per tensor (for the Llama MLP: activations with 0.1 % of the entries times 50), drawn
    # from a device generator here: a CPU draw of these sizes would take most of the suite's time
    gen = torch.Generator(device=gpu).manual_seed(spec["seed"] + 17 * layer)
    x, w, dy, _, _ = bench.synth_layer(spec, layer, M, gen, gpu)
    if spec.get("outliers"):
        big = (x.float().abs() > 8).float().mean().item()
        assert 5e-4 < big < 1.5e-3, big          # N(0, 1) alone puts nothing there
    gl = None if dense else torch.tensor(lens, dtype=torch.int64, device=gpu)
    glens = [M] if dense else lens

    # ---- (1) quantised operands, bit-exact on sampled bands ----
    xq, xs, xqT, xsT = K.quantize_mx_impl(x, a_fmt, rowwise=True, colwise=True, group_lens=gl, pad_to=K.GEMM_K_ALIGN)
    dq, ds, dqT, dsT = K.quantize_mx_impl(dy, a_fmt, rowwise=True, colwise=True, group_lens=gl, pad_to=K.GEMM_K_ALIGN)
    wq, ws, wqT, wsT = K.quantize_mx_weight_2d_impl(w, w_fmt, rowwise=True, colwise=True, pad_to=K.GEMM_K_ALIGN)
    kp = k if k % 128 == 0 else (k + 127) // 128 * 128   # padded contraction width of the row-wise copies
    rows = _sample_rows(glens, rng)
    ridx = torch.tensor(rows, device=gpu)
    for src, q, s, width in ((x, xq, xs, k), (dy, dq, ds, n)):
        oq, os_ = o.quantize_mx_rowwise(src[ridx].cpu(), a_fmt)
        assert np.array_equal(_u8(q)[ridx].cpu().numpy()[:, :width], oq)
        assert np.array_equal(_u8(s)[ridx].cpu().numpy()[:, : width // 32], os_)
        assert not _u8(q)[ridx][:, width:].any()          # GEMM padding: zero codes, scale byte 0
        assert not _u8(s)[ridx][:, width // 32:].any()
    # transposed copies: whole 128-token bands at expert starts / ends, all columns of a sampled column band
    _, seg_off = o.segment_layout(glens)   # start of every expert's segment in the padded transposed layout
    c0 = int(rng.integers(0, k // 32)) * 32
    picked = [g for g, ln in enumerate(glens) if ln > 0][:3] + [g for g, ln in enumerate(glens) if ln > 0][-1:]
    off_rows = np.concatenate([[0], np.cumsum(glens)])
    for g in sorted(set(picked)):
        r0, ln = int(off_rows[g]), glens[g]
        band = x[r0 : r0 + ln, c0 : c0 + 32].cpu()
        oqT, osT = o.quantize_mx_colwise_segmented(band, [ln], a_fmt)
        p0 = int(seg_off[g])
        wpad = oqT.shape[1]                                   # ln rounded up to 128
        got_q = _u8(xqT)[c0 : c0 + 32, p0 : p0 + wpad].cpu().numpy()
        got_s = _u8(xsT)[c0 : c0 + 32, p0 // 32 : (p0 + wpad) // 32].cpu().numpy()
        assert np.array_equal(got_q, oqT) and np.array_equal(got_s, osT), (workload, g)
    # weights: one 2-D tile row band of a sampled expert, both copies
    e = int(rng.integers(0, 1 if dense else G))
    n0 = int(rng.integers(0, n // 32)) * 32
    wb = (w if dense else w[e])[n0 : n0 + 32].cpu()
    oq, os_, oqT, osT = o.quantize_mx_2d(wb, w_fmt)
    per = 2 if w_fmt == o.FMT_E2M1 else 1
    wq_e, ws_e, wqT_e, wsT_e = ((wq, ws, wqT, wsT) if dense else (wq[e], ws[e], wqT[e], wsT[e]))
    assert np.array_equal(_u8(wq_e)[n0 : n0 + 32].cpu().numpy()[:, : k // per], oq)
    assert np.array_equal(_u8(ws_e)[n0 : n0 + 32].cpu().numpy()[:, : k // 32], os_)
    assert np.array_equal(_u8(wqT_e)[:, n0 // per : (n0 + 32) // per].cpu().numpy(), oqT)
    assert np.array_equal(_u8(wsT_e)[:, n0 // 32 : n0 // 32 + 1].cpu().numpy(), osT)

    # ---- (2) the differentiable op at full size; sampled outputs against the oracle ----
    xg, wg = x.clone().requires_grad_(), w.clone().requires_grad_()
    if dense:
        y = pt.ops.gemm_fp8(xg, wg, trans_a=False, trans_b=True, out_dtype=None, config=cfg)
    elif fp4:
        y = pt.ops.grouped_gemm_fp4(xg, wg, gl, trans_b=True, config=cfg)
    else:
        y = pt.ops.grouped_gemm_fp8(xg, wg, gl, trans_b=True, config=cfg)
    y.backward(dy)
    dx, dw = xg.grad, wg.grad
    assert torch.isfinite(y.float()).all() and torch.isfinite(dx.float()).all() and torch.isfinite(dw.float()).all()

    cols_n = np.sort(rng.choice(n, size=48, replace=False))
    cols_k = np.sort(rng.choice(k, size=48, replace=False))
    cn, ck = torch.tensor(cols_n, device=gpu), torch.tensor(cols_k, device=gpu)
    a_rows = _deq_rows(_u8(xq)[ridx].cpu().numpy(), _u8(xs)[ridx].cpu().numpy(), a_fmt)        # [R, kp]
    d_rows = _deq_rows(_u8(dq)[ridx].cpu().numpy(), _u8(ds)[ridx].cpu().numpy(), a_fmt)        # [R, np]
    y_s, dx_s = _bf(y[ridx][:, cn]), _bf(dx[ridx][:, ck])
    want_y, want_dx = np.zeros_like(y_s), np.zeros_like(dx_s)
    abs_y, abs_dx = np.zeros_like(y_s), np.zeros_like(dx_s)      # sum |a_i b_i| of every sampled output
    cache = {}
    for i, r in enumerate(rows):
        g, _ = _group_of(r, glens)
        if g not in cache:
            we = (wq, ws, wqT, wsT) if dense else (wq[g], ws[g], wqT[g], wsT[g])
            b_fwd = _deq_rows(_u8(we[0])[cn].cpu().numpy(), _u8(we[1])[cn].cpu().numpy(), w_fmt)   # [48, kp]
            b_bwd = _deq_rows(_u8(we[2])[ck].cpu().numpy(), _u8(we[3])[ck].cpu().numpy(), w_fmt)   # [48, np]
            cache[g] = (b_fwd, b_bwd)
        want_y[i] = cache[g][0] @ a_rows[i]
        want_dx[i] = cache[g][1] @ d_rows[i]
        abs_y[i] = np.abs(cache[g][0]) @ np.abs(a_rows[i])
        abs_dx[i] = np.abs(cache[g][1]) @ np.abs(d_rows[i])
    assert np.abs(y_s - want_y).max() <= tol * np.abs(want_y).max()
    assert np.abs(dx_s - want_dx).max() <= tol * np.abs(want_dx).max()
    # per element: the output's own bf16 rounding plus the accumulation-order error of the contraction
    assert (np.abs(y_s - want_y) <= _elementwise_bound(want_y, abs_y, kp)).all()
    assert (np.abs(dx_s - want_dx) <= _elementwise_bound(want_dx, abs_dx, d_rows.shape[1])).all()

    # wgrad: sampled (n, k) positions of up to three experts, contraction over the expert's padded segment
    for g in sorted(set(picked))[:3]:
        p0, ln = int(seg_off[g]), glens[g]
        wpad = (ln + 127) // 128 * 128
        a_t = _deq_rows(_u8(dqT)[cn][:, p0 : p0 + wpad].cpu().numpy(), _u8(dsT)[cn][:, p0 // 32 : (p0 + wpad) // 32].cpu().numpy(), a_fmt)
        b_t = _deq_rows(_u8(xqT)[ck][:, p0 : p0 + wpad].cpu().numpy(), _u8(xsT)[ck][:, p0 // 32 : (p0 + wpad) // 32].cpu().numpy(), a_fmt)
        want = a_t @ b_t.T
        got = _bf((dw if dense else dw[g])[cn][:, ck])
        assert np.abs(got - want).max() <= tol * np.abs(want).max(), (workload, g)
        assert (np.abs(got - want) <= _elementwise_bound(want, np.abs(a_t) @ np.abs(b_t).T, wpad)).all(), (workload, g)

    # ---- (3) properties ----
    if not dense:
        for g, ln in enumerate(glens):
            if ln == 0:
                assert not dw[g].any()
        assert y.shape == (M, n) and dx.shape == (M, k) and dw.shape == (G, n, k)


def _exact_codes(gen, rows, k, dev):
    """E4M3 codes of small integers (0, +-1, +-2, +-3, 4) and scales 2^-1..2^1: every product and every
    partial sum over a few thousand of them is exact in fp32, whatever the accumulation order."""
    vals = torch.tensor([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=torch.uint8, device=dev)
    q = vals[torch.randint(0, 8, (rows, k), generator=gen, device=dev)]
    s = torch.randint(126, 129, (rows, k // 32), generator=gen, device=dev, dtype=torch.uint8)
    return q.view(torch.float8_e4m3fn), s.view(torch.float8_e8m0fnu)


def test_full_size_mixtral_every_output_bit_exact(gpu):
    """Mixtral fc1 at full size (32 768 routed rows, ragged over 8 experts, [8, 28672, 4096] weights) on
    exactly representable operands: EVERY element of the forward output and of the weight gradient
    equals the fp32 matrix product of the dequantised operands bit for bit (the exact result does not
    depend on summation order, so the fp32 library GEMM is a valid reference at this size, where the
    CPU oracle would need hours; the dequantiser used to build it is itself tested against the oracle)."""
    from primus_amd.pytorch import kernels as K

    spec = bench.WORKLOADS["mixtral_8x7b_moe_mxfp8"]
    lens = bench.route(spec)
    G, M, k, n = spec["G"], sum(lens), spec["hidden"], spec["fc1_out"]
    gen = torch.Generator(device=gpu).manual_seed(77)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    offs = np.concatenate([[0], np.cumsum(lens)])

    # forward: Y = X . W_g^T per expert
    xq, xs = _exact_codes(gen, M, k, gpu)
    wq, ws = _exact_codes(gen, G * n, k, gpu)
    y = K.grouped_gemm_mx_nt_impl(xq, xs, wq.view(G, n, k), ws.view(G, n, k // 32), gl)
    xf = K.dequantize_mx_impl(xq, xs).float()
    wf = K.dequantize_mx_impl(wq, ws).float().view(G, n, k)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        want = (xf[a:b] @ wf[g].T).bfloat16()
        assert torch.equal(y[a:b], want), g
    del y, wq, ws, wf

    # wgrad: dW_g = dY_g^T . X_g on the segment-padded transposed layout (zero codes in the padding).  Row-wise
    # scales do not transpose into per-32-token blocks, so the transposed operands reuse the CODES with scale 1.
    W = K.padded_width(M, G)
    _, poffs = o.segment_layout(lens)
    nd = 512                                                      # a 512-column slice of dY keeps the test short
    dq, _ = _exact_codes(gen, M, nd, gpu)

    def unit_scales(rows, cols):
        return torch.full((rows, cols // 32), 127, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)

    def transposed(codes_rows):
        cols = codes_rows.shape[1]
        qT = torch.zeros(cols, W, dtype=torch.uint8, device=gpu)
        for g in range(G):
            a, b, p = int(offs[g]), int(offs[g + 1]), int(poffs[g])
            qT[:, p : p + (b - a)] = codes_rows.view(torch.uint8)[a:b].T
        return qT.view(torch.float8_e4m3fn), unit_scales(cols, W)

    dyf = K.dequantize_mx_impl(dq, unit_scales(M, nd)).float()
    xf1 = K.dequantize_mx_impl(xq, unit_scales(M, k)).float()
    dqT, dsT = transposed(dq)
    xqT, xsT = transposed(xq)
    dw = K.grouped_gemm_mx_wgrad_impl(dqT, dsT, xqT, xsT, gl, M)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        want = (dyf[a:b].T @ xf1[a:b]).bfloat16()
        assert torch.equal(dw[g], want), g


def _chunk(codes):
    """Row-major codes [rows, k] -> K-chunk-major [k / 128, rows, 128] (FP8: one byte per element)."""
    rows, k = codes.shape
    return codes.view(torch.uint8).reshape(rows, k // 128, 128).permute(1, 0, 2).contiguous().view(codes.dtype)


def test_full_size_mixtral_chunked_scaled_and_accumulating_bit_exact(gpu):
    """The same full-size case through the later kernel variants: K-chunk-major operands, the scaled GEMM
    with E5M2 x E4M3 operands and per-tensor factors, and the wgrad that adds into a float32 buffer --
    every output element exact (small-integer codes, power-of-two factors, integer buffer contents)."""
    from primus_amd.pytorch import kernels as K

    spec = bench.WORKLOADS["mixtral_8x7b_moe_mxfp8"]
    lens = bench.route(spec)
    G, M, k, n = spec["G"], sum(lens), spec["hidden"], spec["fc1_out"]
    gen = torch.Generator(device=gpu).manual_seed(78)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    offs = np.concatenate([[0], np.cumsum(lens)])
    e5 = torch.tensor([0x00, 0x3C, 0x40, 0x42, 0x44, 0xBC, 0xC0, 0xC2], dtype=torch.uint8, device=gpu)   # 0, +-1, +-2, +-3, 4
    e5val = torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0, -1.0, -2.0, -3.0], device=gpu)

    def unit(rows, cols):
        return torch.full((rows, cols // 32), 127, dtype=torch.uint8, device=gpu).view(torch.float8_e8m0fnu)

    # forward-shaped: a = E5M2 codes [M, k] (chunked), b = E4M3 weights [G, n, k] (chunked), factors 0.5 and 0.25
    idx = torch.randint(0, 8, (M, k), generator=gen, device=gpu)
    a_codes, af = e5[idx].view(torch.float8_e5m2), e5val[idx]
    wq, _ = _exact_codes(gen, G * n, k, gpu)
    wf = K.dequantize_mx_impl(wq, unit(G * n, k)).float().view(G, n, k)
    sa, sb = torch.tensor([0.5], device=gpu), torch.tensor([0.25], device=gpu)
    y = K.gemm_tw_nt_impl(_chunk(a_codes), unit(M, k), sa, _chunk(wq), unit(G * n, k).view(G, n, k // 32), sb, gl, kchunk=True)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        assert torch.equal(y[a:b], ((af[a:b] @ wf[g].T) * 0.125).bfloat16()), g
    del y, wq, wf, idx

    # wgrad-shaped, accumulating: buf[g] += dY_g^T . X_g for a 512-column slice of dY, MX entry point
    W = K.padded_width(M, G)
    _, poffs = o.segment_layout(lens)
    nd = 512
    dq, _ = _exact_codes(gen, M, nd, gpu)
    xq, _ = _exact_codes(gen, M, k, gpu)

    def transposed_chunked(codes_rows):
        cols = codes_rows.shape[1]
        qT = torch.zeros(cols, W, dtype=torch.uint8, device=gpu)
        for g in range(G):
            a, b, p = int(offs[g]), int(offs[g + 1]), int(poffs[g])
            qT[:, p : p + (b - a)] = codes_rows.view(torch.uint8)[a:b].T
        return _chunk(qT.view(torch.float8_e4m3fn)), unit(cols, W)

    dyf = K.dequantize_mx_impl(dq, unit(M, nd)).float()
    xf = K.dequantize_mx_impl(xq, unit(M, k)).float()
    before = torch.randint(-1000, 1000, (G, nd, k), generator=gen, device=gpu).float()
    buf = before.clone()
    dqT, dsT = transposed_chunked(dq)
    xqT, xsT = transposed_chunked(xq)
    K.grouped_gemm_mx_wgrad_impl(dqT, dsT, xqT, xsT, gl, M, kchunk=True, accum_into=buf)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        assert torch.equal(buf[g], before[g] + dyf[a:b].T @ xf[a:b]), g


@pytest.mark.parametrize("fmt,layout", [(0, 2), (1, 3)])
def test_full_size_mixtral_ring_kernel_bit_exact(gpu, fmt, layout):
    """The full-size Mixtral fc1 through the quantisers and the 4-slot ring kernel (K-step-major operands: MXFP8 in
    64-element steps, MXFP4 x MXFP4 in 128-element steps): forward, dgrad and a 512-column slice of the weight gradient,
    EVERY output element.  The inputs are small integers (|v| <= 4) times a power of two per tensor: whatever a block's
    largest magnitude is, its E8M0 scale leaves every element on an E4M3 / E2M1 code, so quantisation is exact, every
    partial sum is an integer below 2^24, and the fp32 matrix product of the bf16 inputs is the exact result in any
    summation order."""
    from primus_amd.pytorch import kernels as K

    spec = bench.WORKLOADS["mixtral_8x7b_moe_mxfp8"]
    lens = bench.route(spec)
    G, M, k, n = spec["G"], sum(lens), spec["hidden"], spec["fc1_out"]
    gen = torch.Generator(device=gpu).manual_seed(79 + fmt)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    offs = np.concatenate([[0], np.cumsum(lens)])

    def ints(rows, cols, factor):
        return (torch.randint(-4, 5, (rows, cols), generator=gen, device=gpu).float() * factor).bfloat16()

    x = ints(M, k, 0.5)
    w = ints(G * n, k, 0.25).view(G, n, k)
    xq = K.quantize_mx_impl(x, fmt, rowwise=True, colwise=True, group_lens=gl, kchunk=layout)
    wq = K.quantize_mx_weight_2d_impl(w, fmt, rowwise=True, colwise=True, kchunk=layout)
    y = K.grouped_gemm_mx_nt_impl(xq[0], xq[1], wq[0], wq[1], gl, kchunk=layout)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        assert torch.equal(y[a:b], (x[a:b].float() @ w[g].float().T).bfloat16()), ("fwd", g)
    del y
    # dgrad: dX = dY . W_g (contraction over n = 28672)
    dy = ints(M, n, 2.0)
    dq = K.quantize_mx_impl(dy, fmt, rowwise=True, colwise=False, group_lens=gl, kchunk=layout)
    dx = K.grouped_gemm_mx_nt_impl(dq[0], dq[1], wq[2], wq[3], gl, kchunk=layout)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        assert torch.equal(dx[a:b], (dy[a:b].float() @ w[g].float()).bfloat16()), ("dgrad", g)
    del dx, dq, wq
    # wgrad on a 512-column slice of dY: dW_g = dY_g^T . X_g over the group's (padded) token segment
    dys = dy[:, :512].contiguous()
    dqs = K.quantize_mx_impl(dys, fmt, rowwise=False, colwise=True, group_lens=gl, kchunk=layout)
    dw = K.grouped_gemm_mx_wgrad_impl(dqs[2], dqs[3], xq[2], xq[3], gl, M, kchunk=layout)
    for g in range(G):
        a, b = int(offs[g]), int(offs[g + 1])
        assert torch.equal(dw[g], (dys[a:b].float().T @ x[a:b].float()).bfloat16()), ("wgrad", g)
