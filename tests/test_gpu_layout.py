"""The K-chunk-major code layout ([ld / 128, rows, 128] instead of [rows, ld]): the quantisers write the
same codes, only arranged differently, and the GEMMs give the same results bit for bit on either layout."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _same(a, b):
    return a.dtype == b.dtype and torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("lens,cols", [([33, 0, 130, 1, 92], 160), ([300], 2048), (None, 64), ([0, 0], 96), ([257, 255], 384)])
def test_quantiser_kchunk_is_a_rearrangement(gpu, fmt, lens, cols):
    from primus_amd.pytorch import kernels as K

    rows = 257 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-2, 2, cols)[None, :]).bfloat16().to(gpu)
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    a = K.quantize_mx_impl(x, fmt, rowwise=True, colwise=True, group_lens=gl, pad_to=128)
    b = K.quantize_mx_impl(x, fmt, rowwise=True, colwise=True, group_lens=gl, kchunk=True)
    assert b[0].dim() == 3 and b[0].shape[1] == rows and b[2].dim() == 3 and b[2].shape[1] == cols
    assert _same(K.unchunk(b[0]), a[0]) and _same(b[1], a[1])
    assert _same(K.unchunk(b[2]), a[2]) and _same(b[3], a[3])
    if rows:
        r = K.quantize_mx_impl(x, fmt, rowwise=True, colwise=False, kchunk=True)
        assert _same(r[0], b[0])
    c = K.quantize_mx_impl(x, fmt, rowwise=False, colwise=True, group_lens=gl, kchunk=True)
    assert _same(c[2], b[2])
    if fmt == 1:
        e = K.quantize_mx_impl(x, 1, rowwise=True, colwise=True, group_lens=gl, pad_to=128, sr_seed=5, rht_signs=0x1234)
        f = K.quantize_mx_impl(x, 1, rowwise=True, colwise=True, group_lens=gl, kchunk=True, sr_seed=5, rht_signs=0x1234)
        assert _same(K.unchunk(f[0]), e[0]) and _same(K.unchunk(f[2]), e[2])


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("shape", [(96, 160), (3, 256, 128), (2, 416, 288), (1, 32, 32)])
def test_weight_quantiser_kchunk_is_a_rearrangement(gpu, fmt, shape):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(sum(shape))
    w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().to(gpu)
    n, k = shape[-2], shape[-1]
    a = K.quantize_mx_weight_2d_impl(w, fmt, rowwise=True, colwise=True, pad_to=128)
    b = K.quantize_mx_weight_2d_impl(w, fmt, rowwise=True, colwise=True, kchunk=True)
    assert _same(K.unchunk(b[0]), a[0].reshape(-1, a[0].shape[-1])) and _same(b[1], a[1])
    assert _same(K.unchunk(b[2]), a[2].reshape(-1, a[2].shape[-1])) and _same(b[3], a[3])


def test_quantisers_write_the_128_element_step_layout_of_e2m1(gpu):
    """Layout 3 holds the codes of the K-chunk-major layout and the scale panels of the K-step-major one."""
    from primus_amd.pytorch import kernels as K

    lens, cols = [33, 0, 130, 1, 92, 600], 672
    rows = sum(lens)
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-2, 2, cols)[None, :]).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    a = K.quantize_mx_impl(x, 1, rowwise=True, colwise=True, group_lens=gl, kchunk=True)
    b = K.quantize_mx_impl(x, 1, rowwise=True, colwise=True, group_lens=gl, kchunk=3)
    assert _same(b[0], a[0]) and _same(b[2], a[2])
    assert _same(K.unpanel(b[1].view(torch.uint8), a[1].shape[1]), a[1].view(torch.uint8))
    # the transposed copy's panels restart at every group: compare group by group
    W, off, pan = a[3].shape[1] * 32, 0, 0
    s_col = b[3].view(torch.uint8)
    for ln in lens:
        seg = (ln + 127) // 128 * 128
        npan = (seg // 128 + 3) // 4
        if seg:
            got = K.unpanel(s_col[pan:pan + npan], seg // 32)
            assert torch.equal(got, a[3].view(torch.uint8)[:, off // 32:(off + seg) // 32])
        off, pan = off + seg, pan + npan
    w = (torch.randn(2, 416, 288, generator=g) * 0.05).bfloat16().to(gpu)
    wa = K.quantize_mx_weight_2d_impl(w, 1, rowwise=True, colwise=True, kchunk=True)
    wb = K.quantize_mx_weight_2d_impl(w, 1, rowwise=True, colwise=True, kchunk=3)
    assert _same(wb[0], wa[0]) and _same(wb[2], wa[2])
    assert _same(K.unpanel(wb[1].view(torch.uint8), wa[1].shape[-1]), wa[1].reshape(-1, wa[1].shape[-1]).view(torch.uint8))
    assert _same(K.unpanel(wb[3].view(torch.uint8), wa[3].shape[-1]), wa[3].reshape(-1, wa[3].shape[-1]).view(torch.uint8))
    with pytest.raises(ValueError):
        K.quantize_mx_impl(x, 0, rowwise=True, colwise=False, kchunk=3)


@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_fused_activation_quantiser_kchunk(gpu, activation):
    from primus_amd.pytorch import kernels as K

    lens, f = [33, 0, 130, 1, 92], 160
    rows = sum(lens)
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(rows, 2 * f, generator=g) * 2).bfloat16().to(gpu)
    p = torch.rand(rows, generator=g).to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    a = K.glu_with_probs_quantize_impl(x, p, None, activation, 0, colwise=True, group_lens=gl, pad_to=128)
    b = K.glu_with_probs_quantize_impl(x, p, None, activation, 0, colwise=True, group_lens=gl, kchunk=True)
    assert _same(K.unchunk(b[0]), a[0]) and _same(K.unchunk(b[2]), a[2]) and _same(b[1], a[1]) and _same(b[3], a[3])


@pytest.mark.parametrize("afmt,wfmt", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("lens,n,k", [([33, 0, 130, 1, 92], 96, 160), ([300, 212], 544, 512), (None, 320, 384),
                                      ([1500, 0, 700, 2048, 300, 1024], 2048, 1024),
                                      # 200 groups: beyond 128, still on the ring kernel (its tables take 256)
                                      ([(37 * i) % 97 if i % 5 else 0 for i in range(200)], 160, 256)])
def test_gemms_give_identical_results_on_either_layout(gpu, afmt, wfmt, lens, n, k):
    """Forward, dgrad and wgrad from K-chunk-major operands equal those from row-major operands bit for bit
    (same codes, same scales, same MFMA sequence; only the addresses of the operand loads differ)."""
    from primus_amd.pytorch import kernels as K

    m = 257 if lens is None else sum(lens)
    G = 1 if lens is None else len(lens)
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16().to(gpu)
    dy = torch.randn(m, n, generator=g).bfloat16().to(gpu)
    w = (torch.randn(G, n, k, generator=g) * 0.05).bfloat16().to(gpu)
    gl = None if lens is None else torch.tensor(lens, dtype=torch.int64, device=gpu)
    res = []
    # 2: K-step-major codes and scales (the 4-slot ring kernel): FP8 activations against FP8 or FP4 weights;
    # 3: the same with steps of 128 elements: E2M1 against E2M1 (1, 2, 3, 5, 8 and 16 steps per tile in these cases)
    for kc in (False, True) + ((2,) if afmt == 0 else ()) + ((3,) if afmt == 1 and wfmt == 1 else ()):
        xq = K.quantize_mx_impl(x, afmt, rowwise=True, colwise=True, group_lens=gl, pad_to=128, kchunk=kc)
        dq = K.quantize_mx_impl(dy, afmt, rowwise=True, colwise=True, group_lens=gl, pad_to=128, kchunk=kc)
        wq = K.quantize_mx_weight_2d_impl(w, wfmt, rowwise=True, colwise=True, pad_to=128, kchunk=kc)
        if lens is None:
            ws_row, ws_col = (wq[1], wq[3]) if kc in (2, 3) else (wq[1][0], wq[3][0])
            w_row = wq[0] if kc else wq[0][0]
            w_col = wq[2] if kc else wq[2][0]
            y = K.gemm_mx_nt_impl(xq[0], xq[1], w_row, ws_row, kchunk=kc)
            dx = K.gemm_mx_nt_impl(dq[0], dq[1], w_col, ws_col, kchunk=kc)
        else:
            y = K.grouped_gemm_mx_nt_impl(xq[0], xq[1], wq[0], wq[1], gl, kchunk=kc)
            dx = K.grouped_gemm_mx_nt_impl(dq[0], dq[1], wq[2], wq[3], gl, kchunk=kc)
        dw = K.grouped_gemm_mx_wgrad_impl(dq[2], dq[3], xq[2], xq[3], gl, m, kchunk=kc)
        res.append((y, dx[:, :k], dw))
    for other in res[1:]:
        for a, b in zip(res[0], other):
            assert a.shape == b.shape and torch.equal(a, b)


def test_kchunk_argument_checks(gpu):
    from primus_amd.pytorch import kernels as K

    x = torch.randn(64, 128, device=gpu).bfloat16()
    q = K.quantize_mx_impl(x, 0, rowwise=True, colwise=False, kchunk=True)
    w = K.quantize_mx_weight_2d_impl(x[:32].contiguous(), 0, rowwise=True, colwise=False, kchunk=True)
    with pytest.raises(ValueError):
        K.gemm_mx_nt_impl(K.unchunk(q[0]), q[1], w[0], w[1], kchunk=True)          # row-major codes passed as chunk-major
    with pytest.raises(ValueError):
        K.unchunk(K.unchunk(q[0]))
    y = K.gemm_mx_nt_impl(q[0], q[1], w[0], w[1], kchunk=True)
    assert y.shape == (64, 32)


def _op_run(gpu, fp4, lens, n, k, cached, glu):
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import (Float4QuantConfig, Float8QuantConfig, Format, QuantizedTensorPair, ScaleDtype,
                                         ScalingGranularity, create_quantized_weight, float4_e2m1fn_x2, float8_e4m3)

    if fp4:
        cfg = Float4QuantConfig(format=Format.E2M1_X2, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
        dest = float4_e2m1fn_x2
    else:
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE,
                                scale_dtype=ScaleDtype.E8M0, block_size=32)
        dest = float8_e4m3
    rows = 200 if lens is None else sum(lens)
    g = torch.Generator().manual_seed(rows + n + k)
    x = torch.randn(rows, 2 * k if glu else k, generator=g).bfloat16().to(gpu).requires_grad_()
    wshape = (n, k) if lens is None else (len(lens), n, k)
    w = (torch.randn(*wshape, generator=g) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(rows, n, generator=g).bfloat16().to(gpu)
    b = QuantizedTensorPair(*create_quantized_weight(w, dest, cfg)) if cached else w
    if lens is None:
        y = (turbo.ops.gemm_fp4 if fp4 else turbo.ops.gemm_fp8)(x, b, config=cfg)
        probs = None
    else:
        gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
        if glu:
            probs = torch.rand(rows, generator=g).to(gpu).requires_grad_()
            y = (turbo.ops.glu_grouped_gemm_fp4 if fp4 else turbo.ops.glu_grouped_gemm_fp8)(x, probs, b, gl, config=cfg)
        else:
            probs = None
            y = (turbo.ops.grouped_gemm_fp4 if fp4 else turbo.ops.grouped_gemm_fp8)(x, b, gl, config=cfg)
    outs = [y]
    if cached:
        outs += list(torch.autograd.grad(y, [x] + ([probs] if glu else []), dy))
        outs.append(b.data.dequantize())
        outs.append(b.data_t.dequantize())
    else:
        outs += list(torch.autograd.grad(y, [x, w] + ([probs] if glu else []), dy))
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("lens,n,k,glu", [(None, 96, 160, False), ([33, 0, 130, 1, 92], 160, 96, False),
                                          ([257, 255], 384, 256, False), ([33, 0, 130, 1, 92], 96, 160, True),
                                          ([0, 0], 64, 64, False)])
@pytest.mark.parametrize("cached", [False, True])
def test_operators_same_on_both_layouts(gpu, fp4, lens, n, k, glu, cached):
    """The differentiable operators keep their operands K-chunk-major by default; forward, dgrad, wgrad,
    probability gradients and the dequantised weight caches equal the row-major run bit for bit."""
    import primus_amd.pytorch as turbo

    try:
        turbo.ops.set_kchunk_layout(False)
        ref = _op_run(gpu, fp4, lens, n, k, cached, glu)
        turbo.ops.set_kchunk_layout(True)
        out = _op_run(gpu, fp4, lens, n, k, cached, glu)
    finally:
        turbo.ops.set_kchunk_layout(True)
    assert len(ref) == len(out)
    for r, o in zip(ref, out):
        assert r.shape == o.shape and _same(r, o)


def test_cache_layout_decides(gpu):
    """A row-major weight cache is used as it is; a chunked cache still serves a row-major call."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import (Float8QuantConfig, Format, QuantizedTensorPair, ScaleDtype, ScalingGranularity,
                                         create_quantized_weight, float8_e4m3)

    cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0,
                            block_size=32)
    g = torch.Generator().manual_seed(3)
    lens = [70, 0, 58]
    x = torch.randn(sum(lens), 160, generator=g).bfloat16().to(gpu).requires_grad_()
    w = (torch.randn(3, 96, 160, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(sum(lens), 96, generator=g).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    res = []
    for cache_kc, call_kc in [(False, False), (False, True), (True, False), (True, True)]:
        pair = QuantizedTensorPair(*create_quantized_weight(w, float8_e4m3, cfg, kchunk=cache_kc))
        assert pair.data.kchunk == cache_kc and pair.data.codes.dim() == 3
        try:
            turbo.ops.set_kchunk_layout(call_kc)
            y = turbo.ops.grouped_gemm_fp8(x, pair, gl, config=cfg)
            (dx,) = torch.autograd.grad(y, [x], dy)
        finally:
            turbo.ops.set_kchunk_layout(True)
        res.append((y, dx))
    for y, dx in res[1:]:
        assert _same(y, res[0][0]) and _same(dx, res[0][1])


@pytest.mark.parametrize("seed", [7, 8])
def test_operators_same_on_both_layouts_random_shapes(gpu, seed):
    """Seeded sweep of the comparison above: dense and grouped, FP8 / FP4 / mixed, fused activation, cached
    weights, contraction and output dims that need padding, empty and one-row experts."""
    rng = np.random.default_rng(seed)
    import primus_amd.pytorch as turbo

    done = 0
    while done < 40:
        dense = rng.random() < 0.25
        lens = None if dense else [int(v) for v in rng.choice([0, 1, 33, 128, 257, 300], size=int(rng.choice([1, 2, 5, 33])))]
        if lens is not None and sum(lens) == 0:
            continue
        n = int(rng.choice([32, 96, 160, 256, 544]))
        k = int(rng.choice([32, 64, 160, 352, 1024]))
        fp4 = bool(rng.random() < 0.5)
        glu = (not dense) and rng.random() < 0.3
        cached = bool(rng.random() < 0.3)
        try:
            turbo.ops.set_kchunk_layout(False)
            ref = _op_run(gpu, fp4, lens, n, k, cached, glu)
            turbo.ops.set_kchunk_layout(True)
            out = _op_run(gpu, fp4, lens, n, k, cached, glu)
        finally:
            turbo.ops.set_kchunk_layout(True)
        for i, (r, o) in enumerate(zip(ref, out)):
            assert r.shape == o.shape and _same(r, o), (i, fp4, lens, n, k, cached, glu)
        done += 1


@pytest.mark.parametrize("act_fp4", [False, True])
def test_fp4_weight_cache_layout_follows_the_activation_format(gpu, act_fp4):
    """A cached E2M1 weight pair is stored for the GEMM it will meet: 64-element K steps when the config's activations
    are FP8, 128-element steps when they are E2M1.  Either cache dequantises to the same values as a row-major one and
    gives the same forward and input gradient bit for bit."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core import (Float4QuantConfig, Format, QuantizedTensorPair, create_quantized_weight,
                                         float4_e2m1fn_x2)

    cfg = Float4QuantConfig(activation_format=Format.E2M1_X2 if act_fp4 else Format.E4M3)
    g = torch.Generator().manual_seed(11)
    lens = [70, 0, 300, 58]
    x = torch.randn(sum(lens), 160, generator=g).bfloat16().to(gpu).requires_grad_()
    w = (torch.randn(4, 96, 160, generator=g) * 0.05).bfloat16().to(gpu)
    dy = torch.randn(sum(lens), 96, generator=g).bfloat16().to(gpu)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    auto = QuantizedTensorPair(*create_quantized_weight(w, float4_e2m1fn_x2, cfg))
    flat = QuantizedTensorPair(*create_quantized_weight(w, float4_e2m1fn_x2, cfg, kchunk=False))
    assert auto.data.kchunk == (K.LAYOUT_KSTEP128 if act_fp4 else K.LAYOUT_KSTEP) and flat.data.kchunk == 0
    assert _same(auto.data.dequantize(), flat.data.dequantize()) and _same(auto.data_t.dequantize(), flat.data_t.dequantize())
    # a cache made for the other activation format still serves this call (its scales are rearranged on the way)
    other_cfg = Float4QuantConfig(activation_format=Format.E4M3 if act_fp4 else Format.E2M1_X2)
    other = QuantizedTensorPair(*create_quantized_weight(w, float4_e2m1fn_x2, other_cfg))
    assert other.data.kchunk != auto.data.kchunk
    res = []
    for pair in (flat, auto, other):
        y = turbo.ops.grouped_gemm_fp4(x, pair, gl, config=cfg)
        (dx,) = torch.autograd.grad(y, [x], dy)
        res.append((y, dx))
    for y, dx in res[1:]:
        assert _same(res[0][0], y) and _same(res[0][1], dx)

