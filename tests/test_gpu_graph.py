"""The operators under HIP graph capture: tokens-per-expert stays on the device and no entry point
allocates, synchronises or reads device memory from the host, so a captured forward + backward can be
replayed on new inputs AND new routing.  Every replay is checked against the eager result."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _cfg(fp4):
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    if fp4:
        return Float4QuantConfig(format=Format.E2M1_X2, granularity=ScalingGranularity.MX_BLOCKWISE,
                                 scale_dtype=ScaleDtype.E8M0, block_size=32)
    return Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0,
                             block_size=32)


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("overlap", [True, False])
def test_grouped_linear_replays_with_new_routing(gpu, fp4, overlap):
    import primus_amd.pytorch as turbo

    op = turbo.ops.grouped_gemm_fp4 if fp4 else turbo.ops.grouped_gemm_fp8
    cfg = _cfg(fp4)
    G, n, k, rows = 4, 384, 256, 700
    gen = torch.Generator().manual_seed(11)
    x = torch.randn(rows, k, generator=gen).bfloat16().to(gpu).requires_grad_()
    w = (torch.randn(G, n, k, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(rows, n, generator=gen).bfloat16().to(gpu)
    lens = torch.tensor([100, 0, 343, 257], dtype=torch.int64, device=gpu)

    def step():
        y = op(x, w, lens, config=cfg)
        dx, dw = torch.autograd.grad(y, [x, w], dy)
        return y, dx, dw

    turbo.ops.set_wgrad_overlap(overlap)
    try:
        # warm-up on a side stream, as torch asks for before a capture
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = step()
        cases = [([100, 0, 343, 257], 1), ([0, 0, 0, 700], 2), ([175, 175, 175, 175], 3), ([699, 1, 0, 0], 4),
                 ([100, 0, 343, 257], 5)]
        for new_lens, seed in cases:
            g2 = torch.Generator().manual_seed(seed)
            with torch.no_grad():
                x.copy_(torch.randn(rows, k, generator=g2).bfloat16())
                w.copy_((torch.randn(G, n, k, generator=g2) * 0.05).bfloat16())
                dy.copy_(torch.randn(rows, n, generator=g2).bfloat16())
                lens.copy_(torch.tensor(new_lens, dtype=torch.int64))
            graph.replay()
            torch.cuda.synchronize()
            got = [t.clone() for t in outs]
            want = step()          # eager work and a synchronisation between the replays
            torch.cuda.synchronize()
            for a, b in zip(got, want):
                assert _same(a, b), (new_lens, seed)
    finally:
        turbo.ops.set_wgrad_overlap(True)


def test_dense_and_fused_activation_replay(gpu):
    import primus_amd.pytorch as turbo

    cfg = _cfg(False)
    rows, f, n, G = 512, 256, 128, 2
    gen = torch.Generator().manual_seed(5)
    h = torch.randn(rows, 2 * f, generator=gen).bfloat16().to(gpu).requires_grad_()
    probs = torch.rand(rows, generator=gen).to(gpu).requires_grad_()
    w2 = (torch.randn(G, n, f, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    wd = (torch.randn(2 * f, n, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(rows, 2 * f, generator=gen).bfloat16().to(gpu)
    lens = torch.tensor([200, 312], dtype=torch.int64, device=gpu)

    def step():
        y = turbo.ops.glu_grouped_gemm_fp8(h, probs, w2, lens, config=cfg)      # [rows, n]
        z = turbo.ops.gemm_fp8(y, wd, config=cfg)                                # [rows, 2f]
        return (z,) + torch.autograd.grad(z, [h, probs, w2, wd], dy)

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for new_lens, seed in [([200, 312], 1), ([512, 0], 2), ([1, 511], 3)]:
        g2 = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            h.copy_(torch.randn(rows, 2 * f, generator=g2).bfloat16())
            probs.copy_(torch.rand(rows, generator=g2))
            lens.copy_(torch.tensor(new_lens, dtype=torch.int64))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert _same(a, b), (new_lens, seed)


@pytest.mark.parametrize("recipe", ["tensorwise", "mxfp8"])
def test_tensorwise_norm_and_fused_accumulation_replay(gpu, recipe):
    """The later additions under capture: the tensor-wise recipe (abs-max by atomics into a kernel-initialised
    word), the RMSNorm folded into the quantiser and the wgrad that adds into a float32 main_grad."""
    import primus_amd.pytorch as turbo
    from primus_amd.pytorch.core import Float8QuantConfig, Format, ScalingGranularity

    cfg = (Float8QuantConfig(format=Format.HYBRID, granularity=ScalingGranularity.TENSORWISE) if recipe == "tensorwise"
           else _cfg(False))
    G, n, k, rows = 3, 256, 256, 600
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(rows, k, generator=gen).bfloat16().to(gpu).requires_grad_()
    nw = (1 + 0.1 * torch.randn(k, generator=gen)).bfloat16().to(gpu).requires_grad_()
    w1 = (torch.randn(k, k, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    w2 = (torch.randn(G, n, k, generator=gen) * 0.05).bfloat16().to(gpu).requires_grad_()
    dy = torch.randn(rows, n, generator=gen).bfloat16().to(gpu)
    lens = torch.tensor([100, 0, 500], dtype=torch.int64, device=gpu)
    w2.main_grad = torch.zeros(G, n, k, device=gpu)
    w2.grad_added_to_main_grad = False

    def step():
        if recipe == "tensorwise":
            h = turbo.ops.gemm_fp8(turbo.ops.rmsnorm(x, nw, 1e-5), w1, config=cfg)
        else:
            h = turbo.ops.rmsnorm_gemm_fp8(x, nw, 1e-5, w1, config=cfg)
        y = turbo.ops.grouped_gemm_fp8(h, w2, lens, config=cfg, fuse_bgrad_accum_pattern="megatron")
        return (y,) + torch.autograd.grad(y, [x, nw, w1, w2], dy)[:3]

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for new_lens, seed in [([100, 0, 500], 1), ([600, 0, 0], 2), ([1, 299, 300], 3)]:
        g2 = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            x.copy_(torch.randn(rows, k, generator=g2).bfloat16() * (seed * 3.0))     # the abs-max changes too
            dy.copy_(torch.randn(rows, n, generator=g2).bfloat16())
            lens.copy_(torch.tensor(new_lens, dtype=torch.int64))
            w2.main_grad.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs] + [w2.main_grad.clone()]
        with torch.no_grad():
            w2.main_grad.zero_()
        want = list(step()) + [w2.main_grad.clone()]
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert _same(a, b), (new_lens, seed)
        assert got[-1].abs().sum() > 0


def test_expert_mlp_with_explicit_padding_replays_with_new_routing(gpu):
    """The expert MLP on its explicit-padding route (groups padded to 32 rows on the device, fc1, the activation, fc2,
    unpadding) captured once and replayed with other tokens and other tokens-per-expert: nothing in it reads the
    counts on the host."""
    from types import SimpleNamespace

    from primus_amd.megatron import runtime
    from primus_amd.megatron.extensions import primus_turbo as pt
    from primus_amd.megatron.transformer.experts import PrimusGroupedMLP
    from primus_amd.pytorch.core import Format, ScaleDtype, ScalingGranularity

    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.bind()
    runtime.set_num_microbatches(1)
    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=False, use_turbo_fused_act_with_probs=True)
    try:
        torch.manual_seed(23)
        cfg = SimpleNamespace(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                              tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                              layernorm_epsilon=1e-5, hidden_size=256, ffn_hidden_size=384, moe_ffn_hidden_size=384,
                              gated_linear_unit=True, fp8="e4m3", fp8_recipe="mxfp8", fp4=None, add_bias_linear=False)
        mlp = PrimusGroupedMLP(4, cfg)
        assert mlp._use_explicit_quantization_padding()
        qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E4M3, block_size=32,
                                       scale_dtype=ScaleDtype.E8M0)
        rows = 500
        gen = torch.Generator().manual_seed(4)
        x = torch.randn(rows, 256, generator=gen).bfloat16().to(gpu).requires_grad_()
        probs = torch.rand(rows, generator=gen).to(gpu).requires_grad_()
        dy = torch.randn(rows, 256, generator=gen).bfloat16().to(gpu)
        lens = torch.tensor([100, 0, 143, 257], dtype=torch.int64, device=gpu)
        params = [mlp.linear_fc1.weights, mlp.linear_fc2.weights]

        def step():
            for lin in (mlp.linear_fc1, mlp.linear_fc2):
                lin.set_is_first_microbatch()
            with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
                y, _ = mlp(x, lens, probs)
            return (y,) + torch.autograd.grad(y, [x, probs] + params, dy)

        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = step()
        for new_lens, seed in [([100, 0, 143, 257], 1), ([0, 0, 0, 500], 2), ([125, 125, 125, 125], 3), ([499, 1, 0, 0], 4)]:
            g2 = torch.Generator().manual_seed(seed)
            with torch.no_grad():
                x.copy_(torch.randn(rows, 256, generator=g2).bfloat16())
                probs.copy_(torch.rand(rows, generator=g2))
                dy.copy_(torch.randn(rows, 256, generator=g2).bfloat16())
                lens.copy_(torch.tensor(new_lens, dtype=torch.int64))
            graph.replay()
            torch.cuda.synchronize()
            got = [t.clone() for t in outs]
            want = step()
            torch.cuda.synchronize()
            for a, b in zip(got, want):
                assert _same(a, b), (new_lens, seed)
            assert got[0].abs().sum() > 0
    finally:
        pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
        runtime.set_args()
