"""Expert groups padded to the quantisation alignment on the device (mxl_pad_groups / mxl_unpad_groups through
the C-ABI) against the numpy oracle, bit for bit, and the expert MLP's explicit-padding route against the route
that reads the counts on the host as the reference does (experts.py:196-209, :262-264)."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu

CASES = [
    ([5, 0, 33, 64], 32), ([0, 0, 0], 32), ([32], 32), ([1] * 9, 16), ([31, 33, 0, 1, 0], 32), ([100, 257, 0, 27], 16),
    ([7, 0, 0, 0, 0, 0, 0], 1), ([3, 4, 5], 7),
]


def _rand(rows, tail, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.uint8:
        return torch.randint(1, 256, (rows,) + tail, generator=g, dtype=torch.uint8)
    return (torch.rand((rows,) + tail, generator=g) + 0.5).to(dtype)      # no zero rows among the real ones


def _bytes(t):
    width = int(np.prod(t.shape[1:])) * t.element_size()      # rows may be single elements, and there may be none
    return t.flatten().view(torch.uint8).reshape(t.shape[0], width).numpy()


@pytest.mark.parametrize("tail,dtype", [((96,), torch.bfloat16), ((1,), torch.bfloat16), ((1,), torch.float32),
                                        ((3,), torch.uint8), ((20,), torch.bfloat16), ((2, 24), torch.float32), ((), torch.float32)])
@pytest.mark.parametrize("lens,align", CASES)
def test_pad_and_unpad_match_the_oracle(gpu, lens, align, tail, dtype):
    from primus_amd.pytorch import kernels as K

    rows = sum(lens)
    x = _rand(rows, tail, dtype, rows + align)
    gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
    out, padded_lens = K.pad_groups_impl(x.to(gpu), gl, align)
    bound = o.padded_rows_bound(rows, len(lens), align)
    want, want_lens = o.pad_groups(_bytes(x), lens, align, bound)
    got = _bytes(out.cpu())
    assert got.shape == want.shape and np.array_equal(got, want)
    assert padded_lens.cpu().tolist() == want_lens.tolist() and int(padded_lens.sum()) == bound
    back = K.unpad_groups_impl(out, gl, align, rows + 2)          # two rows behind the counts: zeros
    assert torch.equal(back[:rows].cpu(), x) and not back[rows:].view(torch.uint8).any()


def test_many_groups_wide_rows_and_an_offset_pointer(gpu):
    from primus_amd.pytorch import kernels as K

    g = torch.Generator().manual_seed(3)
    lens = torch.randint(0, 70, (1024,), generator=g)
    lens[::5] = 0
    rows = int(lens.sum())
    base = (torch.rand((rows + 1, 520), generator=g) + 0.5).bfloat16().to(gpu)
    x = base[1:]                                                   # 1040-byte rows: the start is 16-byte aligned only
    gl = lens.to(gpu)
    out, padded_lens = K.pad_groups_impl(x, gl, 32)
    want, want_lens = o.pad_groups(x.cpu().view(torch.int16).numpy(), lens.tolist(), 32, out.shape[0])
    assert np.array_equal(out.cpu().view(torch.int16).numpy(), want)
    assert padded_lens.cpu().tolist() == want_lens.tolist()
    assert torch.equal(K.unpad_groups_impl(out, gl, 32, rows), x)


def test_full_size_round_trip(gpu):
    """65 536 routed tokens of width 7168 over 256 experts: pad, then unpad, returns the input; the padded
    buffer has every group at a multiple of 32 and nothing but zeros in between."""
    from primus_amd.pytorch import kernels as K

    g = torch.Generator(device=gpu).manual_seed(1)
    rows, groups = 65536, 256
    cuts = torch.sort(torch.randint(0, rows + 1, (groups - 1,), generator=g, device=gpu)).values
    edges = torch.cat([cuts.new_zeros(1), cuts, cuts.new_full((1,), rows)])
    gl = (edges[1:] - edges[:-1]).contiguous()
    x = torch.randn(rows, 7168, generator=g, device=gpu, dtype=torch.bfloat16)
    out, padded_lens = K.pad_groups_impl(x, gl, 32)
    assert out.shape[0] == (rows + groups * 31) // 32 * 32 and int(padded_lens.sum()) == out.shape[0]
    assert not (padded_lens % 32).any() and bool((padded_lens >= gl).all())
    assert torch.equal(K.unpad_groups_impl(out, gl, 32, rows), x)
    # the sum of every column survives (zero rows add nothing); checked in integers on the bit patterns' low byte
    assert int(out.view(torch.uint8)[:, ::2].sum(dtype=torch.int64)) == int(x.view(torch.uint8)[:, ::2].sum(dtype=torch.int64))
    live = torch.repeat_interleave(torch.arange(groups, device=gpu), padded_lens)
    start = torch.cumsum(padded_lens, 0) - padded_lens
    local = torch.arange(out.shape[0], device=gpu) - start[live]
    assert not out[local >= gl[live]].any()


def test_gradients_are_each_others_inverse(gpu):
    import primus_amd.pytorch as turbo

    lens = torch.tensor([5, 0, 33, 64], dtype=torch.int64, device=gpu)
    x = torch.randn(102, 64, device=gpu).bfloat16().requires_grad_()
    out, padded_lens = turbo.ops.pad_groups(x, lens, 32)
    assert not padded_lens.requires_grad
    dout = torch.randn_like(out)
    (dx,) = torch.autograd.grad(out, x, dout)
    want = torch.from_numpy(o.unpad_groups(dout.cpu().view(torch.int16).numpy(), lens.tolist(), 32)).view(torch.bfloat16)
    assert torch.equal(dx.cpu(), want)
    y = out.detach().requires_grad_()
    back = turbo.ops.unpad_groups(y, lens, 32, 102)
    assert torch.equal(back, x.detach())
    dback = torch.randn_like(back)
    (dy,) = torch.autograd.grad(back, y, dback)
    want, _ = o.pad_groups(dback.cpu().view(torch.int16).numpy(), lens.tolist(), 32, out.shape[0])
    assert torch.equal(dy.cpu().view(torch.int16), torch.from_numpy(want))


def test_arguments_are_checked(gpu):
    from primus_amd import _lib

    lib = _lib.load()
    EINVAL = -1
    x = torch.zeros(64, 16, device=gpu)
    gl = torch.tensor([64], dtype=torch.int64, device=gpu)
    out = torch.zeros(96, 16, device=gpu)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.mxl_padded_rows_bound(64, 1, 32) == 64 and lib.mxl_padded_rows_bound(65, 2, 32) == 96
    assert lib.mxl_padded_rows_bound(-1, 1, 32) == -1
    assert lib.mxl_pad_groups(x.data_ptr(), 64, 64, gl.data_ptr(), 1, 32, out.data_ptr(), 32, None, s) == EINVAL
    assert lib.mxl_pad_groups(x.data_ptr(), 64, 64, gl.data_ptr(), 1025, 32, out.data_ptr(), 1 << 20, None, s) == EINVAL
    assert lib.mxl_pad_groups(x.data_ptr(), 64, 64, None, 1, 32, out.data_ptr(), 64, None, s) == EINVAL
    assert lib.mxl_pad_groups(x.data_ptr(), 64, 64, gl.data_ptr(), 1, 0, out.data_ptr(), 64, None, s) == EINVAL
    assert lib.mxl_unpad_groups(out.data_ptr(), 96, 0, gl.data_ptr(), 1, 32, x.data_ptr(), 64, s) == EINVAL


@pytest.mark.parametrize("fused_act", [False, True])
def test_expert_mlp_pads_on_the_device_like_on_the_host(gpu, fused_act):
    """The explicit-padding route of the expert MLP with the counts on the device (no host read-back) gives the
    output and gradients of the same route with the counts on the host, which pads as the reference does."""
    from types import SimpleNamespace

    from primus_amd.megatron import runtime
    from primus_amd.megatron.extensions import primus_turbo as pt
    from primus_amd.megatron.transformer.experts import PrimusGroupedMLP
    from primus_amd.pytorch.core import Format, ScaleDtype, ScalingGranularity

    pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
    runtime.bind()
    runtime.set_num_microbatches(1)
    runtime.set_args(enable_primus_turbo=True, use_turbo_gemm=True, use_turbo_grouped_gemm=True,
                     turbo_grouped_gemm_without_padding=False, use_turbo_fused_act_with_probs=fused_act)
    try:
        torch.manual_seed(17)
        cfg = SimpleNamespace(params_dtype=torch.bfloat16, use_cpu_initialization=False, perform_initialization=True,
                              tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                              layernorm_epsilon=1e-5, hidden_size=128, ffn_hidden_size=256, moe_ffn_hidden_size=256,
                              gated_linear_unit=True, fp8="e4m3", fp8_recipe="mxfp8", fp4=None, add_bias_linear=False)
        mlp = PrimusGroupedMLP(4, cfg)
        assert mlp._use_explicit_quantization_padding()
        qc = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E4M3, block_size=32,
                                       scale_dtype=ScaleDtype.E8M0)
        lens = [5, 0, 33, 64]
        x = torch.randn(sum(lens), 128, device=gpu).bfloat16()
        probs = torch.rand(sum(lens), device=gpu)
        dy = torch.randn(sum(lens), 128, device=gpu).bfloat16()
        res = []
        for tpe in (torch.tensor(lens), torch.tensor(lens, device=gpu)):
            mlp.zero_grad(set_to_none=True)
            for lin in (mlp.linear_fc1, mlp.linear_fc2):
                lin.set_is_first_microbatch()
            xi, pi = x.clone().requires_grad_(), probs.clone().requires_grad_()
            with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=qc):
                out, _ = mlp(xi, tpe, pi)
            out.backward(dy)
            res.append((out.detach(), xi.grad, pi.grad, mlp.linear_fc1.weights.grad.clone(), mlp.linear_fc2.weights.grad.clone()))
        for name, a, b in zip(("y", "dx", "dprobs", "dw1", "dw2"), *res):
            assert a.shape == b.shape and torch.equal(a, b), name
        assert res[0][0].shape == (sum(lens), 128)
    finally:
        pt.PrimusTurboLowPrecisionGlobalStateManager.reset()
        runtime.set_args()
