"""CPU tests of the Megatron-side host logic (no GPU, no kernels).

They follow the reference's own unit tests for this layer where it has them:
the padding truth table (tests/unit_tests/backends/megatron/test_grouped_mlp.py:24-53),
argument validation (test_rocm_arg_validation.py:30-66), the gradient
stochastic-rounding option (test_fp4_utils_mxfp4.py:40-78), the local-shard
tiling (test_weight_deosc.py:82-127) and the dual-quantise output shapes
(primus_turbo_mxfp4_local.py:164-207).
"""

from types import SimpleNamespace

import pytest
import torch

from primus_amd.megatron import fp4_utils, fp8_utils, runtime
from primus_amd.megatron.enums import Fp4Recipe, Fp8Recipe
from primus_amd.megatron.extensions import primus_turbo as pt
from primus_amd.megatron.extensions import primus_turbo_mxfp4_local as mxfp4_local
from primus_amd.megatron.extensions.transformer_engine_spec_provider import PrimusTurboSpecProvider
from primus_amd.megatron.optimizer import weight_deosc
from primus_amd.megatron.patches import (
    PatchContext,
    apply_patches,
    is_primus_turbo_can_patch,
    registered_patches,
    validate_args_on_rocm,
    validate_turbo_grouped_gemm_without_padding,
)
from primus_amd.megatron.transformer.experts import PrimusGroupedMLP
from primus_amd.pytorch.core.low_precision import (
    Float4QuantConfig,
    Float8QuantConfig,
    Format,
    ScaleDtype,
    ScalingGranularity,
)
from primus_amd.pytorch.core.quantized_tensor import QuantizedTensor, QuantizedTensorPair

Manager = pt.PrimusTurboLowPrecisionGlobalStateManager


@pytest.fixture(autouse=True)
def _clean_state(monkeypatch):
    # the support probes need a GPU; the state logic under test does not
    for name in ("check_fp8_support", "check_mxfp8_support", "check_mxfp4_support"):
        monkeypatch.setattr(pt, name, lambda: (True, ""))
    Manager.reset()
    runtime.bind()
    runtime.set_args()
    runtime.set_num_microbatches(1)
    yield
    Manager.reset()
    runtime.set_args()
    runtime.set_num_microbatches(1)


def _mxfp8():
    return pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E4M3, block_size=32,
                                     scale_dtype=ScaleDtype.E8M0)


def _mxfp4(**kw):
    return pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E2M1_X2,
                                     block_size=32, scale_dtype=ScaleDtype.E8M0, **kw)


# --------------------------------------------------------------------------- a1
def test_quant_config_predicates():
    default = pt.PrimusTurboQuantConfig()
    assert default.is_fp8() and not default.is_fp4()
    assert default.current_scaling() and not default.mxfp8_scaling() and not default.block_scaling()
    assert isinstance(default.data(), Float8QuantConfig)

    c8 = _mxfp8()
    assert c8.mxfp8_scaling() and not c8.current_scaling() and not c8.mxfp4_scaling()
    assert c8.data().block_size == 32 and c8.data().scale_dtype == ScaleDtype.E8M0

    c4 = _mxfp4()
    assert c4.is_fp4() and c4.mxfp4_scaling() and not c4.mxfp8_scaling()
    assert isinstance(c4.data(), Float4QuantConfig)

    blk = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    assert blk.block_scaling() and not blk.mxfp8_scaling()
    # hybrid is not the MXFP8 recipe (E4M3 only)
    hyb = pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.HYBRID,
                                    scale_dtype=ScaleDtype.E8M0)
    assert not hyb.mxfp8_scaling()


def test_mx_config_rejects_wrong_block_or_scale_dtype():
    with pytest.raises(ValueError):
        pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, block_size=64, scale_dtype=ScaleDtype.E8M0)
    with pytest.raises(ValueError):
        pt.PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.FP32)


# --------------------------------------------------------------------------- a2
def test_autocast_sets_and_restores_the_nine_tuple():
    before = Manager.get_fp8_autocast_state()
    assert len(before) == 9
    cfg = _mxfp8()
    with pt.primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=cfg):
        assert Manager.is_turbo_fp8_enabled() and not Manager.is_turbo_fp4_enabled()
        assert Manager.get_turbo_quant_config() is cfg
        inner = _mxfp4()
        with pt.primus_turbo_fp4_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=inner):
            assert Manager.is_turbo_fp4_enabled() and not Manager.is_turbo_fp8_enabled()
            assert Manager.get_turbo_quant_config() is inner
        assert Manager.is_turbo_fp8_enabled() and Manager.get_turbo_quant_config() is cfg
    assert Manager.get_fp8_autocast_state() == before
    assert Manager.FP8_AUTOCAST_DEPTH == 0


def test_autocast_restores_on_exception_and_defaults_to_tensorwise():
    with pytest.raises(RuntimeError):
        with pt.primus_turbo_fp8_autocast(enabled_turbo=True):
            assert Manager.get_turbo_quant_config().current_scaling()
            raise RuntimeError("boom")
    assert not Manager.is_turbo_fp8_enabled() and Manager.get_turbo_quant_config() is None


def test_autocast_asserts_when_hardware_support_is_missing(monkeypatch):
    monkeypatch.setattr(pt, "check_mxfp8_support", lambda: (False, "no gfx950"))
    with pytest.raises(AssertionError, match="no gfx950"):
        with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
            pass
    # not enabled: the probes are not consulted
    with pt.primus_turbo_fp8_autocast(enabled_turbo=False, turbo_quant_config=_mxfp8()):
        assert not Manager.is_turbo_fp8_enabled()


# --------------------------------------------------------------------------- a3
def _model_config(**kw):
    values = dict(fp8="e4m3", fp8_recipe=Fp8Recipe.mxfp8, fp8_param=False, fp4=None, fp4_recipe=None,
                  first_last_layers_bf16=False, num_layers_at_start_in_bf16=0, num_layers_at_end_in_bf16=0,
                  num_layers=8)
    values.update(kw)
    return SimpleNamespace(**values)


@pytest.mark.parametrize("recipe,pred", [("tensorwise", "current_scaling"), ("blockwise", "block_scaling"),
                                          ("mxfp8", "mxfp8_scaling")])
def test_fp8_recipe_to_quant_config(recipe, pred):
    cfg, why = fp8_utils.get_fp8_quant_config(_model_config(fp8_recipe=recipe))
    assert why == "" and getattr(cfg, pred)()
    if recipe == "mxfp8":
        assert cfg.data().block_size == 32 and cfg.data().scale_dtype == ScaleDtype.E8M0
    if recipe == "blockwise":
        assert cfg.data().block_size == 128


def test_fp8_delayed_recipe_has_no_turbo_config_and_bad_format_raises():
    cfg, why = fp8_utils.get_fp8_quant_config(_model_config(fp8_recipe=Fp8Recipe.delayed))
    assert cfg is None and "delayed" in why
    with pytest.raises(ValueError):
        fp8_utils.get_fp8_quant_config(_model_config(fp8="e5m2"))


def test_fp8_context_per_layer_bf16_bypass():
    cfg = _model_config(first_last_layers_bf16=True, num_layers_at_start_in_bf16=1, num_layers_at_end_in_bf16=2)
    enabled = []
    for layer in range(cfg.num_layers):
        with fp8_utils.get_fp8_context(cfg, layer):
            enabled.append(Manager.is_turbo_fp8_enabled())
    assert enabled == [False, True, True, True, True, True, False, False]
    with fp8_utils.get_fp8_context(cfg, -1):  # "all layers" context
        assert Manager.is_turbo_fp8_enabled() and Manager.get_turbo_quant_config().mxfp8_scaling()
    with fp8_utils.get_fp8_context(_model_config(fp8=None), 3):
        assert not Manager.is_turbo_fp8_enabled()


def test_fp4_context_and_gradient_sr_resolution():
    runtime.set_args(enable_primus_turbo=True)
    cfg = _model_config(fp8=None, fp8_recipe=None, fp4="e2m1", fp4_recipe=Fp4Recipe.mxfp4,
                        first_last_layers_bf16=True, num_layers_at_start_in_bf16=2, num_layers_at_end_in_bf16=0)
    seen = []
    for layer in range(4):
        with fp4_utils.get_fp4_context(cfg, layer):
            seen.append(Manager.is_turbo_fp4_enabled())
    assert seen == [False, False, True, True]
    with fp4_utils.get_fp4_context(cfg, 5):
        assert Manager.get_turbo_quant_config().mxfp4_scaling()
    qc, why = fp4_utils.get_fp4_quant_config(_model_config(fp4_recipe=Fp4Recipe.nvfp4))
    assert qc is None and "MXFP4" in why
    # local transformer implementation quantises inside its own modules
    cfg.transformer_impl = "local"
    with fp4_utils.get_fp4_context(cfg, 3):
        assert not Manager.is_turbo_fp4_enabled()


def test_gradient_sr_explicit_config_wins_then_global_args_then_off():
    def unexpected():
        raise AssertionError("global args must not be read for an explicit config value")

    runtime.bind(get_args=unexpected)
    assert fp4_utils._mxfp4_gradient_sr_enabled(SimpleNamespace(mxfp4_gradient_stochastic_rounding=True))
    assert not fp4_utils._mxfp4_gradient_sr_enabled(SimpleNamespace(mxfp4_gradient_stochastic_rounding=False))
    runtime.bind(get_args=lambda: SimpleNamespace(mxfp4_gradient_stochastic_rounding=True))
    assert fp4_utils._mxfp4_gradient_sr_enabled(SimpleNamespace())

    def unavailable():
        raise RuntimeError("global args are not initialized")

    runtime.bind(get_args=unavailable)
    assert not fp4_utils._mxfp4_gradient_sr_enabled(SimpleNamespace())
    assert not fp4_utils._primus_turbo_enabled()


def test_per_module_recipe_override():
    R = pt.QuantizationRecipe
    # not overriding the surrounding non-quantised autocast -> nothing happens
    with pt._get_fp8_autocast_for_quant_recipe(R(fp8_quantization_recipe=Fp8Recipe.mxfp8)):
        assert not Manager.is_turbo_fp8_enabled()
    with pt._get_fp8_autocast_for_quant_recipe(R(fp8_quantization_recipe=Fp8Recipe.mxfp8,
                                                 override_nonquantized_autocast=True)):
        assert Manager.get_turbo_quant_config().mxfp8_scaling()
    with pt._get_fp8_autocast_for_quant_recipe(R(fp4_quantization_recipe=Fp4Recipe.mxfp4,
                                                 override_nonquantized_autocast=True)):
        assert Manager.is_turbo_fp4_enabled()
    # inside a quantised autocast a recipe-less module is forced to bf16
    with pt.primus_turbo_fp8_autocast(enabled=True, enabled_turbo=True, turbo_quant_config=_mxfp8()):
        with pt._get_fp8_autocast_for_quant_recipe(R()):
            assert not Manager.is_turbo_fp8_enabled()
        assert Manager.is_turbo_fp8_enabled()
    with pytest.raises(AssertionError):
        pt._get_fp8_autocast_for_quant_recipe(R(fp4_quantization_recipe=Fp4Recipe.nvfp4,
                                                override_nonquantized_autocast=True))
    with pytest.raises(ValueError):
        pt._get_fp8_autocast_for_quant_recipe(R(fp8_quantization_recipe=Fp8Recipe.mxfp8, fp8_format="e5m2",
                                                override_nonquantized_autocast=True))
    params = pt.QuantizationParams(training_recipe=R(fp8_quantization_recipe=Fp8Recipe.tensorwise,
                                                     override_nonquantized_autocast=True),
                                   evaluation_recipe=R(override_nonquantized_autocast=True))
    with pt._get_fp8_autocast_for_quant_params(params, training=True):
        assert Manager.get_turbo_quant_config().current_scaling()
    with pt._get_fp8_autocast_for_quant_params(params, training=False):
        assert not Manager.is_turbo_fp8_enabled()


# --------------------------------------------------------------------------- a5
def _fake_quantized(weight):
    n, k = weight.shape[-2:]
    lead = tuple(weight.shape[:-2])
    row = QuantizedTensor(torch.zeros(lead + (n, k), dtype=torch.uint8), torch.zeros(lead + (n, k // 32), dtype=torch.uint8),
                          logical_shape=weight.shape, axis=-1, use_2d_block=True)
    col = QuantizedTensor(torch.zeros(lead + (k, n), dtype=torch.uint8), torch.zeros(lead + (k, n // 32), dtype=torch.uint8),
                          logical_shape=lead + (k, n), axis=-2, use_2d_block=True)
    return row, col


class _StubGemm(torch.autograd.Function):
    """Stands in for the quantised GEMM: returns a known weight gradient for
    the row-wise copy and nothing for the transposed one."""

    @staticmethod
    def forward(ctx, x, q, q_t, wgrad):
        ctx.save_for_backward(wgrad)
        return x * 2.0

    @staticmethod
    def backward(ctx, gy):
        (wgrad,) = ctx.saved_tensors
        return gy * 2.0, wgrad, None, None


def test_weight_grad_bridge_accumulates_into_main_grad_once():
    weight = torch.nn.Parameter(torch.zeros(64, 32, dtype=torch.bfloat16))
    weight.main_grad = torch.ones(64, 32, dtype=torch.float32)
    weight.grad_added_to_main_grad = False
    row, col = _fake_quantized(weight)
    wgrad = torch.full((64, 32), 3.0, dtype=torch.bfloat16)
    x = torch.randn(4, 32, dtype=torch.bfloat16, requires_grad=True)

    x2, pair = pt._bridge_weight_grad(x, weight, QuantizedTensorPair(data=row, data_t=col))
    assert isinstance(pair.data, QuantizedTensor) and pair.data.axis == -1 and pair.data_t.axis == -2
    assert pair.data.requires_grad  # the GEMM must produce a gradient for it
    y = _StubGemm.apply(x2, pair.data, pair.data_t, wgrad)
    y.sum().backward()

    assert torch.equal(weight.main_grad, torch.full((64, 32), 4.0))
    assert weight.grad_added_to_main_grad is True
    assert weight.grad is not None and weight.grad.shape == weight.shape  # dummy wgrad fired the hooks
    assert torch.equal(x.grad, torch.full_like(x, 2.0))

    # a second microbatch with the flag still set must not add again
    x3, pair = pt._bridge_weight_grad(x.detach().requires_grad_(), weight, QuantizedTensorPair(data=row, data_t=col))
    _StubGemm.apply(x3, pair.data, pair.data_t, wgrad).sum().backward()
    assert torch.equal(weight.main_grad, torch.full((64, 32), 4.0))


def test_bridge_requires_main_grad():
    weight = torch.nn.Parameter(torch.zeros(32, 32, dtype=torch.bfloat16))
    row, col = _fake_quantized(weight)
    x = torch.randn(2, 32, dtype=torch.bfloat16, requires_grad=True)
    x2, pair = pt._bridge_weight_grad(x, weight, QuantizedTensorPair(data=row, data_t=col))
    with pytest.raises(AssertionError, match="main_grad"):
        _StubGemm.apply(x2, pair.data, pair.data_t, torch.zeros(32, 32, dtype=torch.bfloat16)).sum().backward()
    with pytest.raises(AssertionError):
        pt._bridge_weight_grad(x, weight, (row, col))


def test_dummy_wgrad_is_cached_per_shape_and_dtype():
    a = pt._get_dummy_wgrad([4, 8], torch.bfloat16, device="cpu", zero=True)
    b = pt._get_dummy_wgrad((4, 8), torch.bfloat16, device="cpu")
    c = pt._get_dummy_wgrad((2, 4, 8), torch.bfloat16, device="cpu")
    assert a.data_ptr() == b.data_ptr() and a.data_ptr() != c.data_ptr()
    assert not a.requires_grad and torch.count_nonzero(a) == 0


def test_fused_wgrad_accumulation_is_off_for_mx_and_fp4():
    cfg = SimpleNamespace(gradient_accumulation_fusion=True)
    w = torch.nn.Parameter(torch.zeros(32, 32, dtype=torch.bfloat16))
    w.main_grad, w.grad_added_to_main_grad = torch.zeros(32, 32), False
    assert pt._fuse_wgrad_accum_pattern(SimpleNamespace(gradient_accumulation_fusion=False), w) is None
    assert pt._fuse_wgrad_accum_pattern(cfg, w) == "megatron"  # bf16
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        assert pt._fuse_wgrad_accum_pattern(cfg, w) is None
    with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
        assert pt._fuse_wgrad_accum_pattern(cfg, w) is None
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=pt.PrimusTurboQuantConfig()):
        assert pt._fuse_wgrad_accum_pattern(cfg, w) == "megatron"  # tensorwise has the epilogue
    # this package's wgrad kernel accumulates for the MX recipes too: opt-in switch
    runtime.set_args(turbo_fuse_wgrad_accum_mx=True)
    try:
        with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
            assert pt._fuse_wgrad_accum_pattern(cfg, w) == "megatron"
        with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
            assert pt._fuse_wgrad_accum_pattern(cfg, w) == "megatron"
    finally:
        runtime.set_args()
    bare = torch.nn.Parameter(torch.zeros(32, 32, dtype=torch.bfloat16))
    with pytest.raises(AssertionError):
        pt._fuse_wgrad_accum_pattern(cfg, bare)
    assert pt._fuse_wgrad_accum_pattern(cfg, torch.nn.Parameter(torch.zeros(2, 2))) is None  # fp32 weight


# --------------------------------------------------------------------------- a6 / a7
def _layer_config(**kw):
    values = dict(params_dtype=torch.bfloat16, use_cpu_initialization=True, perform_initialization=True,
                  tensor_model_parallel_size=1, gradient_accumulation_fusion=False, normalization="RMSNorm",
                  layernorm_epsilon=1e-5)
    values.update(kw)
    return SimpleNamespace(**values)


class _Recorder:
    """Replaces the operator namespace: records which op ran with what."""

    def __init__(self):
        self.calls = []

    def _dense(self, name):
        def op(a, b, trans_a=False, trans_b=True, out_dtype=None, config=None, fuse_bgrad_accum_pattern=None):
            self.calls.append((name, type(b).__name__, config, fuse_bgrad_accum_pattern))
            n = b.data.shape[0] if isinstance(b, QuantizedTensorPair) else b.shape[0]
            return a.new_zeros(a.shape[0], n) + a.sum() * 0
        return op

    def _grouped(self, name):
        def op(a, b, group_lens, trans_b=True, config=None, fuse_bgrad_accum_pattern=None):
            self.calls.append((name, type(b).__name__, config, group_lens))
            n = b.data.shape[1] if isinstance(b, QuantizedTensorPair) else b.shape[1]
            return a.new_zeros(a.shape[0], n) + a.sum() * 0
        return op

    def __getattr__(self, name):
        if name.startswith("grouped_gemm"):
            return self._grouped(name)
        if name.startswith("gemm"):
            return self._dense(name)
        raise AttributeError(name)


@pytest.fixture
def recorder(monkeypatch):
    rec = _Recorder()
    monkeypatch.setattr(pt, "ops", rec)
    monkeypatch.setattr(pt, "create_quantized_weight",
                        lambda w, dt, qc, need_weight_transpose_cache=True:
                        (lambda r, c: (r, c if need_weight_transpose_cache else None))(*_fake_quantized(w)))
    return rec


def test_linear_selects_op_by_autocast_state(recorder):
    lin = pt.PrimusTurboLinear(64, 96, parallel_mode=None, config=_layer_config(), bias=True, skip_bias_add=False)
    x = torch.randn(5, 2, 64, dtype=torch.bfloat16)
    out, bias = lin(x)
    assert out.shape == (5, 2, 96) and bias is None
    assert recorder.calls[-1][0] == "gemm"
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        lin(x)
    name, btype, cfg, _ = recorder.calls[-1]
    assert name == "gemm_fp8" and btype == "Parameter" and isinstance(cfg, Float8QuantConfig)
    with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
        lin.set_is_first_microbatch()
        lin(x)
    name, btype, cfg, _ = recorder.calls[-1]
    assert name == "gemm_fp4" and btype == "Parameter" and isinstance(cfg, Float4QuantConfig)
    # one microbatch per step + FP4: the empty buffer marks the weight as FP4-quantised
    assert lin.quantized_weight_buffer.numel() == 0 and lin.quantized_weight_buffer.dtype == torch.uint8


def test_linear_caches_quantized_weight_across_microbatches(recorder, monkeypatch):
    made = []
    orig = pt.create_quantized_weight

    def counting(w, dt, qc, need_weight_transpose_cache=True):
        made.append((dt, need_weight_transpose_cache))
        return orig(w, dt, qc, need_weight_transpose_cache=need_weight_transpose_cache)

    monkeypatch.setattr(pt, "create_quantized_weight", counting)
    runtime.set_num_microbatches(4)
    lin = pt.PrimusTurboColumnParallelLinear(64, 64, config=_layer_config(), bias=False)
    lin.weight.main_grad = torch.zeros(64, 64)
    lin.weight.grad_added_to_main_grad = False
    x = torch.randn(3, 1, 64, dtype=torch.bfloat16)
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        for _ in range(3):
            lin(x)
    assert len(made) == 1 and made[0] == (torch.float8_e4m3fn, True)
    assert all(c[0] == "gemm_fp8" and c[1] == "QuantizedTensorPair" for c in recorder.calls)
    lin.set_is_first_microbatch()  # next optimizer step
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        lin(x)
    assert len(made) == 2
    # tensorwise never keeps a transposed copy (it can transpose the row-wise one)
    lin.set_is_first_microbatch()
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=pt.PrimusTurboQuantConfig()):
        lin(x)
    assert made[-1] == (torch.float8_e4m3fn, False)


def test_linear_variants_and_constraints(recorder):
    with pytest.raises(AssertionError, match="tensor parallel size = 1"):
        pt.PrimusTurboRowParallelLinear(32, 32, config=_layer_config(tensor_model_parallel_size=2))
    with pytest.raises(ValueError):
        pt.PrimusTurboColumnParallelLinear(32, 32, config=_layer_config(), gather_output=True)
    with pytest.raises(ValueError):
        pt.PrimusTurboRowParallelLinear(32, 32, config=_layer_config(), input_is_parallel=False)
    ln = pt.PrimusTurboLayerNormColumnParallelLinear(32, 64, config=_layer_config(), bias=False)
    assert ln.layer_norm_bias is None
    out, _ = ln(torch.randn(4, 2, 32, dtype=torch.bfloat16))
    assert out.shape == (4, 2, 64)
    ln2 = pt.PrimusTurboLayerNormColumnParallelLinear(32, 64, config=_layer_config(normalization="LayerNorm"))
    assert ln2.layer_norm_bias is not None
    assert "in_features=32" in repr(ln2) and "TP=1" in repr(ln2)


def test_norm_in_front_of_the_gemm_is_what_the_gemm_sees(monkeypatch):
    seen = {}

    def fake_gemm(a, b, **kw):
        seen["a"] = a.clone()
        return a.new_zeros(a.shape[0], b.shape[0])

    monkeypatch.setattr(pt, "ops", SimpleNamespace(gemm=fake_gemm, grouped_gemm=None))
    ln = pt.PrimusTurboLayerNormColumnParallelLinear(32, 32, config=_layer_config(params_dtype=torch.float32), bias=False)
    with torch.no_grad():
        ln.layer_norm_weight.copy_(torch.linspace(0.5, 1.5, 32))
    x = torch.randn(3, 2, 32)
    ln(x)
    want = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * ln.layer_norm_weight
    torch.testing.assert_close(seen["a"], want.view(-1, 32), rtol=1e-5, atol=1e-6)


def test_grouped_linear_consolidates_weights_and_keeps_splits_on_device(recorder):
    gl = pt.PrimusTurboColumnParallelGroupedLinear(4, 32, 64, config=_layer_config())
    assert tuple(gl.weights.shape) == (4, 64, 32) and gl.weights.requires_grad
    assert [n for n, _ in gl.named_parameters()] == ["weights"]
    x = torch.randn(10, 32, dtype=torch.bfloat16)
    splits = torch.tensor([3, 0, 5, 2])
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        out, bias = gl(x, splits)
    assert out.shape == (10, 64) and bias is None
    name, btype, cfg, lens = recorder.calls[-1]
    assert name == "grouped_gemm_fp8" and btype == "Parameter" and torch.equal(lens, splits)
    with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
        gl(x, splits)
    assert recorder.calls[-1][0] == "grouped_gemm_fp4"
    gl(x, splits)
    assert recorder.calls[-1][0] == "grouped_gemm"
    # per-expert names exist in checkpoints and alias the consolidated storage
    sd = gl.state_dict()
    assert {"weights", "weight0", "weight3"} <= set(sd)
    assert sd["weight2"].data_ptr() == gl.weights[2].data_ptr()
    assert not gl.weight0.requires_grad


def test_grouped_linear_cached_pair_with_several_microbatches(recorder):
    runtime.set_num_microbatches(2)
    gl = pt.PrimusTurboRowParallelGroupedLinear(2, 32, 32, config=_layer_config())
    gl.weights.main_grad = torch.zeros(2, 32, 32)
    gl.weights.grad_added_to_main_grad = False
    x = torch.randn(6, 32, dtype=torch.bfloat16)
    with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
        gl(x, torch.tensor([4, 2]))
        gl(x, torch.tensor([1, 5]))
    assert [c[:2] for c in recorder.calls] == [("grouped_gemm_fp4", "QuantizedTensorPair")] * 2
    assert gl.quantized_weight_buffer.axis == -1 and gl.quantized_weight_t_buffer.axis == -2


# --------------------------------------------------------------------------- a8
def _grouped_mlp_state(**overrides):
    values = {
        "config": SimpleNamespace(fp8="e4m3", fp4=False),
        "moe_router_padding_for_quantization": False,
        "turbo_grouped_gemm_without_padding": True,
    }
    values.update(overrides)
    return SimpleNamespace(**values)


@pytest.mark.parametrize("config", [SimpleNamespace(fp8="e4m3", fp4=False), SimpleNamespace(fp8=None, fp4="e2m1")])
def test_without_padding_option_skips_explicit_padding(config):
    assert not PrimusGroupedMLP._use_explicit_quantization_padding(_grouped_mlp_state(config=config))


def test_disabled_without_padding_option_keeps_explicit_padding():
    state = _grouped_mlp_state(turbo_grouped_gemm_without_padding=False)
    assert PrimusGroupedMLP._use_explicit_quantization_padding(state)


@pytest.mark.parametrize("overrides", [{"config": SimpleNamespace(fp8=None, fp4=False)},
                                       {"moe_router_padding_for_quantization": True}])
def test_explicit_padding_is_not_duplicated(overrides):
    assert not PrimusGroupedMLP._use_explicit_quantization_padding(_grouped_mlp_state(**overrides))


def _mlp_config(**kw):
    return _layer_config(hidden_size=32, ffn_hidden_size=64, moe_ffn_hidden_size=64, gated_linear_unit=True,
                         fp8="e4m3", fp8_recipe="mxfp8", fp4=None, add_bias_linear=False, **kw)


def test_grouped_mlp_matches_a_per_expert_loop_in_bf16():
    runtime.set_args(use_turbo_grouped_gemm=True, turbo_grouped_gemm_without_padding=True)
    mlp = PrimusGroupedMLP(3, _mlp_config(params_dtype=torch.float32))
    lens = [5, 0, 7]
    x = torch.randn(sum(lens), 32)
    probs = torch.rand(sum(lens))
    out, bias = mlp(x, torch.tensor(lens), probs)
    assert bias is None and out.shape == (12, 32)
    want, r = [], 0
    for g, n in enumerate(lens):
        h = x[r:r + n] @ mlp.linear_fc1.weights[g].T
        a, b = h.chunk(2, dim=-1)
        h = torch.nn.functional.silu(a) * b * probs[r:r + n, None]
        want.append(h @ mlp.linear_fc2.weights[g].T)
        r += n
    torch.testing.assert_close(out, torch.cat(want), rtol=1e-4, atol=1e-5)


def test_grouped_mlp_explicit_padding_pads_to_the_recipe_multiple_and_unpads():
    runtime.set_args(use_turbo_grouped_gemm=True, turbo_grouped_gemm_without_padding=False)
    mlp = PrimusGroupedMLP(3, _mlp_config(params_dtype=torch.float32))
    seen = []
    fc1 = mlp.linear_fc1.forward

    def spy(x, splits):
        seen.append((x.shape[0], splits.tolist()))
        return fc1(x, splits)

    mlp.linear_fc1.forward = spy
    lens = [5, 0, 33]
    x = torch.randn(sum(lens), 32)
    probs = torch.rand(sum(lens))
    out, _ = mlp(x, torch.tensor(lens), probs)
    assert seen == [(32 + 0 + 64, [32, 0, 64])]  # MXFP8: multiples of 32
    assert out.shape == (38, 32)
    runtime.set_args(use_turbo_grouped_gemm=True, turbo_grouped_gemm_without_padding=True)
    ref = PrimusGroupedMLP(3, _mlp_config(params_dtype=torch.float32))
    ref.load_state_dict(mlp.state_dict())
    want, _ = ref(x, torch.tensor(lens), probs)
    torch.testing.assert_close(out, want, rtol=1e-4, atol=1e-5)
    # the other FP8 recipes pad to 16
    mlp.config.fp8_recipe = "tensorwise"
    _, padded = mlp.quantization_padding(x, lens)
    assert padded == [16, 0, 48]


# --------------------------------------------------------------------------- a9 / a10 / a11
def test_spec_provider_selects_turbo_classes_by_switch():
    runtime.set_args(use_turbo_gemm=True, use_turbo_grouped_gemm=True)
    sp = PrimusTurboSpecProvider()
    assert sp.linear() is pt.PrimusTurboLinear
    assert sp.column_parallel_linear() is pt.PrimusTurboColumnParallelLinear
    assert sp.row_parallel_linear() is pt.PrimusTurboRowParallelLinear
    assert sp.column_parallel_layer_norm_linear() is pt.PrimusTurboLayerNormColumnParallelLinear
    assert sp.fuse_layernorm_and_linear()
    cls, sub = sp.grouped_mlp_modules(moe_use_grouped_gemm=True)
    assert cls is PrimusGroupedMLP
    assert sub.linear_fc1 is pt.PrimusTurboColumnParallelGroupedLinear
    assert sub.linear_fc2 is pt.PrimusTurboRowParallelGroupedLinear
    with pytest.raises(AssertionError, match="not compatible"):
        sp.grouped_mlp_modules(True, moe_use_legacy_grouped_gemm=True)


def test_spec_provider_delegates_when_switches_are_off():
    runtime.set_args(use_turbo_gemm=False, use_turbo_grouped_gemm=False)
    other = SimpleNamespace(linear=lambda: "TELinear", column_parallel_linear=lambda: "TECol",
                            row_parallel_linear=lambda: "TERow", column_parallel_layer_norm_linear=lambda: "TELN",
                            grouped_mlp_modules=lambda a, b: ("TEGroupedMLP", (a, b)))
    sp = PrimusTurboSpecProvider(fallback=other)
    assert (sp.linear(), sp.column_parallel_linear(), sp.row_parallel_linear(),
            sp.column_parallel_layer_norm_linear()) == ("TELinear", "TECol", "TERow", "TELN")
    assert sp.grouped_mlp_modules(True) == ("TEGroupedMLP", (True, False))
    with pytest.raises(RuntimeError):
        PrimusTurboSpecProvider().linear()


def test_patch_gating_and_targets():
    assert registered_patches()[0] == "megatron.turbo.te_spec_provider"  # priority 41 runs first
    assert not is_primus_turbo_can_patch(PatchContext(args=SimpleNamespace(enable_primus_turbo=False)))
    ctx = PatchContext(args=SimpleNamespace(enable_primus_turbo=True))
    assert is_primus_turbo_can_patch(ctx)
    assert not is_primus_turbo_can_patch(ctx, package="no_such_package_here") and "not found" in ctx.log[-1]

    paths = ["megatron.core.transformer.transformer_block", "megatron.core.ssm.mamba_block",
             "megatron.core.transformer.multi_token_prediction", "megatron.core.fp8_utils", "megatron.core.fp4_utils",
             "megatron.core.enums", "megatron.core.extensions.transformer_engine_spec_provider",
             "megatron.core.models.gpt.gpt_layer_specs", "megatron.core.models.gpt.moe_module_specs"]
    targets = {p: SimpleNamespace() for p in paths}
    apply_patches(SimpleNamespace(enable_primus_turbo=True, fp8="e4m3", fp4=None), targets)
    assert targets["megatron.core.fp8_utils"].get_fp8_context is fp8_utils.get_fp8_context
    assert targets["megatron.core.ssm.mamba_block"].get_fp8_context is fp8_utils.get_fp8_context
    assert targets["megatron.core.models.gpt.moe_module_specs"].TESpecProvider is PrimusTurboSpecProvider
    assert not hasattr(targets["megatron.core.fp4_utils"], "get_fp4_context")

    targets = {p: SimpleNamespace() for p in paths}
    apply_patches(SimpleNamespace(enable_primus_turbo=False, fp8=None, fp4="e2m1"), targets)
    assert targets["megatron.core.fp4_utils"].get_fp4_context is fp4_utils.get_fp4_context
    assert targets["megatron.core.enums"].Fp4Recipe is Fp4Recipe
    assert not hasattr(targets["megatron.core.fp8_utils"], "get_fp8_context")
    assert not hasattr(targets["megatron.core.models.gpt.gpt_layer_specs"], "TESpecProvider")

    targets = {p: SimpleNamespace() for p in paths}
    apply_patches(SimpleNamespace(enable_primus_turbo=True, fp8="e4m3", disable_fp8_context_patches=True), targets)
    assert not hasattr(targets["megatron.core.fp8_utils"], "get_fp8_context")


def _no_padding_args(**overrides):
    values = {"turbo_grouped_gemm_without_padding": True, "enable_primus_turbo": True, "use_turbo_grouped_gemm": True,
              "fp8": "e4m3", "fp8_recipe": "tensorwise", "fp4": False, "moe_router_padding_for_quantization": False}
    values.update(overrides)
    return SimpleNamespace(**values)


@pytest.mark.parametrize("overrides", [{}, {"fp8_recipe": "blockwise"}, {"fp8_recipe": "mxfp8"},
                                       {"fp8": None, "fp8_recipe": None, "fp4": "e2m1", "fp4_recipe": "mxfp4"},
                                       {"fp8": None, "fp8_recipe": None, "fp4": False}])
def test_without_padding_accepts_every_precision_mode(overrides):
    validate_turbo_grouped_gemm_without_padding(_no_padding_args(**overrides))
    validate_turbo_grouped_gemm_without_padding(SimpleNamespace())  # option absent: no-op


@pytest.mark.parametrize(("overrides", "message"), [
    ({"enable_primus_turbo": False}, "requires enable_primus_turbo"),
    ({"use_turbo_grouped_gemm": False}, "requires enable_primus_turbo"),
    ({"moe_router_padding_for_quantization": True}, "requires moe_router_padding_for_quantization=False"),
])
def test_without_padding_rejects_unsupported_config(overrides, message):
    with pytest.raises(ValueError, match=message):
        validate_turbo_grouped_gemm_without_padding(_no_padding_args(**overrides))


def test_validate_args_on_rocm_low_precision_part(monkeypatch):
    base = dict(use_turbo_gemm=True, fp8="e4m3", fp8_recipe="tensorwise", fp4=None, fp4_recipe=None)
    validate_args_on_rocm(SimpleNamespace(**base))
    with pytest.raises(AssertionError, match="delayed recipe is not support"):
        validate_args_on_rocm(SimpleNamespace(**{**base, "fp8_recipe": "delayed"}))
    monkeypatch.delenv("NVTE_ROCM_ENABLE_MXFP8", raising=False)
    with pytest.raises(AssertionError, match="NVTE_ROCM_ENABLE_MXFP8"):
        validate_args_on_rocm(SimpleNamespace(**{**base, "fp8_recipe": "mxfp8"}))
    monkeypatch.setenv("NVTE_ROCM_ENABLE_MXFP8", "1")
    validate_args_on_rocm(SimpleNamespace(**{**base, "fp8_recipe": "mxfp8"}))
    fp4 = dict(use_turbo_gemm=True, fp8=None, fp8_recipe=None, fp4="e2m1", fp4_recipe="mxfp4")
    validate_args_on_rocm(SimpleNamespace(**fp4))
    with pytest.raises(AssertionError, match="nvfp4 recipe is not support"):
        validate_args_on_rocm(SimpleNamespace(**{**fp4, "fp4_recipe": "nvfp4"}))
    with pytest.raises(ValueError, match="fp4_use_native_te_autocast"):
        validate_args_on_rocm(SimpleNamespace(**{**fp4, "fp4_use_native_te_autocast": True}))
    validate_args_on_rocm(SimpleNamespace(**{**fp4, "fp4_use_native_te_autocast": True, "transformer_impl": "local"}))
    with pytest.raises(AssertionError, match="use_turbo_parallel_linear"):
        validate_args_on_rocm(SimpleNamespace(**{**base, "use_turbo_parallel_linear": True}))


# --------------------------------------------------------------------------- a12
@pytest.mark.parametrize("M,N", [(128, 256), (512, 256), (100, 96), (1, 32)])
@pytest.mark.parametrize("shuffle", [False, True])
def test_dual_quantize_output_contract(M, N, shuffle):
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        row, row_s, col, col_s = torch.ops.primus_amd.quantize_mxfp4_dual(
            x, torch.float4_e2m1fn_x2, 128, False, False, False, False, False, False, shuffle, False, shuffle, False)
    M_pad, N_pad = -(-M // 128) * 128, -(-N // 128) * 128
    assert row.dtype == col.dtype == torch.float4_e2m1fn_x2
    assert row_s.dtype == col_s.dtype == torch.float8_e8m0fnu
    assert tuple(row.shape) == (M, N_pad // 2) and tuple(col.shape) == (N, M_pad // 2)  # col-wise copy is transposed
    if shuffle:
        assert tuple(row_s.shape) == (-(-M // 256) * 256, -(-(N_pad // 32) // 8) * 8)
        assert tuple(col_s.shape) == (-(-N // 256) * 256, -(-(M_pad // 32) // 8) * 8)
    else:
        assert tuple(row_s.shape) == (M, N_pad // 32) and tuple(col_s.shape) == (N, M_pad // 32)


def test_dual_quantize_recipes_per_operand(monkeypatch):
    calls = []
    monkeypatch.setattr(mxfp4_local, "_quantize_mxfp4_dual_op", lambda *a: calls.append(a[1:]) or (None,) * 4)
    x = torch.empty(4, 32)
    mxfp4_local._quantize_input_dual(x)
    mxfp4_local._quantize_weight_dual(x)
    mxfp4_local._quantize_grad_dual(x, use_sr=True)
    mxfp4_local._quantize_input_dual(x, preshuffle=True, use_rht=True)
    fp4, pad = torch.float4_e2m1fn_x2, 128
    #            dtype pad  r2d   rsr    rrht   c2d   csr    crht   shuffles
    # activations and gradients: transform on the col-wise copy (the reference's recipes, :234-250, :272-288)
    assert calls[0] == (fp4, pad, False, False, False, False, False, True, False, False, False, False)
    assert calls[1] == (fp4, pad, True, False, False, True, False, False, False, False, False, False)
    assert calls[2] == (fp4, pad, False, True, False, False, True, True, False, False, False, False)
    # the reference's activation recipe: transform on the col-wise copy only; shuffled scales, shuffled col data
    assert calls[3] == (fp4, pad, False, False, False, False, False, True, True, False, True, True)


def test_preshuffle_switch_follows_the_reference_environment(monkeypatch):
    """_enable_preshuffle (primus_turbo_mxfp4_local.py:61-74): on when the FP4 GEMM backend is pinned to AITER and
    autotuning is off; the contract check never refuses here."""
    monkeypatch.delenv("PRIMUS_TURBO_GEMM_BACKEND", raising=False)
    monkeypatch.delenv("PRIMUS_TURBO_AUTO_TUNE", raising=False)
    assert mxfp4_local._enable_preshuffle() is False
    monkeypatch.setenv("PRIMUS_TURBO_GEMM_BACKEND", "FP4:AITER")
    assert mxfp4_local._enable_preshuffle() is True
    monkeypatch.setenv("PRIMUS_TURBO_GEMM_BACKEND", "fp8:hipblaslt, fp4:aiter")
    assert mxfp4_local._enable_preshuffle() is True
    monkeypatch.setenv("PRIMUS_TURBO_AUTO_TUNE", "1")
    assert mxfp4_local._enable_preshuffle() is False
    monkeypatch.setenv("PRIMUS_TURBO_GEMM_BACKEND", "FP4:HIPBLASLT")
    monkeypatch.delenv("PRIMUS_TURBO_AUTO_TUNE")
    assert mxfp4_local._enable_preshuffle() is False
    import types
    assert mxfp4_local._assert_preshuffle_contract(types.SimpleNamespace(fp4="mxfp4"), False) is None


# --------------------------------------------------------------------------- a13
def test_local_shard_qdq_keeps_tile_coordinates(monkeypatch):
    calls = []
    monkeypatch.setattr(weight_deosc, "qdq_mxfp4", lambda t: calls.append(t.clone()) or t)
    shape = (128, 64)
    start, end = 35 * 64 + 5, 80 * 64 + 7
    shard = torch.linspace(1.0001, 2.0001, end - start, dtype=torch.float32)
    q = weight_deosc.qdq_mxfp4_local_shard(shard, shape, start, end, torch.bfloat16)
    assert q.dtype == torch.bfloat16 and torch.equal(q, shard.to(torch.bfloat16))
    assert len(calls) == 1 and calls[0].shape == (64, 64)  # rows 32..96 of the full weight
    flat = calls[0].reshape(-1)
    b0, b1 = (35 - 32) * 64 + 5, (80 - 32) * 64 + 7
    assert torch.count_nonzero(flat[:b0]) == 0 and torch.count_nonzero(flat[b1:]) == 0
    assert torch.equal(flat[b0:b1], shard.to(torch.bfloat16))


def test_local_shard_qdq_treats_experts_as_independent_matrices(monkeypatch):
    calls = []
    monkeypatch.setattr(weight_deosc, "qdq_mxfp4", lambda t: calls.append(t.clone()) or t)
    shape = (3, 64, 64)
    start, end = 40 * 64 + 3, 2 * 64 * 64 + 10 * 64 + 5
    shard = torch.arange(end - start, dtype=torch.float32)
    q = weight_deosc.qdq_mxfp4_local_shard(shard, shape, start, end, torch.bfloat16)
    assert torch.equal(q, shard.to(torch.bfloat16))
    assert [tuple(t.shape) for t in calls] == [(32, 64), (64, 64), (32, 64)]
    with pytest.raises(ValueError):
        weight_deosc.qdq_mxfp4_local_shard(shard, shape, start, end + 1, torch.bfloat16)
    with pytest.raises(ValueError):
        weight_deosc.qdq_mxfp4_local_shard(shard, (4,), 0, 4, torch.bfloat16)
    assert weight_deosc.qdq_mxfp4_local_shard(torch.empty(0), shape, 7, 7, torch.bfloat16).numel() == 0


# --------------------------------------------------------------------------- a14
def test_router_pad_multiple():
    assert pt.router_pad_multiple(True) == 0  # no low-precision recipe active
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=_mxfp8()):
        assert pt.router_pad_multiple(True) == 32
        assert pt.router_pad_multiple(False) == 0
    with pt.primus_turbo_fp8_autocast(enabled_turbo=True, turbo_quant_config=pt.PrimusTurboQuantConfig()):
        assert pt.router_pad_multiple(True) == 16
    with pt.primus_turbo_fp4_autocast(enabled_turbo=True, turbo_quant_config=_mxfp4()):
        assert pt.router_pad_multiple(True) == 32
    t = torch.tensor([0, 1, 32, 33])
    assert pt.pad_tokens_per_expert(t, 32).tolist() == [0, 32, 32, 64]
    assert pt.pad_tokens_per_expert(t, 0) is t
