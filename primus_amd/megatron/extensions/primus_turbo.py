"""Megatron-side host logic of the MX linear path.

What the reference keeps in
primus/backends/megatron/core/extensions/primus_turbo.py, restated without
Megatron-LM / Transformer Engine underneath:

* ``PrimusTurboQuantConfig`` (:425-495) and the recipe predicates,
* ``PrimusTurboLowPrecisionGlobalStateManager`` with the two autocast context
  managers (:498-653) and the per-module override (:656-738),
* cached quantised weight copies (:278-358) and the autograd bridge that
  routes their gradient into ``weight.main_grad`` (:141-275),
* the dense linear modules (:993-1828) and the grouped linear (:1983-2294),
* the router's padding multiple (:2344-2353).

The five module classes of the reference repeat one GEMM-selection block; here
it lives once in ``_LowPrecisionGemm`` and the classes differ only in what the
reference makes them differ in (normalisation in front, bias sharding names,
dense vs grouped operands).
"""

from __future__ import annotations

from contextlib import contextmanager, nullcontext
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ...pytorch import ops
from ...pytorch.core.low_precision import (
    Float4QuantConfig,
    Float8QuantConfig,
    Format,
    ScaleDtype,
    ScaleMode,
    ScalingGranularity,
    ScalingStrategy,
    check_fp8_support,
    check_mxfp4_support,
    check_mxfp8_support,
    float4_e2m1fn_x2,
    float8_e4m3,
)
from ...pytorch.core.quantized_tensor import QuantizedTensor, QuantizedTensorPair, create_quantized_weight
from .. import runtime
from ..enums import Fp4Recipe, Fp8Recipe

# Block sizes of the recipes (primus/backends/megatron/core/fp8_utils.py:47-48, fp4_utils.py:79)
SCALING_BLOCK_SIZE = 128
MXFP8_SCALING_BLOCK_SIZE = 32
MXFP4_SCALING_BLOCK_SIZE = 32


# ---------------------------------------------------------------------------
# a1  quant config
# ---------------------------------------------------------------------------
class PrimusTurboQuantConfig:
    """One object for both precisions: wraps a ``Float4QuantConfig`` when the
    format is ``E2M1_X2`` and a ``Float8QuantConfig`` otherwise
    (primus_turbo.py:425-459)."""

    def __init__(
        self,
        format: Format = Format.E4M3,
        granularity: ScalingGranularity = ScalingGranularity.TENSORWISE,
        strategy: ScalingStrategy = ScalingStrategy.DYNAMIC,
        scale_dtype: ScaleDtype = ScaleDtype.FP32,
        block_size: Optional[int] = None,
        use_gradient_sr: bool = True,
        scale_mode: ScaleMode = ScaleMode.OCP_FLOOR,
        activation_format: Optional[Format] = None,
    ):
        self._is_fp4 = format == Format.E2M1_X2
        self._is_fp8 = not self._is_fp4
        if self._is_fp4:
            extra = {} if activation_format is None else {"activation_format": activation_format}
            self._quant_config = Float4QuantConfig(
                format=format, granularity=granularity, strategy=strategy, scale_dtype=scale_dtype,
                block_size=block_size, use_gradient_sr=use_gradient_sr, scale_mode=scale_mode, **extra,
            )
        else:
            self._quant_config = Float8QuantConfig(
                format=format, granularity=granularity, strategy=strategy, scale_dtype=scale_dtype,
                block_size=block_size, scale_mode=scale_mode,
            )

    def data(self):
        return self._quant_config

    def is_fp4(self) -> bool:
        return self._is_fp4

    def is_fp8(self) -> bool:
        return self._is_fp8

    def _dynamic(self, granularity: ScalingGranularity) -> bool:
        c = self._quant_config
        return c.granularity == granularity and c.strategy == ScalingStrategy.DYNAMIC

    def block_scaling(self) -> bool:
        return self._dynamic(ScalingGranularity.BLOCKWISE)

    def current_scaling(self) -> bool:
        return self._dynamic(ScalingGranularity.TENSORWISE)

    def mxfp8_scaling(self) -> bool:
        # the MXFP8 recipe is E4M3 for every operand (primus_turbo.py:481-487)
        return self._dynamic(ScalingGranularity.MX_BLOCKWISE) and self._quant_config.format == Format.E4M3

    def mxfp4_scaling(self) -> bool:
        c = self._quant_config
        return (
            self._dynamic(ScalingGranularity.MX_BLOCKWISE)
            and c.format == Format.E2M1_X2
            and c.scale_dtype == ScaleDtype.E8M0
        )

    def __repr__(self):  # noqa: D105
        return f"PrimusTurboQuantConfig({self._quant_config!r})"


# ---------------------------------------------------------------------------
# a2  global low-precision state and the autocast context managers
# ---------------------------------------------------------------------------
class PrimusTurboLowPrecisionGlobalStateManager:
    """Class-level state read by every module's forward (primus_turbo.py:498-596).

    The first six fields are the ones the reference inherits from Transformer
    Engine's ``FP8GlobalStateManager``; they are carried here so that the saved
    and restored state is the same 9-tuple (:564-596)."""

    FP8_ENABLED: bool = False
    FP8_CALIBRATION: bool = False
    FP8_RECIPE: Any = None
    FP8_DISTRIBUTED_GROUP: Any = None
    IS_FIRST_FP8_MODULE: bool = False
    FP8_GRAPH_CAPTURING: bool = False
    FP8_AUTOCAST_DEPTH: int = 0

    PRIMUS_TURBO_QUANT_CONFIG: Optional[PrimusTurboQuantConfig] = None
    PRIMUS_TURBO_FP8_ENABLED: bool = False
    PRIMUS_TURBO_FP4_ENABLED: bool = False

    @classmethod
    def is_fp8_enabled(cls) -> bool:
        return cls.FP8_ENABLED

    @classmethod
    def is_turbo_fp8_enabled(cls) -> bool:
        return cls.PRIMUS_TURBO_FP8_ENABLED

    @classmethod
    def is_turbo_fp4_enabled(cls) -> bool:
        return cls.PRIMUS_TURBO_FP4_ENABLED

    @classmethod
    def get_turbo_quant_config(cls) -> Optional[PrimusTurboQuantConfig]:
        return cls.PRIMUS_TURBO_QUANT_CONFIG

    @classmethod
    def reset(cls) -> None:
        cls.FP8_ENABLED = False
        cls.FP8_CALIBRATION = False
        cls.FP8_RECIPE = None
        cls.FP8_DISTRIBUTED_GROUP = None
        cls.IS_FIRST_FP8_MODULE = False
        cls.FP8_GRAPH_CAPTURING = False
        cls.FP8_AUTOCAST_DEPTH = 0
        cls.PRIMUS_TURBO_FP8_ENABLED = False
        cls.PRIMUS_TURBO_FP4_ENABLED = False
        cls.PRIMUS_TURBO_QUANT_CONFIG = None

    @classmethod
    def autocast_enter(cls, enabled=False, calibrating=False, fp8_recipe=None, fp8_group=None, _graph=False,
                       enabled_turbo=False, turbo_quant_config: Optional[PrimusTurboQuantConfig] = None) -> None:
        cls.FP8_ENABLED = enabled
        cls.FP8_CALIBRATION = calibrating
        cls.FP8_RECIPE = fp8_recipe
        cls.FP8_DISTRIBUTED_GROUP = fp8_group
        cls.FP8_GRAPH_CAPTURING = _graph
        if cls.FP8_AUTOCAST_DEPTH == 0:
            cls.IS_FIRST_FP8_MODULE = True
        cls.FP8_AUTOCAST_DEPTH += 1

        # no config means the default one: FP8 tensorwise (primus_turbo.py:537-538)
        cfg = PrimusTurboQuantConfig() if turbo_quant_config is None else turbo_quant_config
        cls.PRIMUS_TURBO_FP8_ENABLED = bool(enabled_turbo and cfg.is_fp8())
        cls.PRIMUS_TURBO_FP4_ENABLED = bool(enabled_turbo and cfg.is_fp4())
        cls.PRIMUS_TURBO_QUANT_CONFIG = cfg

        if enabled_turbo:
            ok, why = check_fp8_support()
            assert ok, why
            if cfg.mxfp8_scaling():
                ok, why = check_mxfp8_support()
                assert ok, why
            if cfg.mxfp4_scaling():
                ok, why = check_mxfp4_support()
                assert ok, why

    @classmethod
    def autocast_exit(cls) -> None:
        cls.FP8_AUTOCAST_DEPTH = max(0, cls.FP8_AUTOCAST_DEPTH - 1)

    @classmethod
    def get_fp8_autocast_state(cls) -> Tuple:
        return (
            cls.FP8_ENABLED, cls.FP8_CALIBRATION, cls.FP8_RECIPE, cls.FP8_DISTRIBUTED_GROUP,
            cls.IS_FIRST_FP8_MODULE, cls.FP8_GRAPH_CAPTURING,
            cls.PRIMUS_TURBO_FP8_ENABLED, cls.PRIMUS_TURBO_FP4_ENABLED, cls.PRIMUS_TURBO_QUANT_CONFIG,
        )

    @classmethod
    def set_fp8_autocast_state(cls, state: Tuple) -> None:
        (
            cls.FP8_ENABLED, cls.FP8_CALIBRATION, cls.FP8_RECIPE, cls.FP8_DISTRIBUTED_GROUP,
            cls.IS_FIRST_FP8_MODULE, cls.FP8_GRAPH_CAPTURING,
            cls.PRIMUS_TURBO_FP8_ENABLED, cls.PRIMUS_TURBO_FP4_ENABLED, cls.PRIMUS_TURBO_QUANT_CONFIG,
        ) = state


@contextmanager
def primus_turbo_fp8_autocast(enabled: bool = True, calibrating: bool = False, fp8_recipe=None, fp8_group=None,
                              _graph: bool = False, enabled_turbo: bool = False,
                              turbo_quant_config: Optional[PrimusTurboQuantConfig] = None):
    """Scope in which the modules below quantise (primus_turbo.py:599-625): the
    previous state comes back on exit, exception or not."""
    manager = PrimusTurboLowPrecisionGlobalStateManager
    saved = manager.get_fp8_autocast_state()
    manager.autocast_enter(enabled=enabled, calibrating=calibrating, fp8_recipe=fp8_recipe, fp8_group=fp8_group,
                           _graph=_graph, enabled_turbo=enabled_turbo, turbo_quant_config=turbo_quant_config)
    try:
        yield
    finally:
        manager.set_fp8_autocast_state(saved)
        manager.autocast_exit()


@contextmanager
def primus_turbo_fp4_autocast(enabled: bool = True, calibrating: bool = False, fp4_recipe=None, fp4_group=None,
                              _graph: bool = False, enabled_turbo: bool = False,
                              turbo_quant_config: Optional[PrimusTurboQuantConfig] = None):
    """FP4 shares the FP8 state slots (primus_turbo.py:628-653)."""
    with primus_turbo_fp8_autocast(enabled=enabled, calibrating=calibrating, fp8_recipe=fp4_recipe,
                                   fp8_group=fp4_group, _graph=_graph, enabled_turbo=enabled_turbo,
                                   turbo_quant_config=turbo_quant_config):
        yield


# ---------------------------------------------------------------------------
# a3  per-module recipe override
# ---------------------------------------------------------------------------
@dataclass
class QuantizationRecipe:
    """Per-module override of the surrounding autocast (the fields the
    reference reads from Megatron's ``TEQuantizationRecipe``, primus_turbo.py:656-725)."""

    fp8_quantization_recipe: Optional[Fp8Recipe] = None
    fp4_quantization_recipe: Optional[Fp4Recipe] = None
    fp8_format: str = "e4m3"
    custom_recipe_factory: Optional[Callable] = None
    override_quantized_autocast: bool = True
    override_nonquantized_autocast: bool = False


@dataclass
class QuantizationParams:
    training_recipe: QuantizationRecipe
    evaluation_recipe: Optional[QuantizationRecipe] = None


def _get_fp8_autocast_for_quant_recipe(qrecipe: QuantizationRecipe):
    manager = PrimusTurboLowPrecisionGlobalStateManager
    overrides = qrecipe.override_quantized_autocast if manager.is_fp8_enabled() else qrecipe.override_nonquantized_autocast
    if not overrides:
        return nullcontext()
    fp8, fp4 = qrecipe.fp8_quantization_recipe, qrecipe.fp4_quantization_recipe
    if fp8 is None and fp4 is None:
        # this module runs in bf16 whatever the surrounding autocast says
        return primus_turbo_fp8_autocast(enabled=False, enabled_turbo=False)
    if fp8 == Fp8Recipe.custom or fp4 == Fp4Recipe.custom:
        assert qrecipe.custom_recipe_factory is not None
        raise AssertionError("Custom recipe is not supported for Primus-Turbo")
    if fp8 is not None:
        formats = {"e4m3": Format.E4M3, "hybrid": Format.HYBRID}
        if qrecipe.fp8_format not in formats:
            raise ValueError(f"Unhandled fp8_format {qrecipe.fp8_format}")
        fmt = formats[qrecipe.fp8_format]
        if fp8 == Fp8Recipe.tensorwise:
            cfg = PrimusTurboQuantConfig(granularity=ScalingGranularity.TENSORWISE, format=fmt)
        elif fp8 == Fp8Recipe.blockwise:
            cfg = PrimusTurboQuantConfig(granularity=ScalingGranularity.BLOCKWISE, format=fmt,
                                         block_size=SCALING_BLOCK_SIZE)
        elif fp8 == Fp8Recipe.mxfp8:
            cfg = PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=fmt,
                                         block_size=MXFP8_SCALING_BLOCK_SIZE, scale_dtype=ScaleDtype.E8M0)
        else:
            raise ValueError(f"Unhandled fp8 recipe: {fp8}")
        return primus_turbo_fp8_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=cfg)
    if fp4 == Fp4Recipe.nvfp4:
        raise AssertionError("NVFP4 is not supported for Primus-Turbo")
    if fp4 == Fp4Recipe.mxfp4:
        cfg = PrimusTurboQuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, format=Format.E2M1_X2,
                                     block_size=MXFP4_SCALING_BLOCK_SIZE, scale_dtype=ScaleDtype.E8M0)
        return primus_turbo_fp4_autocast(enabled=False, enabled_turbo=True, turbo_quant_config=cfg)
    raise ValueError(f"Unhandled fp4 recipe: {fp4}")


def _get_fp8_autocast_for_quant_params(qparams: Optional[QuantizationParams], training: bool):
    """primus_turbo.py:731-738."""
    if qparams is None:
        return nullcontext()
    if not training and qparams.evaluation_recipe is not None:
        return _get_fp8_autocast_for_quant_recipe(qparams.evaluation_recipe)
    return _get_fp8_autocast_for_quant_recipe(qparams.training_recipe)


def _use_split_wgrad_op() -> bool:
    """Zero-bubble pipelines split wgrad from dgrad; never together with a
    quantised recipe (primus_turbo.py:404-422)."""
    args = runtime.get_args()
    split = bool(getattr(args, "patch_zero_bubble", False) and getattr(args, "enable_zero_bubble", False))
    manager = PrimusTurboLowPrecisionGlobalStateManager
    if split:
        assert not (manager.is_turbo_fp8_enabled() or manager.is_turbo_fp4_enabled()), (
            "split wgrad op is not supported when turbo fp8 or fp4 is enabled."
        )
    return split


# ---------------------------------------------------------------------------
# a4  cached quantised weight copies
# ---------------------------------------------------------------------------
def _maybe_create_quantized_weight_buffers(weight: torch.Tensor, dest_dtype: torch.dtype,
                                           quant_config: PrimusTurboQuantConfig,
                                           disable_parameter_transpose_cache: bool):
    """``(rowwise, colwise_or_None)`` copies of ``weight`` ([N, K] or [G, N, K]).

    Row-wise (``axis=-1``) feeds the forward GEMM; the optional second copy is
    quantised along ``axis=-2`` and therefore stored transposed, for dgrad
    (primus_turbo.py:278-358).  MX weights use 2-D 32x32 blocks (:313-317), so
    one pass over the weight writes both copies."""
    return create_quantized_weight(
        weight, dest_dtype, quant_config.data(),
        need_weight_transpose_cache=not disable_parameter_transpose_cache,
    )


# ---------------------------------------------------------------------------
# a5  weight-gradient bridge
# ---------------------------------------------------------------------------
_dummy_wgrads: Dict[Tuple, torch.Tensor] = {}


def _get_dummy_wgrad(shape, dtype: torch.dtype, device=None, zero: bool = False) -> torch.Tensor:
    """A persistent placeholder gradient per (shape, dtype, device): handing it
    to autograd makes the parameter's grad-ready hooks fire although the real
    gradient went to ``main_grad`` (primus_turbo.py:141-163)."""
    device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    key = (tuple(shape), dtype, device)
    buf = _dummy_wgrads.get(key)
    if buf is None:
        buf = torch.empty(tuple(shape), dtype=dtype, device=device, requires_grad=False)
        _dummy_wgrads[key] = buf
    if zero:
        buf.fill_(0)
    return buf.detach()


class _WeightGradBridge(torch.autograd.Function):
    """Identity on ``(x, quantised copies)`` that ties the copies to the
    parameter they were made from: in backward the gradient computed with
    respect to the row-wise copy (weight-shaped bf16) is accumulated into
    ``weight.main_grad`` (primus_turbo.py:194-213)."""

    @staticmethod
    def forward(ctx, x, weight, quantized_weight, quantized_weight_trans, fuse_wgrad_accum):
        ctx.save_for_backward(weight)
        ctx.fuse_wgrad_accum = fuse_wgrad_accum
        return x, quantized_weight, quantized_weight_trans

    @staticmethod
    def backward(ctx, grad_x, grad_quantized_weight, grad_quantized_weight_trans):
        (weight,) = ctx.saved_tensors
        assert hasattr(weight, "main_grad"), "weight.main_grad should be set before backward pass."
        assert hasattr(weight, "grad_added_to_main_grad"), (
            "weight.grad_added_to_main_grad don't have grad_added_to_main_grad attribute."
        )
        if ctx.fuse_wgrad_accum:
            # the GEMM epilogue accumulated already; what arrives here is its placeholder
            weight.grad_added_to_main_grad = True
        elif not weight.grad_added_to_main_grad:
            weight.main_grad.add_(grad_quantized_weight)
            weight.grad_added_to_main_grad = True
        dummy = _get_dummy_wgrad(weight.shape, weight.dtype, weight.device)
        return grad_x, dummy, None, None, None


def _bridge_weight_grad(x: torch.Tensor, weight: torch.nn.Parameter, weight_buffer: QuantizedTensorPair,
                        fuse_wgrad_accum: bool = False):
    """Call before the GEMM: then in backward the GEMM's node runs first and
    hands the bridge the real weight gradient (primus_turbo.py:166-240)."""
    assert isinstance(weight_buffer, QuantizedTensorPair), "weight_buffer must be a QuantizedTensorPair"
    assert weight_buffer.data is not None, "weight_buffer.data must not be None"
    x, q, q_t = _WeightGradBridge.apply(x, weight, weight_buffer.data, weight_buffer.data_t, fuse_wgrad_accum)
    if fuse_wgrad_accum:
        # the GEMM resolves its accumulation target off the operand it is handed
        q.main_grad = weight.main_grad
        q.grad_added_to_main_grad = weight.grad_added_to_main_grad
    return x, QuantizedTensorPair(data=q, data_t=q_t)


def _fuse_wgrad_accum_pattern(config, weight: torch.Tensor) -> Optional[str]:
    """``"megatron"`` when the wgrad GEMM itself should add into
    ``weight.main_grad``, else None.  Only bf16/fp16 and FP8 tensorwise GEMMs
    have that epilogue; MXFP8, blockwise FP8 and every FP4 recipe keep the
    separate add (primus_turbo.py:243-275)."""
    if not getattr(config, "gradient_accumulation_fusion", False):
        return None
    manager = PrimusTurboLowPrecisionGlobalStateManager
    # the wgrad kernel of this package adds into a float32 buffer for every recipe; the reference's kernels do
    # so for bf16 and tensor-wise FP8 only, which stays the default (switch: turbo_fuse_wgrad_accum_mx, ours)
    mx_too = bool(getattr(runtime.get_args(), "turbo_fuse_wgrad_accum_mx", False))
    if manager.is_turbo_fp4_enabled():
        if not mx_too:
            return None
    elif manager.is_turbo_fp8_enabled():
        quant_config = manager.get_turbo_quant_config()
        if quant_config is None:
            return None
        if not quant_config.current_scaling() and not (mx_too and quant_config.mxfp8_scaling()):
            return None
    elif weight.dtype not in (torch.bfloat16, torch.float16):
        return None
    assert hasattr(weight, "main_grad") and hasattr(weight, "grad_added_to_main_grad"), (
        "gradient_accumulation_fusion is enabled but the weight carries neither main_grad nor "
        "grad_added_to_main_grad; they are set up by the distributed-data-parallel wrapper, so the module "
        "ran before the model was wrapped or a quantized buffer was passed instead of the parameter."
    )
    return "megatron"


# ---------------------------------------------------------------------------
# a6 / a7  the GEMM-selection block shared by all modules
# ---------------------------------------------------------------------------
class _LowPrecisionGemm:
    """Mixin: ``_gemm(x2d, weight, is_first_microbatch, group_lens=None)``.

    One microbatch per step: quantise the weight inside the op, every call.
    Several: quantise once in the first microbatch, keep both copies in
    ``quantized_weight_buffer`` / ``quantized_weight_t_buffer`` and bridge the
    gradient back (primus_turbo.py:1087-1196, :2115-2218)."""

    def _init_weight_cache(self, config) -> None:
        self.register_buffer("quantized_weight_buffer", None, persistent=False)
        self.register_buffer("quantized_weight_t_buffer", None, persistent=False)
        self.disable_parameter_transpose_cache = bool(getattr(config, "disable_parameter_transpose_cache", False))

    def _quantized(self, x, weight, is_first_microbatch, dest_dtype, quant_config, no_transpose_cache):
        if is_first_microbatch:
            self.quantized_weight_buffer, self.quantized_weight_t_buffer = _maybe_create_quantized_weight_buffers(
                weight, dest_dtype, quant_config, disable_parameter_transpose_cache=no_transpose_cache
            )
        assert self.quantized_weight_buffer is not None, (
            "no cached quantised weight: the first microbatch of a step must run with is_first_microbatch=True"
        )
        fuse_pattern = _fuse_wgrad_accum_pattern(self.config, weight)
        x, pair = _bridge_weight_grad(
            x, weight,
            QuantizedTensorPair(data=self.quantized_weight_buffer, data_t=self.quantized_weight_t_buffer),
            fuse_wgrad_accum=fuse_pattern is not None,
        )
        return x, pair, fuse_pattern

    def _gemm(self, x: torch.Tensor, weight: torch.Tensor, is_first_microbatch: bool,
              group_lens: Optional[torch.Tensor] = None, glu: Optional[Tuple] = None,
              norm: Optional[Tuple] = None) -> torch.Tensor:
        """``glu = (probs, row_mask, activation)``: ``x`` is the previous linear's output and the gated
        activation is applied on the way into this GEMM (grouped only).  ``norm = (weight, eps)``: ``x`` is
        the input of an RMSNorm that is applied on the way into this GEMM (dense only)."""
        manager = PrimusTurboLowPrecisionGlobalStateManager
        grouped = group_lens is not None
        one_microbatch = runtime.get_num_microbatches() == 1
        assert glu is None or grouped, "the activation prologue exists for the grouped (expert) linears only"
        assert norm is None or not grouped, "the normalisation prologue exists for the dense linears only"

        def run(op_dense, op_grouped, a, b, fuse_pattern, **kw):
            # the prologues are folded into the MX quantisers only: under the tensor-wise (current scaling) recipe,
            # as outside a low-precision autocast, the normalisation / activation runs as an operator of its own
            # in front of the GEMM, which is what the reference does (primus_turbo.py:1689-1741)
            mx = "config" in kw and kw["config"].granularity == ScalingGranularity.MX_BLOCKWISE
            if norm is not None:
                norm_weight, eps = norm
                if not mx:
                    return op_dense(ops.rmsnorm(a, norm_weight, eps), b, trans_a=False, trans_b=True, out_dtype=None,
                                    fuse_bgrad_accum_pattern=fuse_pattern, **kw)
                fused = ops.rmsnorm_gemm_fp8 if op_dense is ops.gemm_fp8 else ops.rmsnorm_gemm_fp4
                return fused(a, norm_weight, eps, b, trans_a=False, trans_b=True, out_dtype=None,
                             fuse_bgrad_accum_pattern=fuse_pattern, **kw)
            if glu is not None:
                probs, row_mask, activation = glu
                if not mx:
                    act = ops.swiglu_with_probs if activation == "silu" else ops.geglu_with_probs
                    return op_grouped(act(a, probs, row_mask), b, group_lens, trans_b=True,
                                      fuse_bgrad_accum_pattern=fuse_pattern, **kw)
                fused = ops.glu_grouped_gemm_fp8 if op_grouped is ops.grouped_gemm_fp8 else ops.glu_grouped_gemm_fp4
                return fused(a, probs, b, group_lens, activation=activation, row_mask=row_mask, trans_b=True,
                             fuse_bgrad_accum_pattern=fuse_pattern, **kw)
            if grouped:
                return op_grouped(a, b, group_lens, trans_b=True, fuse_bgrad_accum_pattern=fuse_pattern, **kw)
            return op_dense(a, b, trans_a=False, trans_b=True, out_dtype=None,
                            fuse_bgrad_accum_pattern=fuse_pattern, **kw)

        if manager.is_turbo_fp8_enabled():
            qc = manager.get_turbo_quant_config()
            assert qc.mxfp8_scaling() or qc.current_scaling() or qc.block_scaling(), (
                "Turbo FP8 is enabled but quant config is not mxfp8, current scaling, or block scaling."
            )
            # the 128-blockwise operator quantises from the bf16 weight at every call, whatever the number of
            # microbatches (same codes as a cached copy; its backward needs the bf16 weight for the other format anyway,
            # primus_turbo_float8_local.py:1059-1062)
            if one_microbatch or qc.block_scaling():
                return run(ops.gemm_fp8, ops.grouped_gemm_fp8, x, weight,
                           _fuse_wgrad_accum_pattern(self.config, weight), config=qc.data())
            x, pair, fuse_pattern = self._quantized(
                x, weight, is_first_microbatch, float8_e4m3, qc,
                self.disable_parameter_transpose_cache or qc.current_scaling(),
            )
            return run(ops.gemm_fp8, ops.grouped_gemm_fp8, x, pair, fuse_pattern, config=qc.data())

        if manager.is_turbo_fp4_enabled():
            qc = manager.get_turbo_quant_config()
            assert qc.mxfp4_scaling(), "Turbo FP4 is enabled but quant config is not mxfp4."
            if one_microbatch:
                if is_first_microbatch:
                    # nothing is cached on this path; the empty buffer marks the weight as one that the
                    # FP4 forward really quantises (read by weight de-oscillation, weight_deosc.py:148-151)
                    self.quantized_weight_buffer = torch.empty(0, device=weight.device, dtype=torch.uint8)
                return run(ops.gemm_fp4, ops.grouped_gemm_fp4, x, weight,
                           _fuse_wgrad_accum_pattern(self.config, weight), config=qc.data())
            x, pair, fuse_pattern = self._quantized(
                x, weight, is_first_microbatch, float4_e2m1fn_x2, qc, self.disable_parameter_transpose_cache
            )
            return run(ops.gemm_fp4, ops.grouped_gemm_fp4, x, pair, fuse_pattern, config=qc.data())

        return run(ops.gemm, ops.grouped_gemm, x, weight, _fuse_wgrad_accum_pattern(self.config, weight))


def _tensor_parallel_size(config) -> int:
    return int(getattr(config, "tensor_model_parallel_size", 1) or 1)


def _default_init(weight: torch.Tensor) -> None:
    torch.nn.init.normal_(weight, mean=0.0, std=0.02)


class PrimusTurboLinear(_LowPrecisionGemm, torch.nn.Module):
    """``y = x W^T (+ b)`` on ``[s, b, h]`` activations; returns ``(y, None)``
    (primus_turbo.py:993-1196).  Tensor parallelism must be 1 (:1035-1036)."""

    def __init__(self, input_size: int, output_size: int, *, parallel_mode: Optional[str] = None, config=None,
                 init_method: Optional[Callable] = None, bias: bool = True, skip_bias_add: bool = False,
                 skip_weight_param_allocation: bool = False, tp_comm_buffer_name: Optional[str] = None,
                 is_expert: bool = False, symmetric_ar_type: Optional[str] = None, tp_group=None):
        super().__init__()
        args = runtime.get_args()
        self.offload = bool(getattr(args, "offload", False)) and "parallel_gemm" in getattr(args, "offload_ops", ())
        assert not self.offload, "gemm offload still have some problems"
        if skip_weight_param_allocation:
            raise ValueError("PrimusTurbo linear layers own their weight; skip_weight_param_allocation is not supported")
        self.config = config
        self.in_features, self.out_features = int(input_size), int(output_size)
        self.parallel_mode = parallel_mode
        self.skip_bias_add = skip_bias_add
        self.is_expert = is_expert
        self.tp_size = _tensor_parallel_size(config)
        assert self.tp_size == 1, f"{type(self).__name__} only supports tensor parallel size = 1"
        dtype = getattr(config, "params_dtype", torch.bfloat16)
        device = None if getattr(config, "use_cpu_initialization", False) else _default_device()
        self.weight = torch.nn.Parameter(torch.empty(self.out_features, self.in_features, dtype=dtype, device=device))
        if getattr(config, "perform_initialization", True):
            (init_method or _default_init)(self.weight)
        self.use_bias = bool(bias)
        self.bias_names = ["bias"] if self.use_bias else []
        if self.use_bias:
            self.bias = torch.nn.Parameter(torch.zeros(self.out_features, dtype=dtype, device=device))
        else:
            self.register_parameter("bias", None)
        self.te_quant_params: Optional[QuantizationParams] = None
        self.is_first_microbatch = True
        self._init_weight_cache(config)

    def set_is_first_microbatch(self) -> None:
        """Called at the start of every optimizer step: the next forward
        re-quantises the weight."""
        self.is_first_microbatch = True

    def __repr__(self):  # noqa: D105
        return (f"{type(self).__name__}(in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.use_bias}, TP={self.tp_size})")

    def forward(self, x: torch.Tensor):
        first = self.is_first_microbatch
        with _get_fp8_autocast_for_quant_params(self.te_quant_params, self.training):
            out = self.forward_internal(x, first)
        self.is_first_microbatch = False
        return out

    def _prologue(self, x: torch.Tensor) -> torch.Tensor:
        return x

    def _norm_for_gemm(self, x: torch.Tensor) -> Optional[Tuple]:
        """``(weight, eps)`` if a normalisation in front of this linear is to be folded into the GEMM's
        quantiser; the plain linears have none."""
        return None

    def forward_internal(self, x: torch.Tensor, is_first_microbatch: bool = False):
        norm = self._norm_for_gemm(x)
        inp = x if norm is not None else self._prologue(x)
        weight = self._parameters["weight"]
        bias_tensor = torch.cat([getattr(self, n) for n in self.bias_names]) if self.use_bias else None
        shape = x.size()
        if not inp.is_contiguous():
            inp = inp.contiguous()
        inp = inp.view(-1, shape[-1])
        if _use_split_wgrad_op():
            raise NotImplementedError("the split-wgrad (zero-bubble) GEMM is a bf16 path outside this package")
        out = self._gemm(inp, weight, is_first_microbatch, norm=norm)
        out = out.view(shape[0], shape[1], -1)
        if bias_tensor is not None:
            out = out + bias_tensor
        return out, None


def _default_device():
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")


class PrimusTurboRowParallelLinear(PrimusTurboLinear):
    """Row-parallel flavour (primus_turbo.py:1199-1407); with TP = 1 the
    arithmetic is the plain linear."""

    def __init__(self, input_size: int, output_size: int, *, config=None, init_method: Optional[Callable] = None,
                 bias: bool = True, input_is_parallel: bool = True, skip_bias_add: bool = False,
                 is_expert: bool = False, tp_comm_buffer_name: Optional[str] = None, tp_group=None):
        if not input_is_parallel:
            raise ValueError("Transformer Engine linear layers do not support input_is_parallel = False")
        super().__init__(input_size, output_size, parallel_mode="row", config=config, init_method=init_method,
                         bias=bias, skip_bias_add=skip_bias_add, is_expert=is_expert,
                         tp_comm_buffer_name=tp_comm_buffer_name, tp_group=tp_group)


class PrimusTurboColumnParallelLinear(PrimusTurboLinear):
    """Column-parallel flavour (primus_turbo.py:1410-1611)."""

    def __init__(self, input_size: int, output_size: int, *, config=None, init_method: Optional[Callable] = None,
                 gather_output: bool = False, bias: bool = True, skip_bias_add: bool = False, is_expert: bool = False,
                 skip_weight_param_allocation: bool = False, tp_comm_buffer_name: Optional[str] = None, tp_group=None):
        if gather_output:
            raise ValueError("Transformer Engine linear layers do not support gather_output = True")
        super().__init__(input_size, output_size, parallel_mode="column", config=config, init_method=init_method,
                         bias=bias, skip_bias_add=skip_bias_add, is_expert=is_expert,
                         skip_weight_param_allocation=skip_weight_param_allocation,
                         tp_comm_buffer_name=tp_comm_buffer_name, tp_group=tp_group)


class PrimusTurboLayerNormColumnParallelLinear(PrimusTurboColumnParallelLinear):
    """LayerNorm / RMSNorm in front of the column-parallel linear
    (primus_turbo.py:1614-1828; normalisation selected at :1691-1700)."""

    def __init__(self, input_size: int, output_size: int, *, config=None, init_method: Optional[Callable] = None,
                 gather_output: bool = False, bias: bool = True, skip_bias_add: bool = False, is_expert: bool = False,
                 skip_weight_param_allocation: bool = False, tp_comm_buffer_name: Optional[str] = None, tp_group=None):
        super().__init__(input_size, output_size, config=config, init_method=init_method,
                         gather_output=gather_output, bias=bias, skip_bias_add=skip_bias_add, is_expert=is_expert,
                         skip_weight_param_allocation=skip_weight_param_allocation,
                         tp_comm_buffer_name=tp_comm_buffer_name, tp_group=tp_group)
        self.normalization = getattr(config, "normalization", "LayerNorm")
        self.eps = float(getattr(config, "layernorm_epsilon", 1e-5))
        # fold the RMSNorm into the quantiser of the GEMM's input (same values bit for bit, the normalised
        # tensor is never written); off = the reference's kernel sequence
        self.fuse_norm_into_quantize = bool(getattr(runtime.get_args(), "turbo_fuse_norm_into_quantize", True))
        dtype, device = self.weight.dtype, self.weight.device
        self.layer_norm_weight = torch.nn.Parameter(torch.ones(self.in_features, dtype=dtype, device=device))
        if self.normalization == "LayerNorm":
            self.layer_norm_bias = torch.nn.Parameter(torch.zeros(self.in_features, dtype=dtype, device=device))
        else:
            self.register_parameter("layer_norm_bias", None)

    def _native_rmsnorm_ok(self, x: torch.Tensor) -> bool:
        """The RMSNorm kernels take bf16 CUDA tensors with a last dim that is a multiple of 8 up to 16384."""
        k = x.size(-1)
        return (self.normalization == "RMSNorm" and x.is_cuda and x.dtype == torch.bfloat16
                and self.layer_norm_weight.dtype == torch.bfloat16 and k % 8 == 0 and k <= 16384)

    def _norm_for_gemm(self, x: torch.Tensor) -> Optional[Tuple]:
        if not (self.fuse_norm_into_quantize and self._native_rmsnorm_ok(x) and x.size(-1) % 32 == 0):
            return None
        return self.layer_norm_weight, self.eps

    def _prologue(self, x: torch.Tensor) -> torch.Tensor:
        if self.normalization == "LayerNorm":
            return torch.nn.functional.layer_norm(x, [x.size(-1)], self.layer_norm_weight, self.layer_norm_bias, self.eps)
        if self.normalization == "RMSNorm":
            if self._native_rmsnorm_ok(x):
                return ops.rmsnorm(x, self.layer_norm_weight, self.eps)     # primus_turbo.py:1696-1698
            # other dtypes / devices: the library routine (the reference's operator is GPU-only as well)
            return torch.nn.functional.rms_norm(x, [x.size(-1)], self.layer_norm_weight, self.eps)
        raise AssertionError("Not support normalization type.")


class PrimusTurboGroupedLinear(_LowPrecisionGemm, torch.nn.Module):
    """``num_gemms`` expert linears as one ``[G, out, in]`` parameter
    (``weights``) and one grouped GEMM; ``forward(x, m_splits)`` with
    ``m_splits`` = tokens per expert, kept on the device
    (primus_turbo.py:1983-2218).  Per-expert ``weight{i}`` entries are views of
    the consolidated parameter, registered lazily so that checkpoints keep the
    per-expert names (:2060-2092)."""

    def __init__(self, num_gemms: int, input_size: int, output_size: int, *, parallel_mode: Optional[str] = None,
                 config=None, init_method: Optional[Callable] = None, bias: bool = False, skip_bias_add: bool = False,
                 is_expert: bool = False, tp_comm_buffer_name: Optional[str] = None, pg_collection=None):
        super().__init__()
        args = runtime.get_args()
        self.offload = bool(getattr(args, "offload", False)) and "column_parallel_gemm" in getattr(args, "offload_ops", ())
        assert not self.offload, "gemm offload still have some problems"
        if bias:
            raise NotImplementedError("grouped linears of the MoE path carry no bias")
        self.config = config
        self.num_gemms = int(num_gemms)
        self.in_features, self.out_features = int(input_size), int(output_size)
        self.parallel_mode = parallel_mode
        self.use_bias = False
        self.skip_bias_add = skip_bias_add
        self.is_expert = is_expert
        self.tp_size = _tensor_parallel_size(config)
        assert self.tp_size == 1, f"{type(self).__name__} only supports tensor parallel size = 1"
        dtype = getattr(config, "params_dtype", torch.bfloat16)
        device = None if getattr(config, "use_cpu_initialization", False) else _default_device()
        weights = torch.empty(self.num_gemms, self.out_features, self.in_features, dtype=dtype, device=device)
        if getattr(config, "perform_initialization", True):
            with torch.no_grad():
                for i in range(self.num_gemms):
                    (init_method or _default_init)(weights[i])
        self.weights = torch.nn.Parameter(weights)
        self._weight_views_registered = False
        self.register_forward_pre_hook(self._forward_pre_hook_ensure_weight_views)
        self.te_quant_params: Optional[QuantizationParams] = None
        self.is_first_microbatch = True
        self._init_weight_cache(config)

    def set_is_first_microbatch(self) -> None:
        self.is_first_microbatch = True

    def _ensure_weight_views(self) -> None:
        if self._weight_views_registered:
            return
        for i in range(self.num_gemms):
            self.register_parameter(f"weight{i}", torch.nn.Parameter(self.weights[i], requires_grad=False))
        self._weight_views_registered = True

    @staticmethod
    def _forward_pre_hook_ensure_weight_views(module, _inputs):
        module._ensure_weight_views()

    def state_dict(self, *args, **kwargs):
        self._ensure_weight_views()
        return super().state_dict(*args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        # a checkpoint carries the per-expert names too; they load into views of ``weights``
        self._ensure_weight_views()
        return super()._load_from_state_dict(*args, **kwargs)

    def forward(self, x: torch.Tensor, m_splits: torch.Tensor, glu: Optional[Tuple] = None):
        """``glu = (probs [tokens], row_mask or None, "silu" | "gelu")`` makes this linear consume the
        previous one's output ``[tokens, 2 * in_features]`` through the gated activation (no
        counterpart in the reference, which runs the activation as its own kernel)."""
        first = self.is_first_microbatch
        with _get_fp8_autocast_for_quant_params(self.te_quant_params, self.training):
            out = self.forward_internal(x, m_splits, first, glu=glu)
        self.is_first_microbatch = False
        return out

    def forward_internal(self, x: torch.Tensor, m_splits: torch.Tensor, is_first_microbatch: bool = False,
                         glu: Optional[Tuple] = None):
        if not torch.is_tensor(m_splits):
            m_splits = torch.as_tensor(m_splits, dtype=torch.int64)
        if m_splits.device != x.device:
            m_splits = m_splits.to(x.device)  # the op consumes the lens on the device (no host read-back)
        return self._gemm(x, self.weights, is_first_microbatch, group_lens=m_splits, glu=glu), None


class PrimusTurboColumnParallelGroupedLinear(PrimusTurboGroupedLinear):
    """fc1 of the expert MLP (primus_turbo.py:2221-2256)."""

    def __init__(self, num_gemms: int, input_size: int, output_size: int, *, config=None,
                 init_method: Optional[Callable] = None, bias: bool = False, skip_bias_add: bool = False,
                 is_expert: bool = True, tp_comm_buffer_name: Optional[str] = None, pg_collection=None):
        super().__init__(num_gemms, input_size, output_size, parallel_mode="column", config=config,
                         init_method=init_method, bias=bias, skip_bias_add=skip_bias_add, is_expert=is_expert,
                         tp_comm_buffer_name=tp_comm_buffer_name, pg_collection=pg_collection)


class PrimusTurboRowParallelGroupedLinear(PrimusTurboGroupedLinear):
    """fc2 of the expert MLP (primus_turbo.py:2259-2294)."""

    def __init__(self, num_gemms: int, input_size: int, output_size: int, *, config=None,
                 init_method: Optional[Callable] = None, bias: bool = False, skip_bias_add: bool = False,
                 is_expert: bool = True, tp_comm_buffer_name: Optional[str] = None, pg_collection=None):
        super().__init__(num_gemms, input_size, output_size, parallel_mode="row", config=config,
                         init_method=init_method, bias=bias, skip_bias_add=skip_bias_add, is_expert=is_expert,
                         tp_comm_buffer_name=tp_comm_buffer_name, pg_collection=pg_collection)


# ---------------------------------------------------------------------------
# fused activation with router probabilities (primus_turbo.py:1954-1980)
# ---------------------------------------------------------------------------
def fused_bias_act_with_probs(intermediate_parallel: torch.Tensor, bias_parallel: Optional[torch.Tensor],
                              permuted_probs: torch.Tensor, tokens_per_experts: torch.Tensor,
                              activation_func: str) -> torch.Tensor:
    """``act(x[:, :F]) * x[:, F:] * probs`` with the rows past the routed tokens zeroed; ``x`` is
    fc1's output ``[tokens, 2F]``, ``activation_func`` "silu" or "gelu"."""
    assert intermediate_parallel.ndim == 2
    assert permuted_probs.ndim == 1
    assert tokens_per_experts.device == intermediate_parallel.device
    if bias_parallel is not None:
        intermediate_parallel = intermediate_parallel + bias_parallel
    row_mask = ops.tokens_per_expert_to_mask(tokens_per_experts, intermediate_parallel.shape[0])
    if activation_func == "silu":
        fused = ops.swiglu_with_probs
    elif activation_func == "gelu":
        fused = ops.geglu_with_probs
    else:
        raise ValueError(f"Activation function {activation_func} is not supported.")
    return fused(intermediate_parallel, permuted_probs, row_mask)


# ---------------------------------------------------------------------------
# a14  router-side padding multiple
# ---------------------------------------------------------------------------
def router_pad_multiple(moe_router_padding_for_quantization: bool) -> int:
    """Multiple the token dispatcher pads every expert's token count to, given
    the active recipe: 32 for MXFP8 and for FP4 (one MX block), 16 for the other
    FP8 recipes, 0 = no padding (primus_turbo.py:2344-2353)."""
    if not moe_router_padding_for_quantization:
        return 0
    manager = PrimusTurboLowPrecisionGlobalStateManager
    if manager.is_turbo_fp8_enabled():
        return 32 if manager.get_turbo_quant_config().mxfp8_scaling() else 16
    if manager.is_turbo_fp4_enabled():
        return 32
    return 0


def pad_tokens_per_expert(tokens_per_expert: torch.Tensor, multiple: int) -> torch.Tensor:
    """Token counts rounded up to ``multiple`` (device-side, no host sync)."""
    if multiple <= 0:
        return tokens_per_expert
    return (tokens_per_expert + (multiple - 1)) // multiple * multiple


__all__ = [
    "PrimusTurboQuantConfig", "PrimusTurboLowPrecisionGlobalStateManager", "primus_turbo_fp8_autocast",
    "primus_turbo_fp4_autocast", "QuantizationRecipe", "QuantizationParams", "PrimusTurboLinear",
    "PrimusTurboRowParallelLinear", "PrimusTurboColumnParallelLinear", "PrimusTurboLayerNormColumnParallelLinear",
    "PrimusTurboGroupedLinear", "PrimusTurboColumnParallelGroupedLinear", "PrimusTurboRowParallelGroupedLinear",
    "router_pad_multiple", "pad_tokens_per_expert", "fused_bias_act_with_probs", "QuantizedTensor", "QuantizedTensorPair",
]
