"""Tensor-level wrappers of the C-ABI extension (include/mxlinear.h).

The ``*_impl`` names follow the low-level entry points the reference calls
directly (gemm_fp8_impl: primus_turbo_float8_local.py:239-250; gemm_fp4_impl:
primus_turbo_mxfp4_local.py:319-331; grouped_gemm_fp8_impl /
grouped_gemm_fp8_variable_k_impl / group_offs_from_lens:
zbpp_gemm.py:585-603,710-724).  Every function launches on the current HIP
stream, allocates only its outputs and never reads device data from the host.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from ... import _lib
from ..core.low_precision import (
    ScalingGranularity,
    dtype_to_fmt_code,
    float4_e2m1fn_x2,
    float8_e4m3,
    float8_e5m2,
    float8_e8m0,
)

BLOCK = _lib.BLOCK

# Optional observer of kernel launches: ``hook(name, info)`` is entered as a
# context manager around every C-ABI call (benchmarks use it to bracket the
# launches with events on the launch stream).  None in normal operation.
_launch_hook = None


def set_launch_hook(hook) -> None:
    global _launch_hook
    _launch_hook = hook


class _NoHook:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_HOOK = _NoHook()


def _hooked(name: str, **info):
    return _launch_hook(name, info) if _launch_hook is not None else _NO_HOOK


# Seeds of the stochastic-rounding quantiser.  Every call draws the next seed of a sequence that
# depends only on the base seed (torch's global seed unless set here) and on the number of calls
# made so far: runs repeat after ``torch.manual_seed`` + ``manual_sr_seed(None)``, and nothing is
# read back from the device.
_sr_base: Optional[int] = None
_sr_calls = 0


def manual_sr_seed(seed: Optional[int]) -> None:
    """Restart the seed sequence of stochastic rounding from ``seed`` (``None``: from
    ``torch.initial_seed()`` as it is at the next draw)."""
    global _sr_base, _sr_calls
    _sr_base = None if seed is None else int(seed)
    _sr_calls = 0


def next_sr_seed() -> int:
    global _sr_calls
    base = torch.initial_seed() if _sr_base is None else _sr_base
    _sr_calls += 1
    return (base * 0x9E3779B97F4A7C15 + _sr_calls * 0xD1B54A32D192ED03) & 0xFFFFFFFFFFFFFFFF


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


KCHUNK = 128   # elements of a row that stay together in the K-chunk-major code layout (one GEMM K slot)
KSTEP = 64     # ... in the K-step-major layout (one MFMA K step); its scales travel in 16-byte panels (512 elements)
PANEL = 512

# Storage layouts of quantised operands, the value of the ``kchunk`` arguments below:
#   0 / False  row-major codes [rows, ld] and scales [rows, ld / 32]
#   1 / True   K-chunk-major codes [ld / 128, rows, 128 elements], row-major scales
#   2          K-step-major codes [ld / 64, rows, 64] and scales [panels, rows, 16] (FP8 formats only): what the
#              ring GEMM kernel reads; a transposed copy that is split into groups has its scale panels restart
#              at every group (ceil(ld / 512) + groups + 1 panels are allocated)
#   3          the K-step-major layout of E2M1 operands that meet E2M1 operands: steps of 128 elements, i.e. codes
#              [ld / 128, rows, 64 bytes] (the bytes of layout 1) with the scale panels of layout 2
LAYOUT_ROWMAJOR, LAYOUT_KCHUNK, LAYOUT_KSTEP, LAYOUT_KSTEP128 = 0, 1, 2, 3
RING_MAX_GROUPS = 256   # the ring GEMM kernel keeps its group tables for at most this many groups


def _layout(kchunk) -> int:
    if kchunk is True or kchunk is False or kchunk is None:
        return LAYOUT_KCHUNK if kchunk else LAYOUT_ROWMAJOR
    if int(kchunk) not in (0, 1, 2, 3):
        raise ValueError(f"unknown operand layout {kchunk!r}")
    return int(kchunk)


def _paneled(kchunk) -> bool:
    """Whether the layout keeps its scales in K-step-major panels."""
    return _layout(kchunk) >= LAYOUT_KSTEP


def _code_shape(rows: int, ld: int, per: int, kchunk):
    lay = _layout(kchunk)
    if lay == LAYOUT_KSTEP128 and per != 2:
        raise ValueError("the 128-element K-step layout holds E2M1 codes only")
    if lay == LAYOUT_KSTEP:
        return (ld // KSTEP, rows, KSTEP // per)
    return (ld // KCHUNK, rows, KCHUNK // per) if lay else (rows, ld // per)


def _scale_shape(rows: int, ld: int, kchunk, groups: int = 0):
    if _paneled(kchunk):
        return ((ld + PANEL - 1) // PANEL + (groups + 1 if groups else 0), rows, 16)
    return (rows, ld // BLOCK)


def _qflag(kchunk) -> int:
    return (0, _lib.QF_KCHUNK, _lib.QF_KSTEP, _lib.QF_KSTEP | _lib.QF_KSTEP128)[_layout(kchunk)]


def _gflag(kchunk) -> int:
    return (0, _lib.GF_KCHUNK, _lib.GF_KSTEP, _lib.GF_KSTEP)[_layout(kchunk)]


def pick_layout(groups: int, n: int, k: int, rows: int = 0, fp8: bool = True, fp4: bool = False) -> int:
    """Layout the differentiable operators store their quantised operands in: K-step-major when the activations and
    gradients are FP8 (``fp8``; steps of 64 elements, the weights FP8 or E2M1) or every operand is E2M1 (``fp4``; steps
    of 128 elements) and the groups fit the ring kernel -- also when the weight gradient is accumulated into float32
    inside the GEMM, which the ring kernel's wgrad instantiations do; otherwise K-chunk-major; row-major when the
    layouts are switched off or an operand reaches 4 GiB."""
    if not (kchunk_default() and kchunk_fits(groups, n, k, rows)):
        return LAYOUT_ROWMAJOR
    if (fp8 or fp4) and groups <= RING_MAX_GROUPS and _kstep_default:
        return LAYOUT_KSTEP if fp8 else LAYOUT_KSTEP128
    return LAYOUT_KCHUNK


_kstep_default = True


def set_kstep_default(enabled: bool) -> None:
    """Whether ``pick_layout`` may choose the K-step-major layout (default) or stops at K-chunk-major."""
    global _kstep_default
    _kstep_default = bool(enabled)


_kchunk_default = True


def set_kchunk_default(enabled: bool) -> None:
    """Whether the differentiable operators and ``create_quantized_weight`` store codes K-chunk-major
    (default) or row-major.  Results are identical; the GEMMs load the chunked layout faster."""
    global _kchunk_default
    _kchunk_default = bool(enabled)


def kchunk_default() -> bool:
    return _kchunk_default


def kchunk_fits(groups: int, n: int, k: int, rows: int = 0) -> bool:
    """The GEMMs address a K-chunk-major operand with 32-bit offsets from its base, so every operand of a
    linear with weights ``[groups, n, k]`` and ``rows`` tokens has to stay under 4 GiB."""
    np_, kp = _round_up(n, KCHUNK), _round_up(k, KCHUNK)
    limit = 1 << 32
    if groups * np_ * kp >= limit:
        return False
    w = padded_width(rows, groups) if rows else 0
    return w * max(np_, kp) < limit


def unchunk(codes: torch.Tensor) -> torch.Tensor:
    """K-chunk-major ``[ld / 128, rows, 128]`` or K-step-major ``[ld / 64, rows, 64]`` codes as a row-major
    ``[rows, ld]`` tensor (a copy)."""
    if codes.dim() != 3:
        raise ValueError("expected 3-D K-chunk-major codes")
    return codes.permute(1, 0, 2).reshape(codes.shape[1], codes.shape[0] * codes.shape[2])


def unpanel(scales: torch.Tensor, blocks: int) -> torch.Tensor:
    """K-step-major scales ``[panels, rows, 16]`` of an operand that is NOT split into groups as row-major
    ``[rows, blocks]`` (a copy)."""
    if scales.dim() != 3 or scales.shape[2] != 16:
        raise ValueError("expected 3-D K-step-major scales [panels, rows, 16]")
    panels, rows = scales.shape[0], scales.shape[1]
    # a panel row is [block parity][K step]: block 2 s + g of the panel sits at byte 8 g + s
    by_block = scales.reshape(panels, rows, 2, 8).permute(1, 0, 3, 2)
    return by_block.reshape(rows, panels * 16)[:, :blocks].contiguous()


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None or t.numel() == 0 else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("the MX linear path runs on the GPU only: got a CPU tensor")
        if not t.is_contiguous():
            raise ValueError("operands must be contiguous")


def _codes_u8(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.uint8 else t.view(torch.uint8)


def _per_byte(fmt: int) -> int:
    return 2 if fmt == _lib.FMT_E2M1 else 1


def _code_dtype(fmt: int) -> torch.dtype:
    return {_lib.FMT_E4M3: float8_e4m3, _lib.FMT_E2M1: float4_e2m1fn_x2, _lib.FMT_E5M2: float8_e5m2}[fmt]


def fmt_of(codes: torch.Tensor) -> int:
    return dtype_to_fmt_code(codes.dtype)


def padded_width(total_rows: int, num_groups: int) -> int:
    """Width of the segment-padded transposed layout (see mxl_padded_width)."""
    return _lib.padded_width(total_rows, num_groups)


def group_offs_from_lens(group_lens: torch.Tensor) -> torch.Tensor:
    """Exclusive prefix sum [G+1] of tokens-per-expert, on the device
    (zbpp_gemm.py:585).  The kernels here rebuild it themselves from
    ``group_lens``; it is provided for callers that keep it around."""
    offs = torch.zeros(group_lens.numel() + 1, dtype=torch.int64, device=group_lens.device)
    torch.cumsum(group_lens.to(torch.int64), dim=0, out=offs[1:])
    return offs


def _check_group_lens(group_lens: Optional[torch.Tensor], device) -> int:
    if group_lens is None:
        return 0
    if group_lens.dtype != torch.int64 or group_lens.dim() != 1:
        raise ValueError("group_lens must be a 1-D int64 tensor")
    if group_lens.device != device:
        raise ValueError("group_lens must live on the same device as the activations")
    if not group_lens.is_contiguous():
        raise ValueError("group_lens must be contiguous")
    if group_lens.numel() < 1 or group_lens.numel() > _lib.MAX_GROUPS:
        raise ValueError(f"number of groups must be in [1, {_lib.MAX_GROUPS}]")
    return group_lens.numel()


# --------------------------------------------------------------------------
# quantise / dequantise
# --------------------------------------------------------------------------
def quantize_mx_impl(
    x: torch.Tensor,
    fmt: int,
    scale_mode: int = _lib.SCALE_OCP_FLOOR,
    *,
    rowwise: bool = True,
    colwise: bool = False,
    group_lens: Optional[torch.Tensor] = None,
    pad_to: int = 1,
    sr_seed: Optional[int] = None,
    rht_signs: Optional[int] = None,
    kchunk=False,
):
    """MX-quantise bf16 ``x[rows, cols]``.

    ``kchunk`` stores the codes K-chunk-major, the layout the GEMMs load fastest: the code tensors come
    back 3-D, ``[ld / 128, rows, 128]`` (``64`` bytes in the last dim for FP4) instead of ``[rows, ld]``
    (``unchunk`` turns them back); the column count is padded to a multiple of 128; scales are unchanged.

    ``sr_seed`` (an integer; E2M1 only) rounds the codes stochastically instead of to nearest even
    (gradients of the MXFP4 recipe); the same seed reproduces the same codes.  ``rht_signs`` (16 sign
    bits; E2M1 only, needs ``colwise``) takes the transposed copy from the randomised Hadamard
    transform of ``x`` over groups of 16 tokens; both operands of a wgrad GEMM must use the same signs.

    ``pad_to`` rounds the column count of the row-wise copy up to a multiple
    (zero codes, scale byte 0 in the padding) so that it can feed a GEMM,
    whose contraction dim must be a multiple of 128.

    Returns ``(q_row, s_row, q_colT, s_colT)``; the pair that was not requested
    is ``None``.  ``q_row``: codes ``[rows, cols]`` (``cols/2`` bytes for FP4),
    ``s_row``: E8M0 ``[rows, cols/32]``.  ``q_colT``: codes of the transposed
    tensor ``[cols, W]`` with 32-blocks along the token dim that restart at
    each group boundary, ``W = padded_width(rows, G)``; ``s_colT``:
    ``[cols, W/32]``.
    """
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise ValueError("quantize expects a 2-D bfloat16 tensor")
    _require_cuda(x, group_lens)
    rows, cols = x.shape
    if cols % BLOCK != 0:
        raise ValueError(f"the quantised dim ({cols}) must be a multiple of {BLOCK}")
    if not (rowwise or colwise):
        raise ValueError("nothing to quantise: rowwise and colwise are both False")
    if (sr_seed is not None or rht_signs is not None) and fmt != _lib.FMT_E2M1:
        raise ValueError("stochastic rounding and the Hadamard transform exist for the E2M1 format only")
    if rht_signs is not None and not colwise:
        raise ValueError("the Hadamard transform applies to the transposed (colwise) copy")
    G = _check_group_lens(group_lens, x.device)
    per = _per_byte(fmt)
    dev = x.device
    q_row = s_row = q_col = s_col = None
    row_ld = _round_up(cols, KCHUNK if kchunk else pad_to)
    if rowwise:
        q_row = torch.empty(_code_shape(rows, row_ld, per, kchunk), dtype=torch.uint8, device=dev)
        s_row = torch.empty(_scale_shape(rows, row_ld, kchunk), dtype=torch.uint8, device=dev)
    if colwise:
        W = padded_width(rows, G)
        q_col = torch.empty(_code_shape(cols, W, per, kchunk), dtype=torch.uint8, device=dev)
        s_col = torch.empty(_scale_shape(cols, W, kchunk, G), dtype=torch.uint8, device=dev)
    if rows > 0 or (q_col is not None and q_col.numel() > 0):
        # with no tokens only the padding of the transposed copy is left to write
        row_ok = rows > 0
        args = (_ptr(x) if row_ok else None, rows, cols, row_ld, fmt, scale_mode, _ptr(group_lens), G,
                _ptr(q_row) if row_ok else None, _ptr(s_row) if row_ok else None, _ptr(q_col), _ptr(s_col))
        with _hooked("quantize", rows=rows, cols=cols, fmt=fmt, rowwise=rowwise, colwise=colwise):
            if sr_seed is None and rht_signs is None and not kchunk:
                rc = _lib.load().mxl_quantize(*args, _stream())
            else:
                flags = ((_lib.QF_SR if sr_seed is not None else 0) | (_lib.QF_RHT_COL if rht_signs is not None else 0)
                         | _qflag(kchunk))
                rc = _lib.load().mxl_quantize_ex(
                    *args, flags, int(sr_seed or 0) & 0xFFFFFFFFFFFFFFFF, int(rht_signs or 0) & 0xFFFF, _stream())
        _lib.check(rc, "mxl_quantize")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0)


def quantize_mx_weight_2d_impl(
    w: torch.Tensor,
    fmt: int,
    scale_mode: int = _lib.SCALE_OCP_FLOOR,
    *,
    rowwise: bool = True,
    colwise: bool = True,
    pad_to: int = 1,
    kchunk=False,
    col_scales_only: bool = False,
):
    """2-D (32x32 tile) MX quantisation of ``w[n, k]`` or ``w[G, n, k]``;
    returns ``(q_row [.., n, k], s_row [.., n, k/32], q_colT [.., k, n],
    s_colT [.., k, n/32])`` with ``None`` for a copy that was not requested.
    ``pad_to`` rounds the last dim of both copies up (zero padding).  With ``kchunk`` the codes come back
    K-chunk-major over the flattened batch: ``[k_ld / 128, G * n, 128]`` and ``[n_ld / 128, G * k, 128]``.
    ``col_scales_only`` (with ``rowwise`` and ``colwise``): the transposed copy's SCALES are written, its codes are not
    (``q_colT`` comes back None): with 2-D blocks they are the row-wise codes transposed, which the forward / dgrad
    GEMM reads as they lie (``b_transposed``)."""
    if w.dtype != torch.bfloat16 or w.dim() not in (2, 3):
        raise ValueError("weight quantisation expects a 2-D or 3-D bfloat16 tensor")
    _require_cuda(w)
    lead = tuple(w.shape[:-2])
    batch = 1 if not lead else lead[0]
    n, k = w.shape[-2], w.shape[-1]
    if n % BLOCK != 0 or k % BLOCK != 0:
        raise ValueError(f"2-D block quantisation needs both weight dims to be multiples of {BLOCK}, got {n}x{k}")
    if not (rowwise or colwise):
        raise ValueError("nothing to quantise: rowwise and colwise are both False")
    per = _per_byte(fmt)
    dev = w.device
    q_row = s_row = q_col = s_col = None
    k_ld, n_ld = _round_up(k, KCHUNK if kchunk else pad_to), _round_up(n, KCHUNK if kchunk else pad_to)
    if rowwise:
        shape = _code_shape(batch * n, k_ld, per, kchunk) if kchunk else lead + (n, k_ld // per)
        q_row = torch.empty(shape, dtype=torch.uint8, device=dev)
        sshape = _scale_shape(batch * n, k_ld, kchunk) if _paneled(kchunk) else lead + (n, k_ld // BLOCK)
        s_row = torch.empty(sshape, dtype=torch.uint8, device=dev)
    if col_scales_only and not (rowwise and colwise):
        raise ValueError("col_scales_only asks for the row-wise copy plus the transposed copy's scales")
    if colwise:
        if not col_scales_only:
            shape = _code_shape(batch * k, n_ld, per, kchunk) if kchunk else lead + (k, n_ld // per)
            q_col = torch.empty(shape, dtype=torch.uint8, device=dev)
        sshape = _scale_shape(batch * k, n_ld, kchunk) if _paneled(kchunk) else lead + (k, n_ld // BLOCK)
        s_col = torch.empty(sshape, dtype=torch.uint8, device=dev)
    with _hooked("quantize_weight_2d", rows=batch * n, cols=k, fmt=fmt, rowwise=rowwise, colwise=colwise and not col_scales_only):
        rc = _lib.load().mxl_quantize_weight_2d_ex(
            _ptr(w), batch, n, k, k_ld, n_ld, fmt, scale_mode, _ptr(q_row), _ptr(s_row), _ptr(q_col), _ptr(s_col),
            _qflag(kchunk), _stream()
        )
    _lib.check(rc, "mxl_quantize_weight_2d")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0)


def dequantize_mx_impl(codes: torch.Tensor, scales: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Row-wise layout back to bf16: ``out[..., k] = decode(codes) * 2^(scale-127)``."""
    _require_cuda(codes, scales)
    fmt = fmt_of(codes)
    per = _per_byte(fmt)
    k = codes.shape[-1] * per
    rows = codes.numel() // codes.shape[-1] if codes.numel() else 0
    if scales.shape[-1] * BLOCK != k or scales.numel() * BLOCK != rows * k:
        raise ValueError("scale shape does not match the codes (one E8M0 byte per 32 elements)")
    out = torch.empty(tuple(codes.shape[:-1]) + (k,), dtype=torch.bfloat16, device=codes.device)
    rc = _lib.load().mxl_dequantize(_ptr(codes), _ptr(scales), rows, k, fmt, _ptr(out), _stream())
    _lib.check(rc, "mxl_dequantize")
    return out if out_dtype == torch.bfloat16 else out.to(out_dtype)


# --------------------------------------------------------------------------
# GEMMs on pre-quantised operands
# --------------------------------------------------------------------------
GEMM_K_ALIGN = _lib.GEMM_K_ALIGN


def _pad_k(codes: torch.Tensor, scales: torch.Tensor, fmt: int):
    """The GEMM kernels take K in multiples of 128.  Operands produced with
    ``pad_to=128`` already are; anything else gets all-zero MX blocks (zero
    codes, scale 2^0) appended to every row, at the cost of a copy."""
    k = codes.shape[-1] * _per_byte(fmt)
    if k % GEMM_K_ALIGN == 0:
        return codes, scales, k
    kp = _round_up(k, GEMM_K_ALIGN)
    c = torch.nn.functional.pad(codes.view(torch.uint8), (0, (kp - k) // _per_byte(fmt)), value=0).view(codes.dtype)
    s = torch.nn.functional.pad(scales.view(torch.uint8), (0, (kp - k) // BLOCK), value=127).view(scales.dtype)
    return c, s, kp


def _check_contraction(k: int, kb: int) -> None:
    """The two contraction lengths agree, or one is the other padded to the GEMM's granularity (the operators pad
    activations, a copy made by ``QuantizedTensor.quantize`` is not padded)."""
    if k != kb and max(k, kb) != _round_up(min(k, kb), GEMM_K_ALIGN):
        raise ValueError(f"contraction dims differ: {k} vs {kb}")


def _check_out_dtype(out_dtype) -> None:
    if out_dtype not in (None, torch.bfloat16):
        raise ValueError("the MX GEMMs produce bfloat16 output")


def _chunked_dims(codes: torch.Tensor, fmt: int, kchunk=True):
    """(rows, k) of K-chunk-major codes [k / 128, rows, 128] or K-step-major codes [k / 64, rows, 64]."""
    step = KSTEP if _layout(kchunk) == LAYOUT_KSTEP else KCHUNK   # layout 3: 128-element steps
    if codes.dim() != 3 or codes.shape[2] * _per_byte(fmt) != step or not codes.is_contiguous():
        raise ValueError(f"chunked codes must be a contiguous [k / {step}, rows, {step}-element] tensor")
    return codes.shape[1], codes.shape[0] * step


def _check_scales(scales: torch.Tensor, rows: int, k: int, kchunk, what: str) -> None:
    if _paneled(kchunk):
        ok = scales.dim() == 3 and scales.shape[1] == rows and scales.shape[2] == 16 and scales.shape[0] * PANEL >= k
    else:
        ok = scales.numel() == rows * (k // BLOCK) and scales.shape[-1] == k // BLOCK
    if not ok or not scales.is_contiguous():
        raise ValueError(f"{what}: scale shape {tuple(scales.shape)} does not match {rows} rows x {k} elements")


def gemm_mx_nt_impl(a, a_scale, b, b_scale, out_dtype=torch.bfloat16, kchunk=False, b_transposed: bool = False,
                    b_shuffled: bool = False) -> torch.Tensor:
    """c[m, n] = dq(a)[m, k] . dq(b)[n, k]^T.  ``kchunk``: both code tensors are K-chunk-major.  ``b_transposed``: see
    ``grouped_gemm_mx_nt_impl``.  ``b_shuffled`` (row-major E2M1 operands, k a multiple of 128): the codes of ``b`` are
    in the pre-shuffled byte order of ``shuffle_codes_impl``."""
    _check_out_dtype(out_dtype)
    _require_cuda(a, a_scale, b, b_scale)
    a_fmt, b_fmt = fmt_of(a), fmt_of(b)
    if b_shuffled:
        m, n, k = a.shape[0], b.shape[0], a.shape[-1] * _per_byte(a_fmt)
        if kchunk or k % GEMM_K_ALIGN or b.shape[-1] * _per_byte(b_fmt) != k:
            raise ValueError("b_shuffled: row-major operands with the contraction length a multiple of 128")
        if tuple(a_scale.shape) != (m, k // BLOCK) or tuple(b_scale.shape) != (n, k // BLOCK):
            raise ValueError("scale shapes must be [rows, k/32]")
        c = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
        with _hooked("gemm_nt", m=m, n=n, k=k):
            rc = _lib.load().mxl_grouped_gemm_nt_ex(_ptr(a), _ptr(a_scale), a_fmt, _ptr(b), _ptr(b_scale), b_fmt, _ptr(c), None, 1,
                                                    m, n, k, _lib.GF_B_SHUFFLED, _stream())
        _lib.check(rc, "mxl_grouped_gemm_nt_ex")
        return c
    if kchunk:
        return grouped_gemm_mx_nt_impl(a, a_scale, b, b_scale if _paneled(kchunk) else b_scale.unsqueeze(0),
                                       None, kchunk=kchunk, b_transposed=b_transposed)
    _check_contraction(a.shape[-1] * _per_byte(a_fmt), b.shape[-1] * _per_byte(b_fmt))
    a, a_scale, k = _pad_k(a, a_scale, a_fmt)
    b, b_scale, kb = _pad_k(b, b_scale, b_fmt)
    m, n = a.shape[0], b.shape[0]
    if tuple(a_scale.shape) != (m, k // BLOCK) or tuple(b_scale.shape) != (n, k // BLOCK):
        raise ValueError("scale shapes must be [rows, k/32]")
    c = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    with _hooked("gemm_nt", m=m, n=n, k=k):
        rc = _lib.load().mxl_gemm_nt(_ptr(a), _ptr(a_scale), a_fmt, _ptr(b), _ptr(b_scale), b_fmt, _ptr(c), m, n, k, _stream())
    _lib.check(rc, "mxl_gemm_nt")
    return c


def grouped_gemm_mx_nt_impl(a, a_scale, b, b_scale, group_lens, out_dtype=torch.bfloat16, kchunk=False,
                            b_transposed: bool = False) -> torch.Tensor:
    """Forward / dgrad grouped GEMM: rows of ``a[total_m, k]`` split by
    ``group_lens``; ``b`` is ``[G, n, k]``.  ``kchunk``: both code tensors are K-chunk-major,
    ``a [k / 128, total_m, 128]`` and ``b [k / 128, G * n, 128]``; ``b_scale`` is ``[G, n, k / 32]`` as always.
    ``b_transposed`` (K-step-major FP8 operands, or E2M1 operands in 128-element steps): ``b`` holds the codes of the
    transposed matrices, ``[n_ld / 64, G * k, 64]`` (E2M1: ``[n_ld / 128, G * k, 64 bytes]``) -- the row-wise copy of a
    weight ``[G, k, n]`` serving its dgrad GEMM -- and ``b_scale`` the scale panels of ``[G * n, k]`` (the transposed
    copy's scales)."""
    _check_out_dtype(out_dtype)
    _require_cuda(a, a_scale, b, b_scale, group_lens)
    G = _check_group_lens(group_lens, a.device)
    a_fmt, b_fmt = fmt_of(a), fmt_of(b)
    if b_transposed:
        both4 = a_fmt == _lib.FMT_E2M1 and b_fmt == _lib.FMT_E2M1
        if _layout(kchunk) != (LAYOUT_KSTEP128 if both4 else LAYOUT_KSTEP):
            raise ValueError("b_transposed needs K-step-major operands (128-element steps when both are E2M1)")
        total_m, k = _chunked_dims(a, a_fmt, kchunk)
        groups = max(G, 1)
        bt_rows, n_ld = _chunked_dims(b, b_fmt, kchunk)           # rows = groups * k, width = n padded to 128
        if bt_rows != groups * k:
            raise ValueError("b_transposed: the rows of b's code array must be num_groups * k")
        if b_scale.dim() != 3 or b_scale.shape[2] != 16 or b_scale.shape[1] % groups:
            raise ValueError("b_transposed: b_scale must be the K-step-major scale panels of [num_groups * n, k]")
        n = b_scale.shape[1] // groups
        if _round_up(n, KCHUNK) != n_ld:
            raise ValueError("b_transposed: the code array's width does not match the scales' rows")
        _check_scales(a_scale, total_m, k, kchunk, "a_scale")
        _check_scales(b_scale, groups * n, k, kchunk, "b_scale")
        c = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
        with _hooked("grouped_gemm_nt" if G else "gemm_nt", m=total_m, n=n, k=k):
            rc = _lib.load().mxl_grouped_gemm_nt_ex(
                _ptr(a), _ptr(a_scale), a_fmt, _ptr(b), _ptr(b_scale), b_fmt, _ptr(c), _ptr(group_lens), groups, total_m, n, k,
                _lib.GF_KSTEP | _lib.GF_B_TRANSPOSED, _stream()
            )
        _lib.check(rc, "mxl_grouped_gemm_nt_ex")
        return c
    if kchunk:
        total_m, k = _chunked_dims(a, a_fmt, kchunk)
        b_rows, kb = _chunked_dims(b, b_fmt, kchunk)
        groups = max(G, 1)
        if _paneled(kchunk):
            if b_rows % groups:
                raise ValueError("the rows of b do not split into num_groups weights")
            n = b_rows // groups
        else:
            if b_scale.dim() != 3 or b_scale.shape[0] != groups or b_scale.shape[0] * b_scale.shape[1] != b_rows:
                raise ValueError("b_scale must be [num_groups, n, k/32] and match the rows of b")
            n = b_scale.shape[1]
        if k != kb:
            raise ValueError("contraction dims do not match")
        _check_scales(a_scale, total_m, k, kchunk, "a_scale")
        _check_scales(b_scale, b_rows, k, kchunk, "b_scale")
        c = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
        with _hooked("grouped_gemm_nt" if G else "gemm_nt", m=total_m, n=n, k=k):
            rc = _lib.load().mxl_grouped_gemm_nt_ex(
                _ptr(a), _ptr(a_scale), a_fmt, _ptr(b), _ptr(b_scale), b_fmt, _ptr(c), _ptr(group_lens), groups, total_m, n, k,
                _gflag(kchunk), _stream()
            )
        _lib.check(rc, "mxl_grouped_gemm_nt_ex")
        return c
    if b.dim() != 3 or b.shape[0] != G:
        raise ValueError("grouped GEMM expects weights of shape [num_groups, n, k]")
    _check_contraction(a.shape[-1] * _per_byte(a_fmt), b.shape[-1] * _per_byte(b_fmt))
    a, a_scale, k = _pad_k(a, a_scale, a_fmt)
    b, b_scale, kb = _pad_k(b, b_scale, b_fmt)
    total_m, n = a.shape[0], b.shape[1]
    if tuple(a_scale.shape) != (total_m, k // BLOCK) or tuple(b_scale.shape) != (G, n, k // BLOCK):
        raise ValueError("scale shapes must be [rows, k/32]")
    c = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
    with _hooked("grouped_gemm_nt", m=total_m, n=n, k=k):
        rc = _lib.load().mxl_grouped_gemm_nt(
            _ptr(a), _ptr(a_scale), a_fmt, _ptr(b), _ptr(b_scale), b_fmt, _ptr(c), _ptr(group_lens), G, total_m, n, k, _stream()
        )
    _lib.check(rc, "mxl_grouped_gemm_nt")
    return c


def _accum_target(accum_into, shape, kchunk, device):
    """Checks the float32 buffer a wgrad GEMM is to add its result to."""
    if _layout(kchunk) == LAYOUT_ROWMAJOR:
        raise ValueError("accumulating wgrad needs K-chunk-major or K-step-major operands")
    if (accum_into.dtype != torch.float32 or tuple(accum_into.shape) != tuple(shape) or not accum_into.is_contiguous()
            or accum_into.device != device):
        raise ValueError(f"accum_into must be a contiguous float32 tensor of shape {tuple(shape)} on the operands' device")
    return accum_into


def grouped_gemm_mx_wgrad_impl(a_t, a_t_scale, b_t, b_t_scale, group_lens, total_m, out_dtype=torch.bfloat16,
                               kchunk=False, accum_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Variable-K (wgrad) grouped GEMM on segment-padded transposed operands:
    ``a_t`` = dY^T codes ``[n, W]``, ``b_t`` = X^T codes ``[k, W]``; returns
    ``[G, n, k]`` (``[n, k]`` when ``group_lens`` is None).  An expert with no
    tokens gets a zero gradient."""
    _check_out_dtype(out_dtype)
    _require_cuda(a_t, a_t_scale, b_t, b_t_scale, group_lens)
    G = _check_group_lens(group_lens, a_t.device)
    a_fmt, b_fmt = fmt_of(a_t), fmt_of(b_t)
    W = padded_width(total_m, G)
    if kchunk:
        (n, wa), (k, wb) = _chunked_dims(a_t, a_fmt, kchunk), _chunked_dims(b_t, b_fmt, kchunk)
        if wa != W or wb != W:
            raise ValueError(f"transposed operands must have padded width {W}")
    else:
        n, k = a_t.shape[0], b_t.shape[0]
        if a_t.shape[1] * _per_byte(a_fmt) != W or b_t.shape[1] * _per_byte(b_fmt) != W:
            raise ValueError(f"transposed operands must have padded width {W}")
    if _paneled(kchunk):
        for sc, r in ((a_t_scale, n), (b_t_scale, k)):
            if tuple(sc.shape) != _scale_shape(r, W, kchunk, G) or not sc.is_contiguous():
                raise ValueError("K-step-major scales of the transposed operands must be [panels, rows, 16]")
    elif tuple(a_t_scale.shape) != (n, W // BLOCK) or tuple(b_t_scale.shape) != (k, W // BLOCK):
        raise ValueError("scale shapes must be [rows, W/32]")
    shape = (n, k) if group_lens is None else (G, n, k)
    flags = _gflag(kchunk)
    if accum_into is not None:
        # the result is added, in float32, to accum_into (which is returned)
        c = _accum_target(accum_into, shape, kchunk, a_t.device)
        flags |= _lib.GF_ACCUM_F32
    else:
        c = torch.empty(shape, dtype=torch.bfloat16, device=a_t.device)
    with _hooked("grouped_gemm_wgrad", m=total_m, n=n, k=k):
        rc = _lib.load().mxl_grouped_gemm_wgrad_ex(
            _ptr(a_t), _ptr(a_t_scale), a_fmt, _ptr(b_t), _ptr(b_t_scale), b_fmt, _ptr(c), _ptr(group_lens), G, total_m, n, k,
            flags, _stream()
        )
    _lib.check(rc, "mxl_grouped_gemm_wgrad")
    return c


# --------------------------------------------------------------------------
# gated activation with router probabilities
# --------------------------------------------------------------------------
_ACTS = {"silu": _lib.ACT_SILU, "gelu": _lib.ACT_GELU}


def _glu_args(x, probs, row_mask, activation):
    if activation not in _ACTS:
        raise ValueError(f"Activation function {activation} is not supported.")
    if x.dim() != 2 or x.dtype != torch.bfloat16 or x.shape[1] % 16 != 0:
        raise ValueError("expected a 2-D bfloat16 tensor [tokens, 2F] with F a multiple of 8")
    if probs.dim() != 1 or probs.shape[0] != x.shape[0] or probs.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("probs must be a 1-D float32 or bfloat16 tensor with one entry per token")
    if row_mask is not None:
        if row_mask.dim() != 1 or row_mask.shape[0] != x.shape[0]:
            raise ValueError("row_mask must have one entry per token")
        if row_mask.dtype == torch.bool:
            row_mask = row_mask.view(torch.uint8)
        if row_mask.dtype != torch.uint8:
            raise ValueError("row_mask must be a bool or uint8 tensor")
    _require_cuda(x, probs, row_mask)
    pd = _lib.PROBS_BF16 if probs.dtype == torch.bfloat16 else _lib.PROBS_F32
    return _ACTS[activation], pd, row_mask


def _bf16_tile_flag(tile: Optional[int]) -> int:
    if tile is None:
        return 0
    if tile not in (128, 256):
        raise ValueError("tile must be None (the library picks), 128 or 256")
    return _lib.BF_TILE_128 if tile == 128 else _lib.BF_TILE_256


def grouped_gemm_bf16_impl(a: torch.Tensor, b: torch.Tensor, group_lens: Optional[torch.Tensor], b_kn: bool = False,
                           tile: Optional[int] = None) -> torch.Tensor:
    """Grouped GEMM on unquantised bf16 operands: the rows of ``a [total_m, k]`` are split by ``group_lens`` (device,
    never read back) and group g is multiplied by ``b[g]^T`` with ``b [G, n, k]``, or by ``b[g]`` with ``b [G, k, n]``
    when ``b_kn``.  ``group_lens`` None: one group (``b`` 2-D or with a leading 1).  ``tile``: height of the output
    tiles, 128 or 256 rows (None: picked from the average rows per group); the result is the same bit for bit."""
    _require_cuda(a, b, group_lens)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or a.dim() != 2:
        raise ValueError("the bf16 grouped GEMM takes a 2-D bf16 activation and a bf16 weight")
    G = _check_group_lens(group_lens, a.device) or 1
    b3 = b.reshape(1, *b.shape) if b.dim() == 2 else b
    if b3.dim() != 3 or b3.shape[0] != G:
        raise ValueError("b must be [G, n, k] (or [G, k, n]) with one matrix per group")
    total_m, k = a.shape
    kk, n = (b3.shape[1], b3.shape[2]) if b_kn else (b3.shape[2], b3.shape[1])
    if kk != k:
        raise ValueError("contraction lengths of a and b differ")
    if k % 32 != 0 or n % 8 != 0:
        raise ValueError("the bf16 grouped GEMM needs the contraction length in multiples of 32 and n in multiples of 8")
    out = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
    lib = _lib.load()
    with _hooked("grouped_gemm_bf16", m=total_m, n=n, k=k):
        rc = lib.mxl_grouped_gemm_bf16(_ptr(a), _ptr(b3), _ptr(out), _ptr(group_lens), G, total_m, n, k,
                                       (_lib.BF_B_KN if b_kn else 0) | _bf16_tile_flag(tile), _stream())
    _lib.check(rc, "mxl_grouped_gemm_bf16")
    return out


def grouped_gemm_bf16_wgrad_impl(p: torch.Tensor, q: torch.Tensor, group_lens: Optional[torch.Tensor],
                                 accum_into: Optional[torch.Tensor] = None, tile: Optional[int] = None) -> torch.Tensor:
    """``c[g] = p[rows of g]^T . q[rows of g]`` for bf16 ``p [total_m, m_out]``, ``q [total_m, n_out]``: ``[G, m_out,
    n_out]`` bf16, zeros for a group without tokens; or added to the float32 ``accum_into`` of that shape."""
    _require_cuda(p, q, group_lens, accum_into)
    if p.dtype != torch.bfloat16 or q.dtype != torch.bfloat16 or p.dim() != 2 or q.dim() != 2 or p.shape[0] != q.shape[0]:
        raise ValueError("the bf16 weight-gradient GEMM takes two 2-D bf16 tensors with the same number of rows")
    G = _check_group_lens(group_lens, p.device) or 1
    total_m, m_out = p.shape
    n_out = q.shape[1]
    if m_out % 8 != 0 or n_out % 8 != 0:
        raise ValueError("the bf16 weight-gradient GEMM needs both output dims in multiples of 8")
    if accum_into is not None:
        if accum_into.dtype != torch.float32 or accum_into.numel() != G * m_out * n_out:
            raise ValueError("accum_into must be a contiguous float32 buffer of the weight's size")
        out = accum_into
    else:
        out = torch.empty((G, m_out, n_out), dtype=torch.bfloat16, device=p.device)
    lib = _lib.load()
    with _hooked("grouped_gemm_bf16_wgrad", m=total_m, n=m_out, k=n_out):
        rc = lib.mxl_grouped_gemm_bf16_wgrad(_ptr(p), _ptr(q), _ptr(out), _ptr(group_lens), G, total_m, m_out, n_out,
                                             (_lib.BF_ACCUM_F32 if accum_into is not None else 0) | _bf16_tile_flag(tile), _stream())
    _lib.check(rc, "mxl_grouped_gemm_bf16_wgrad")
    return out


def glu_with_probs_fwd_impl(x, probs, row_mask, activation: str) -> torch.Tensor:
    """``act(x[:, :F]) * x[:, F:] * probs[:, None]`` in fp32, one rounding to bf16; masked rows give 0."""
    act, pd, row_mask = _glu_args(x, probs, row_mask, activation)
    rows, f = x.shape[0], x.shape[1] // 2
    y = torch.empty((rows, f), dtype=torch.bfloat16, device=x.device)
    with _hooked("glu_probs_fwd", rows=rows, f=f):
        rc = _lib.load().mxl_glu_probs_fwd(_ptr(x), _ptr(probs), pd, _ptr(row_mask), rows, f, act, _ptr(y), _stream())
    _lib.check(rc, "mxl_glu_probs_fwd")
    return y


def glu_with_probs_bwd_impl(dy, x, probs, row_mask, activation: str):
    """``(dx [tokens, 2F] bf16, dprobs [tokens] fp32)``."""
    act, pd, row_mask = _glu_args(x, probs, row_mask, activation)
    rows, f = x.shape[0], x.shape[1] // 2
    if dy.dtype != torch.bfloat16 or tuple(dy.shape) != (rows, f):
        raise ValueError("dy must be bfloat16 [tokens, F]")
    _require_cuda(dy)
    dx = torch.empty_like(x)
    dp = torch.empty((rows,), dtype=torch.float32, device=x.device)
    with _hooked("glu_probs_bwd", rows=rows, f=f):
        rc = _lib.load().mxl_glu_probs_bwd(_ptr(dy), _ptr(x), _ptr(probs), pd, _ptr(row_mask), rows, f, act, _ptr(dx),
                                           _ptr(dp), _stream())
    _lib.check(rc, "mxl_glu_probs_bwd")
    return dx, dp


def glu_with_probs_quantize_impl(x, probs, row_mask, activation: str, fmt: int, scale_mode: int = _lib.SCALE_OCP_FLOOR, *,
                                 colwise: bool = False, group_lens: Optional[torch.Tensor] = None, pad_to: int = 1,
                                 kchunk=False):
    """``quantize_mx_impl(glu_with_probs_fwd_impl(x, ...))`` in one pass over ``x [tokens, 2F]``, the
    activated tensor never reaching memory; same return tuple (the row-wise copy is always produced)."""
    act, pd, row_mask = _glu_args(x, probs, row_mask, activation)
    _require_cuda(group_lens)
    rows, f = x.shape[0], x.shape[1] // 2
    if f % BLOCK != 0:
        raise ValueError(f"the quantised dim ({f}) must be a multiple of {BLOCK}")
    if rows == 0:  # nothing to activate: only the padding of the transposed copy is left to write
        return quantize_mx_impl(x[:, :f].contiguous(), fmt, scale_mode, rowwise=True, colwise=colwise,
                                group_lens=group_lens, pad_to=pad_to, kchunk=kchunk)
    G = _check_group_lens(group_lens, x.device)
    per = _per_byte(fmt)
    dev = x.device
    row_ld = _round_up(f, KCHUNK if kchunk else pad_to)
    q_row = torch.empty(_code_shape(rows, row_ld, per, kchunk), dtype=torch.uint8, device=dev)
    s_row = torch.empty(_scale_shape(rows, row_ld, kchunk), dtype=torch.uint8, device=dev)
    q_col = s_col = None
    if colwise:
        W = padded_width(rows, G)
        q_col = torch.empty(_code_shape(f, W, per, kchunk), dtype=torch.uint8, device=dev)
        s_col = torch.empty(_scale_shape(f, W, kchunk, G), dtype=torch.uint8, device=dev)
    if rows > 0 or (q_col is not None and q_col.numel() > 0):
        row_ok = rows > 0
        with _hooked("glu_probs_quantize", rows=rows, cols=f, fmt=fmt, rowwise=True, colwise=colwise):
            rc = _lib.load().mxl_glu_probs_quantize(
                _ptr(x) if row_ok else None, _ptr(probs), pd, _ptr(row_mask), rows, f, row_ld, act, fmt, scale_mode,
                _ptr(group_lens), G, _ptr(q_row) if row_ok else None, _ptr(s_row) if row_ok else None, _ptr(q_col),
                _ptr(s_col), _qflag(kchunk), _stream(),
            )
        _lib.check(rc, "mxl_glu_probs_quantize")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0)


# --------------------------------------------------------------------------
# Tensor-wise ("current") FP8 scaling: one fp32 scale per tensor
# (primus_turbo_float8_local.py:194-207 restates the arithmetic, :215-306 the operand flow)
# --------------------------------------------------------------------------
_TW_FMTS = (_lib.FMT_E4M3, _lib.FMT_E5M2)


def amax_impl(x: torch.Tensor) -> torch.Tensor:
    """``max |x|`` of a contiguous bfloat16 tensor as a float32 tensor of one element, on the device."""
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("expected a contiguous bfloat16 tensor")
    _require_cuda(x)
    out = torch.empty((1,), dtype=torch.float32, device=x.device)
    with _hooked("amax", n=x.numel()):
        rc = _lib.load().mxl_amax(_ptr(x) if x.numel() else None, x.numel(), _ptr(out), _stream())
    _lib.check(rc, "mxl_amax")
    return out


def quantize_tensorwise_impl(x, fmt: int, *, rowwise: bool = True, colwise: bool = False,
                             group_lens: Optional[torch.Tensor] = None, pad_to: int = 1, kchunk: bool = False,
                             amax: Optional[torch.Tensor] = None):
    """``(q_row, s_row, q_colT, s_colT, scale_inv)`` for a 2-D bfloat16 ``x``: codes in the layouts of
    ``quantize_mx_impl`` but scaled by ``fp8_max / max(amax, 1e-12)`` for the whole tensor; the ``s_*`` arrays
    hold the unit E8M0 byte (they only make the codes acceptable to the GEMMs), ``scale_inv`` is the float32
    reciprocal scale (one element, on the device).  ``fmt``: E4M3 or E5M2."""
    if fmt not in _TW_FMTS:
        raise ValueError("tensor-wise scaling produces E4M3 or E5M2 codes")
    if x.dim() != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("expected a contiguous 2-D bfloat16 tensor")
    if not (rowwise or colwise):
        raise ValueError("nothing to do: rowwise and colwise are both False")
    _require_cuda(x, group_lens, amax)
    rows, cols = x.shape
    if cols % BLOCK != 0:
        raise ValueError(f"the last dim ({cols}) must be a multiple of {BLOCK}")
    G = _check_group_lens(group_lens, x.device) if colwise else 0
    dev = x.device
    if amax is None:
        amax = amax_impl(x)
    scale_inv = torch.empty((1,), dtype=torch.float32, device=dev)
    q_row = s_row = q_col = s_col = None
    row_ld = _round_up(cols, KCHUNK if kchunk else pad_to)
    if rowwise:
        q_row = torch.empty(_code_shape(rows, row_ld, 1, kchunk), dtype=torch.uint8, device=dev)
        s_row = torch.empty(_scale_shape(rows, row_ld, kchunk), dtype=torch.uint8, device=dev)
    if colwise:
        W = padded_width(rows, G)
        q_col = torch.empty(_code_shape(cols, W, 1, kchunk), dtype=torch.uint8, device=dev)
        s_col = torch.empty(_scale_shape(cols, W, kchunk, G), dtype=torch.uint8, device=dev)
    if rows == 0 and not (colwise and q_col.numel()):
        scale_inv.fill_(1e-12 / (448.0 if fmt == _lib.FMT_E4M3 else 57344.0))
    else:
        with _hooked("quantize_tensorwise", rows=rows, cols=cols, fmt=fmt, rowwise=rowwise, colwise=colwise):
            rc = _lib.load().mxl_quantize_tensorwise(
                _ptr(x) if rows else None, rows, cols, row_ld if rowwise else 0, fmt, _ptr(amax),
                _ptr(group_lens) if colwise else None, G, _ptr(q_row) if rows else None, _ptr(s_row) if rows else None,
                _ptr(q_col), _ptr(s_col), _ptr(scale_inv), _qflag(kchunk), _stream(),
            )
        _lib.check(rc, "mxl_quantize_tensorwise")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0), scale_inv


def quantize_weight_tensorwise_impl(w, fmt: int, *, rowwise: bool = True, colwise: bool = False, pad_to: int = 1,
                                    kchunk: bool = False):
    """Weights ``[n, k]`` or ``[G, n, k]`` with one scale for the whole tensor: the row-wise copy and the
    transposed copy per matrix in the layouts of ``quantize_mx_weight_2d_impl``, plus ``scale_inv``."""
    if fmt not in _TW_FMTS:
        raise ValueError("tensor-wise scaling produces E4M3 or E5M2 codes")
    if w.dim() not in (2, 3) or w.dtype != torch.bfloat16 or not w.is_contiguous():
        raise ValueError("expected a contiguous bfloat16 weight [n, k] or [G, n, k]")
    _require_cuda(w)
    lead = tuple(w.shape[:-2])
    batch = 1 if not lead else lead[0]
    n, k = w.shape[-2], w.shape[-1]
    if n % BLOCK or k % BLOCK:
        raise ValueError(f"weight dims must be multiples of {BLOCK}")
    dev = w.device
    amax = amax_impl(w)
    scale_inv = torch.empty((1,), dtype=torch.float32, device=dev)
    k_ld, n_ld = _round_up(k, KCHUNK if kchunk else pad_to), _round_up(n, KCHUNK if kchunk else pad_to)
    q_row = s_row = q_col = s_col = None
    kstep = _paneled(kchunk)
    if rowwise:
        q_row = torch.empty(_code_shape(batch * n, k_ld, 1, kchunk) if kchunk else lead + (n, k_ld), dtype=torch.uint8, device=dev)
        s_row = torch.empty(_scale_shape(batch * n, k_ld, kchunk) if kstep else lead + (n, k_ld // BLOCK), dtype=torch.uint8, device=dev)
    if colwise:
        q_col = torch.empty(_code_shape(batch * k, n_ld, 1, kchunk) if kchunk else lead + (k, n_ld), dtype=torch.uint8, device=dev)
        s_col = torch.empty(_scale_shape(batch * k, n_ld, kchunk) if kstep else lead + (k, n_ld // BLOCK), dtype=torch.uint8, device=dev)
    with _hooked("quantize_weight_tensorwise", rows=batch * n, cols=k, fmt=fmt, rowwise=rowwise, colwise=colwise):
        rc = _lib.load().mxl_quantize_weight_tensorwise(
            _ptr(w), batch, n, k, k_ld, n_ld, fmt, _ptr(amax), _ptr(q_row), _ptr(s_row), _ptr(q_col), _ptr(s_col),
            _ptr(scale_inv), _qflag(kchunk), _stream(),
        )
    _lib.check(rc, "mxl_quantize_weight_tensorwise")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0), scale_inv


def _alpha_ok(*alphas):
    for t in alphas:
        if t.dtype != torch.float32 or t.numel() != 1:
            raise ValueError("per-tensor factors must be float32 tensors of one element")
    _require_cuda(*alphas)


def gemm_tw_nt_impl(a, a_unit, a_scale_inv, b, b_unit, b_scale_inv, group_lens=None, kchunk: bool = False,
                    b_transposed_n: Optional[int] = None) -> torch.Tensor:
    """``c = (a . b^T) * a_scale_inv * b_scale_inv`` on tensor-wise scaled codes, dense (``group_lens`` None,
    ``b [n, k]``) or grouped (``b [G, n, k]``); layouts and the unit block scales as the quantisers above
    return them (``b_unit`` is ``[n, k/32]`` or ``[G, n, k/32]``).  The contraction dim must be padded to 128.
    ``b_transposed_n`` (K-step-major E4M3 weights): ``b`` holds the ROW-WISE codes of the weight ``[G, k, n]`` whose
    transpose this GEMM multiplies by (its dgrad: one scale per tensor, so the transposed copy would be the same
    codes transposed), ``[n_ld / 64, G * k, 64]``; the value is ``n``, the number of output columns."""
    _require_cuda(a, a_unit, b, b_unit, group_lens)
    _alpha_ok(a_scale_inv, b_scale_inv)
    G = _check_group_lens(group_lens, a.device)
    groups = max(G, 1)
    a_fmt, b_fmt = fmt_of(a), fmt_of(b)
    if b_transposed_n is not None:
        if _layout(kchunk) != LAYOUT_KSTEP:
            raise ValueError("b_transposed_n needs K-step-major operands")
        total_m, k = _chunked_dims(a, a_fmt, kchunk)
        bt_rows, n_ld = _chunked_dims(b, b_fmt, kchunk)
        n = int(b_transposed_n)
        if bt_rows != groups * k or _round_up(n, KCHUNK) != n_ld:
            raise ValueError("b_transposed_n: b must be the K-step-major row-wise codes of a [num_groups, k, n] weight")
        c = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
        with _hooked("grouped_gemm_nt" if G else "gemm_nt", m=total_m, n=n, k=k):
            rc = _lib.load().mxl_grouped_gemm_nt_scaled(
                _ptr(a), _ptr(a_unit), a_fmt, _ptr(b), None, b_fmt, _ptr(c), _ptr(group_lens), groups, total_m, n, k,
                _ptr(a_scale_inv), _ptr(b_scale_inv), _lib.GF_KSTEP | _lib.GF_B_TRANSPOSED, _stream(),
            )
        _lib.check(rc, "mxl_grouped_gemm_nt_scaled")
        return c
    kstep = _paneled(kchunk)
    if kchunk:
        total_m, k = _chunked_dims(a, a_fmt, kchunk)
        b_rows, kb = _chunked_dims(b, b_fmt, kchunk)
    else:
        total_m, k = a.shape
        b_rows, kb = b.numel() // b.shape[-1], b.shape[-1]
    if kstep:
        if b_rows % groups:
            raise ValueError("the rows of b do not split into num_groups weights")
        n = b_rows // groups
        if k != kb or k % _lib.GEMM_K_ALIGN:
            raise ValueError("operand shapes do not match (the contraction dim must be padded to 128)")
        _check_scales(a_unit, total_m, k, kchunk, "a_unit")
        _check_scales(b_unit, b_rows, k, kchunk, "b_unit")
    else:
        n = b_unit.shape[-2]
        if k != kb or k % _lib.GEMM_K_ALIGN or b_rows != groups * n or b_unit.numel() != b_rows * (k // BLOCK):
            raise ValueError("operand shapes do not match (the contraction dim must be padded to 128)")
        if tuple(a_unit.shape) != (total_m, k // BLOCK):
            raise ValueError("scale shapes must be [rows, k/32]")
    c = torch.empty((total_m, n), dtype=torch.bfloat16, device=a.device)
    with _hooked("grouped_gemm_nt" if G else "gemm_nt", m=total_m, n=n, k=k):
        rc = _lib.load().mxl_grouped_gemm_nt_scaled(
            _ptr(a), _ptr(a_unit), a_fmt, _ptr(b), _ptr(b_unit), b_fmt, _ptr(c), _ptr(group_lens), groups, total_m, n, k,
            _ptr(a_scale_inv), _ptr(b_scale_inv), _gflag(kchunk), _stream(),
        )
    _lib.check(rc, "mxl_grouped_gemm_nt_scaled")
    return c


def gemm_tw_wgrad_impl(a_t, a_t_unit, a_scale_inv, b_t, b_t_unit, b_scale_inv, group_lens, total_m,
                       kchunk: bool = False, accum_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Variable-K (wgrad) GEMM on tensor-wise scaled transposed operands, times the two factors; shapes as
    ``grouped_gemm_mx_wgrad_impl`` (also ``accum_into``)."""
    _require_cuda(a_t, a_t_unit, b_t, b_t_unit, group_lens)
    _alpha_ok(a_scale_inv, b_scale_inv)
    G = _check_group_lens(group_lens, a_t.device)
    a_fmt, b_fmt = fmt_of(a_t), fmt_of(b_t)
    W = padded_width(total_m, G)
    kstep = _paneled(kchunk)
    if kchunk:
        (n, wa), (k, wb) = _chunked_dims(a_t, a_fmt, kchunk), _chunked_dims(b_t, b_fmt, kchunk)
    else:
        (n, wa), (k, wb) = a_t.shape, b_t.shape
    if wa != W or wb != W:
        raise ValueError(f"transposed operands must have padded width {W}")
    if kstep:
        for sc, r, what in ((a_t_unit, n, "a_t_unit"), (b_t_unit, k, "b_t_unit")):
            if tuple(sc.shape) != _scale_shape(r, W, kchunk, G) or not sc.is_contiguous():
                raise ValueError(f"{what} must be the K-step-major scale array of its operand")
    elif tuple(a_t_unit.shape) != (n, W // BLOCK) or tuple(b_t_unit.shape) != (k, W // BLOCK):
        raise ValueError("scale shapes must be [rows, W/32]")
    shape = (n, k) if group_lens is None else (G, n, k)
    flags = _gflag(kchunk)
    if accum_into is not None:
        c = _accum_target(accum_into, shape, kchunk, a_t.device)
        flags |= _lib.GF_ACCUM_F32
    else:
        c = torch.empty(shape, dtype=torch.bfloat16, device=a_t.device)
    with _hooked("grouped_gemm_wgrad", m=total_m, n=n, k=k):
        rc = _lib.load().mxl_grouped_gemm_wgrad_scaled(
            _ptr(a_t), _ptr(a_t_unit), a_fmt, _ptr(b_t), _ptr(b_t_unit), b_fmt, _ptr(c), _ptr(group_lens), G, total_m, n, k,
            _ptr(a_scale_inv), _ptr(b_scale_inv), flags, _stream(),
        )
    _lib.check(rc, "mxl_grouped_gemm_wgrad_scaled")
    return c


# --------------------------------------------------------------------------
# RMSNorm in front of the column-parallel linear (rmsnorm(x, weight, eps),
# primus_turbo.py:1689-1700)
# --------------------------------------------------------------------------
RMSNORM_MAX_K = 16384


def _norm_args(x, weight):
    if x.dim() != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("expected a contiguous 2-D bfloat16 tensor [tokens, K]")
    k = x.shape[1]
    if k % 8 != 0 or k > RMSNORM_MAX_K:
        raise ValueError(f"the normalised dim ({k}) must be a multiple of 8 and at most {RMSNORM_MAX_K}")
    if weight.dtype != torch.bfloat16 or tuple(weight.shape) != (k,) or not weight.is_contiguous():
        raise ValueError("the norm weight must be a contiguous bfloat16 vector [K]")
    _require_cuda(x, weight)


def rmsnorm_fwd_impl(x, weight, eps: float, want_y: bool = True):
    """``(y, rstd)``: ``y = (x * rstd) * weight`` in fp32 rounded once to bf16 (``None`` if not wanted),
    ``rstd = 1 / sqrt(mean(x^2) + eps)`` per row in fp32."""
    _norm_args(x, weight)
    rows, k = x.shape
    y = torch.empty_like(x) if want_y else None
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    with _hooked("rmsnorm_fwd", rows=rows, k=k, want_y=want_y):
        rc = _lib.load().mxl_rmsnorm_fwd(_ptr(x), _ptr(weight), float(eps), rows, k, _ptr(y), _ptr(rstd), _stream())
    _lib.check(rc, "mxl_rmsnorm_fwd")
    return y, rstd


def rmsnorm_bwd_impl(dy, x, weight, rstd):
    """``(dx [tokens, K] bf16, dweight [K] bf16)``."""
    _norm_args(x, weight)
    rows, k = x.shape
    if dy.dtype != torch.bfloat16 or tuple(dy.shape) != (rows, k) or not dy.is_contiguous():
        raise ValueError("dy must be a contiguous bfloat16 tensor of the shape of x")
    if rstd.dtype != torch.float32 or tuple(rstd.shape) != (rows,):
        raise ValueError("rstd must be float32 [tokens]")
    _require_cuda(dy, rstd)
    lib = _lib.load()
    dx = torch.empty_like(x)
    dw = torch.empty_like(weight)
    ws = torch.empty((max(int(lib.mxl_rmsnorm_bwd_workspace_bytes(rows, k)), 16) // 4,), dtype=torch.float32, device=x.device)
    with _hooked("rmsnorm_bwd", rows=rows, k=k):
        rc = lib.mxl_rmsnorm_bwd(_ptr(dy), _ptr(x), _ptr(weight), _ptr(rstd), rows, k, _ptr(dx), _ptr(dw), _ptr(ws),
                                 ws.numel() * 4, _stream())
    _lib.check(rc, "mxl_rmsnorm_bwd")
    return dx, dw


def rmsnorm_quantize_impl(x, weight, rstd, fmt: int, scale_mode: int = _lib.SCALE_OCP_FLOOR, *, colwise: bool = False,
                          pad_to: int = 1, kchunk=False):
    """``quantize_mx_impl(rmsnorm_fwd_impl(x, weight, eps)[0])`` in one pass over ``x`` given ``rstd``, the
    normalised tensor never reaching memory; same return tuple (the row-wise copy is always produced)."""
    _norm_args(x, weight)
    rows, k = x.shape
    if k % BLOCK != 0:
        raise ValueError(f"the quantised dim ({k}) must be a multiple of {BLOCK}")
    if rstd.dtype != torch.float32 or tuple(rstd.shape) != (rows,):
        raise ValueError("rstd must be float32 [tokens]")
    _require_cuda(rstd)
    if rows == 0:
        return quantize_mx_impl(x, fmt, scale_mode, rowwise=True, colwise=colwise, pad_to=pad_to, kchunk=kchunk)
    per = _per_byte(fmt)
    dev = x.device
    row_ld = _round_up(k, KCHUNK if kchunk else pad_to)
    q_row = torch.empty(_code_shape(rows, row_ld, per, kchunk), dtype=torch.uint8, device=dev)
    s_row = torch.empty(_scale_shape(rows, row_ld, kchunk), dtype=torch.uint8, device=dev)
    q_col = s_col = None
    if colwise:
        W = padded_width(rows, 0)
        q_col = torch.empty(_code_shape(k, W, per, kchunk), dtype=torch.uint8, device=dev)
        s_col = torch.empty(_scale_shape(k, W, kchunk), dtype=torch.uint8, device=dev)
    with _hooked("rmsnorm_quantize", rows=rows, cols=k, fmt=fmt, rowwise=True, colwise=colwise):
        rc = _lib.load().mxl_rmsnorm_quantize(
            _ptr(x), _ptr(weight), _ptr(rstd), rows, k, row_ld, fmt, scale_mode, None, 0, _ptr(q_row), _ptr(s_row),
            _ptr(q_col), _ptr(s_col), _qflag(kchunk), _stream(),
        )
    _lib.check(rc, "mxl_rmsnorm_quantize")
    cd = _code_dtype(fmt)
    v = lambda t, d: None if t is None else t.view(d)  # noqa: E731
    return v(q_row, cd), v(s_row, float8_e8m0), v(q_col, cd), v(s_col, float8_e8m0)


# --------------------------------------------------------------------------
# reference-named low-level entry points (MX granularity only)
# --------------------------------------------------------------------------
# --------------------------------------------------------------------------
# expert groups padded to the quantisation alignment
# --------------------------------------------------------------------------
def padded_rows_bound(rows: int, groups: int, align: int) -> int:
    """Rows of the buffer ``pad_groups_impl`` fills: the largest total the counts can produce."""
    return (rows + groups * (align - 1)) // align * align


def _pad_args(x, group_lens, align):
    _require_cuda(x, group_lens)
    if x.dim() < 1 or not x.is_contiguous():
        raise ValueError("x must be a contiguous tensor with the rows of the groups along dim 0")
    if int(align) < 1:
        raise ValueError("align must be positive")
    groups = _check_group_lens(group_lens, x.device)
    if groups > 1024:
        raise ValueError("at most 1024 groups")
    row_bytes = x.element_size()
    for d in x.shape[1:]:
        row_bytes *= int(d)
    if row_bytes < 1:
        raise ValueError("rows must not be empty")
    return groups, row_bytes


def pad_groups_impl(x, group_lens, align: int):
    """``(padded, padded_lens)``: each group's rows of ``x`` followed by zero rows up to a multiple of ``align``
    (experts.py:196-209 without the host read of the counts).  ``padded`` has ``padded_rows_bound`` rows; the zero
    rows behind the last group's padding are counted into ``padded_lens[-1]``."""
    groups, row_bytes = _pad_args(x, group_lens, align)
    rows = x.shape[0]
    out_rows = padded_rows_bound(rows, groups, int(align))
    out = torch.empty((out_rows,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
    padded_lens = torch.empty_like(group_lens)
    with _hooked("pad_groups", rows=rows, out_rows=out_rows, row_bytes=row_bytes):
        rc = _lib.load().mxl_pad_groups(_ptr(x), rows, row_bytes, _ptr(group_lens), groups, int(align), _ptr(out),
                                        out_rows, _ptr(padded_lens), _stream())
    _lib.check(rc, "mxl_pad_groups")
    return out, padded_lens


def unpad_groups_impl(y, group_lens, align: int, rows: int):
    """Inverse of ``pad_groups_impl`` (experts.py:262-264): ``[rows, ...]`` from the padded ``y``."""
    groups, row_bytes = _pad_args(y, group_lens, align)
    out = torch.empty((int(rows),) + tuple(y.shape[1:]), dtype=y.dtype, device=y.device)
    with _hooked("unpad_groups", rows=int(rows), padded_rows=y.shape[0], row_bytes=row_bytes):
        rc = _lib.load().mxl_unpad_groups(_ptr(y), y.shape[0], row_bytes, _ptr(group_lens), groups, int(align),
                                          _ptr(out), int(rows), _stream())
    _lib.check(rc, "mxl_unpad_groups")
    return out


# --------------------------------------------------------------------------
# the 128-blockwise FP8 recipe
# --------------------------------------------------------------------------
BW_BLOCK = 128


def _bw_check(x, fmt, what):
    _require_cuda(x)
    if x.dim() != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError(f"{what} must be a contiguous 2-D bfloat16 tensor")
    if fmt not in (_lib.FMT_E4M3, _lib.FMT_E5M2):
        raise ValueError("blockwise scaling is defined for the FP8 formats E4M3 and E5M2")
    if x.shape[1] % BW_BLOCK != 0:
        raise ValueError(f"the blockwise recipe needs the last dimension to be a multiple of {BW_BLOCK} (got {x.shape[1]})")


def quantize_blockwise_impl(x, fmt: int, *, rowwise: bool = True, colwise: bool = False,
                            group_lens: Optional[torch.Tensor] = None):
    """``quant_fp8_blockwise_impl`` for both axes in one launch (primus_turbo_float8_local.py:1019, :1053-1059):
    ``(codes [rows, cols], scale_inv f32 [rows, cols / 128], codes_T [cols, W], scale_inv_T f32 [cols, W / 128])``;
    the row-wise copy has 1 x 128 blocks along the columns, the transposed one 128 x 1 blocks along the rows.
    Without ``group_lens`` W is rows rounded up to 128 (zero codes); with it the rows are split into groups and the
    transposed copy is segment-padded, ``W = padded_width(rows, G)``, blocks restarting at every group
    (``quant_fp8_blockwise_segment_m_row_col_impl``, zbpp_gemm.py:633, :785).  Copies not asked for are None."""
    _bw_check(x, fmt, "x")
    if not (rowwise or colwise):
        raise ValueError("at least one copy must be requested")
    rows, cols = x.shape
    G = _check_group_lens(group_lens, x.device) if colwise else 0
    W = padded_width(rows, G) if G else _round_up(rows, BW_BLOCK)
    dt = _code_dtype(fmt) if fmt != _lib.FMT_E5M2 else torch.float8_e5m2
    q = s = qt = st = None
    if rowwise:
        q = torch.empty((rows, cols), dtype=torch.uint8, device=x.device)
        s = torch.empty((rows, cols // BW_BLOCK), dtype=torch.float32, device=x.device)
    if colwise:
        qt = torch.empty((cols, W), dtype=torch.uint8, device=x.device)
        st = torch.empty((cols, W // BW_BLOCK), dtype=torch.float32, device=x.device)
    with _hooked("quantize_blockwise", rows=rows, cols=cols, fmt=fmt, rowwise=rowwise, colwise=colwise):
        rc = _lib.load().mxl_quantize_blockwise(_ptr(x), rows, cols, fmt, _ptr(group_lens) if G else None, G, _ptr(q), _ptr(s),
                                                _ptr(qt), _ptr(st), _stream())
    _lib.check(rc, "mxl_quantize_blockwise")
    return (q.view(dt) if q is not None else None), s, (qt.view(dt) if qt is not None else None), st


def quantize_blockwise_weight_impl(w, fmt: int, *, rowwise: bool = True, colwise: bool = False):
    """``quant_fp8_blockwise_for_weight_impl`` (primus_turbo_float8_local.py:1020, :1060): one scale per 128 x 128
    block of ``w [n, k]`` or of every matrix of ``w [G, n, k]``.  ``(codes [.., n, k], scale_inv f32 [.., n / 128,
    k / 128], codes_T [.., k, n], scale_inv_T)``."""
    if w.dim() == 3:
        _bw_check(w[0] if w.shape[0] else w.reshape(-1, w.shape[-1]), fmt, "w")
        if not w.is_contiguous():
            raise ValueError("w must be contiguous")
    else:
        _bw_check(w, fmt, "w")
    lead = tuple(w.shape[:-2])
    batch = lead[0] if lead else 1
    n, k = w.shape[-2], w.shape[-1]
    if n % BW_BLOCK != 0:
        raise ValueError(f"the blockwise recipe needs weight dimensions that are multiples of {BW_BLOCK} (got {n})")
    if not (rowwise or colwise):
        raise ValueError("at least one copy must be requested")
    dt = _code_dtype(fmt) if fmt != _lib.FMT_E5M2 else torch.float8_e5m2
    q = s = qt = st = None
    if rowwise:
        q = torch.empty(lead + (n, k), dtype=torch.uint8, device=w.device)
        s = torch.empty(lead + (n // BW_BLOCK, k // BW_BLOCK), dtype=torch.float32, device=w.device)
    if colwise:
        qt = torch.empty(lead + (k, n), dtype=torch.uint8, device=w.device)
        st = torch.empty(lead + (k // BW_BLOCK, n // BW_BLOCK), dtype=torch.float32, device=w.device)
    if batch:
        with _hooked("quantize_blockwise_weight", rows=batch * n, cols=k, fmt=fmt, rowwise=rowwise, colwise=colwise):
            rc = _lib.load().mxl_quantize_blockwise_weight(_ptr(w), batch, n, k, fmt, _ptr(q), _ptr(s), _ptr(qt), _ptr(st), _stream())
        _lib.check(rc, "mxl_quantize_blockwise_weight")
    return (q.view(dt) if q is not None else None), s, (qt.view(dt) if qt is not None else None), st


def _fp8_fmt_of(codes: torch.Tensor) -> int:
    if codes.dtype == torch.float8_e5m2:
        return _lib.FMT_E5M2
    if codes.dtype in (torch.float8_e4m3fn, torch.uint8):
        return _lib.FMT_E4M3
    raise ValueError(f"not an FP8 code tensor: {codes.dtype}")


def _bw_scales(t, shape, what):
    if t.dtype != torch.float32 or tuple(t.shape) != tuple(shape) or not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous float32 {tuple(shape)}")


def set_blockwise_gemm_tile(rows: int) -> None:
    """Output-tile height of the blockwise GEMMs for every later call: 128 or 256 rows, 0 = chosen by the shape (the
    default).  Both give the same bits; a measuring and testing aid (``mxl_blockwise_gemm_tile``)."""
    _lib.check(_lib.load().mxl_blockwise_gemm_tile(int(rows)), "mxl_blockwise_gemm_tile")


def gemm_blockwise_nt_impl(a, a_scale_inv, b, b_scale_inv, group_lens: Optional[torch.Tensor] = None,
                           b_rows_per_scale: Optional[int] = None) -> torch.Tensor:
    """``gemm_fp8_impl`` / ``grouped_gemm_fp8_impl`` with ``granularity=BLOCKWISE`` in NT form
    (primus_turbo_float8_local.py:1022-1033, zbpp_gemm.py:608-630):
    ``c[m, n] = sum_kb a_scale_inv[m, kb] * b_scale_inv[n or n / 128, kb] * (a[m, kb] . b[n, kb])``, bf16.
    Dense: ``b [n, k]``, ``b_scale_inv`` with one row per row of ``b`` (an activation copy) or one per 128 rows (a
    weight).  Grouped: the rows of ``a`` are split by ``group_lens``, ``b [G, n, k]``, ``b_scale_inv [G, n / 128, k / 128]``.
    ``b_rows_per_scale`` (dense): 1 or 128, which of the two forms ``b_scale_inv`` has; None reads it off its shape."""
    _require_cuda(a, a_scale_inv, b, b_scale_inv, group_lens)
    G = _check_group_lens(group_lens, a.device)
    m, k = a.shape
    n = b.shape[-2]
    if b.shape[-1] != k or k % BW_BLOCK != 0 or n % BW_BLOCK != 0 or k == 0:
        raise ValueError("blockwise GEMM: contraction lengths must agree and k, n must be multiples of 128")
    if not (a.is_contiguous() and b.is_contiguous()):
        raise ValueError("code tensors must be contiguous")
    kb = k // BW_BLOCK
    _bw_scales(a_scale_inv, (m, kb), "a_scale_inv")
    c = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    lib = _lib.load()
    if G:
        if b.dim() != 3 or b.shape[0] != G:
            raise ValueError("grouped blockwise GEMM expects weights of shape [num_groups, n, k]")
        _bw_scales(b_scale_inv, (G, n // BW_BLOCK, kb), "b_scale_inv")
        with _hooked("grouped_gemm_blockwise_nt", m=m, n=n, k=k):
            rc = lib.mxl_grouped_gemm_nt_blockwise(_ptr(a), _ptr(a_scale_inv), _fp8_fmt_of(a), _ptr(b), _ptr(b_scale_inv),
                                                   _fp8_fmt_of(b), _ptr(c), _ptr(group_lens), G, m, n, k, _stream())
        _lib.check(rc, "mxl_grouped_gemm_nt_blockwise")
        return c
    if b.dim() != 2:
        raise ValueError("dense blockwise GEMM expects b [n, k]")
    if b_scale_inv.dtype != torch.float32 or not b_scale_inv.is_contiguous() or tuple(b_scale_inv.shape) not in ((n, kb), (n // BW_BLOCK, kb)):
        raise ValueError("b_scale_inv must be contiguous float32 [n, k / 128] or [n / 128, k / 128]")
    per = (1 if b_scale_inv.shape[0] == n else BW_BLOCK) if b_rows_per_scale is None else int(b_rows_per_scale)
    if per not in (1, BW_BLOCK) or b_scale_inv.shape[0] != n // per:
        raise ValueError("b_rows_per_scale must be 1 or 128 and match the rows of b_scale_inv")
    with _hooked("gemm_blockwise_nt", m=m, n=n, k=k):
        rc = lib.mxl_gemm_nt_blockwise(_ptr(a), _ptr(a_scale_inv), _fp8_fmt_of(a), _ptr(b), _ptr(b_scale_inv),
                                       _fp8_fmt_of(b), per, _ptr(c), m, n, k, _stream())
    _lib.check(rc, "mxl_gemm_nt_blockwise")
    return c


def grouped_gemm_blockwise_wgrad_impl(a_t, a_t_scale_inv, b_t, b_t_scale_inv, group_lens, total_m: int) -> torch.Tensor:
    """``grouped_gemm_fp8_variable_k_impl`` with blockwise granularity (zbpp_gemm.py:757-800) on the segment-padded
    transposed copies: ``a_t = q_colT(dY) [n, W]``, ``b_t = q_colT(X) [k, W]`` with their ``[rows, W / 128]`` factors;
    ``c [G, n, k]``, zeros for a group without tokens."""
    _require_cuda(a_t, a_t_scale_inv, b_t, b_t_scale_inv, group_lens)
    G = _check_group_lens(group_lens, a_t.device)
    if not G:
        raise ValueError("group_lens is required")
    W = padded_width(int(total_m), G)
    n, k = a_t.shape[0], b_t.shape[0]
    if a_t.shape[1] != W or b_t.shape[1] != W or n % BW_BLOCK or k % BW_BLOCK or not (a_t.is_contiguous() and b_t.is_contiguous()):
        raise ValueError(f"transposed operands must be contiguous [rows, {W}] with rows a multiple of 128")
    _bw_scales(a_t_scale_inv, (n, W // BW_BLOCK), "a_t_scale_inv")
    _bw_scales(b_t_scale_inv, (k, W // BW_BLOCK), "b_t_scale_inv")
    c = torch.empty((G, n, k), dtype=torch.bfloat16, device=a_t.device)
    with _hooked("grouped_gemm_blockwise_wgrad", m=int(total_m), n=n, k=k):
        rc = _lib.load().mxl_grouped_gemm_wgrad_blockwise(_ptr(a_t), _ptr(a_t_scale_inv), _fp8_fmt_of(a_t), _ptr(b_t),
                                                          _ptr(b_t_scale_inv), _fp8_fmt_of(b_t), _ptr(c), _ptr(group_lens), G,
                                                          int(total_m), n, k, _stream())
    _lib.check(rc, "mxl_grouped_gemm_wgrad_blockwise")
    return c


def _require_mx(granularity) -> None:
    val = getattr(granularity, "value", granularity)
    if val != ScalingGranularity.MX_BLOCKWISE.value:
        raise NotImplementedError("only ScalingGranularity.MX_BLOCKWISE has kernels in this build")


def gemm_fp8_impl(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity=None, default_backend=None):
    """gemm_fp8_impl of the reference (primus_turbo_float8_local.py:239-250)
    for MX operands: only the NT form (trans_a=False, trans_b=True,
    trans_c=False) exists because MX operands are quantised along K."""
    _require_mx(granularity)
    if trans_a or not trans_b or trans_c:
        raise ValueError("MX GEMM supports the NT layout only (trans_a=False, trans_b=True, trans_c=False)")
    return gemm_mx_nt_impl(a, a_scale_inv, b, b_scale_inv, out_dtype)


# --------------------------------------------------------------------------
# pre-shuffled MXFP4 layouts (the shuffle_* flags of quantize_mxfp4_dual,
# primus_turbo_mxfp4_local.py:147-161, :184-198)
# --------------------------------------------------------------------------
def shuffled_scale_shape(rows: int, blocks: int) -> Tuple[int, int]:
    """Shape of a pre-shuffled scale array: rows to 256, blocks to 8 (primus_turbo_mxfp4_local.py:184-187)."""
    return _round_up(rows, 256), _round_up(blocks, 8)


def shuffle_codes_impl(codes: torch.Tensor, inverse: bool = False) -> torch.Tensor:
    """Packed FP4 codes ``[rows, row_bytes]`` in the pre-shuffled byte order (16 x 32-byte blocks made contiguous), or
    back with ``inverse=True``.  Same shape and dtype; rows must be a multiple of 16, row bytes of 32."""
    _require_cuda(codes)
    if codes.dim() != 2:
        raise ValueError("expected 2-D codes [rows, row_bytes]")
    u8 = _codes_u8(codes)
    rows, rb = u8.shape
    if rows % 16 or rb % 32:
        raise ValueError(f"the pre-shuffled code layout needs rows % 16 == 0 and row bytes % 32 == 0 (got {rows} x {rb})")
    out = torch.empty_like(u8)
    rc = _lib.load().mxl_shuffle_codes(_ptr(u8), rows, rb, _ptr(out), int(bool(inverse)), _stream())
    _lib.check(rc, "mxl_shuffle_codes")
    return out.view(codes.dtype)


def shuffle_scales_impl(scales: torch.Tensor) -> torch.Tensor:
    """E8M0 scales ``[rows, blocks]`` -> pre-shuffled ``[ceil(rows/256)*256, ceil(blocks/8)*8]`` (zero bytes in the
    padding)."""
    _require_cuda(scales)
    if scales.dim() != 2:
        raise ValueError("expected 2-D scales [rows, blocks]")
    u8 = scales.view(torch.uint8)
    rows, blocks = u8.shape
    out = torch.empty(shuffled_scale_shape(rows, blocks), dtype=torch.uint8, device=scales.device)
    rc = _lib.load().mxl_shuffle_scales(_ptr(u8), rows, blocks, _ptr(out), 0, _stream())
    _lib.check(rc, "mxl_shuffle_scales")
    return out.view(scales.dtype)


def unshuffle_scales_impl(shuffled: torch.Tensor, rows: int, blocks: int) -> torch.Tensor:
    """The inverse of ``shuffle_scales_impl`` for an operand of ``rows`` rows and ``blocks`` blocks a row."""
    _require_cuda(shuffled)
    if tuple(shuffled.shape) != shuffled_scale_shape(rows, blocks):
        raise ValueError(f"pre-shuffled scales of a [{rows}, {blocks}] operand must be {shuffled_scale_shape(rows, blocks)}")
    u8 = shuffled.view(torch.uint8)
    out = torch.empty((rows, blocks), dtype=torch.uint8, device=shuffled.device)
    rc = _lib.load().mxl_shuffle_scales(_ptr(u8), rows, blocks, _ptr(out), 1, _stream())
    _lib.check(rc, "mxl_shuffle_scales")
    return out.view(shuffled.dtype)


def gemm_fp4_impl(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity=None, default_backend=None, preshuffled=False):
    """gemm_fp4_impl of the reference (primus_turbo_mxfp4_local.py:319-331).  ``preshuffled``: the operands are
    what the reference's MXFP4 linear hands over with its pre-shuffle switch on (:234-288): ``a`` plain codes with
    pre-shuffled scales, ``b`` pre-shuffled codes and scales.  The GEMM reads the pre-shuffled codes of ``b`` as they
    lie; the two scale arrays (1/16 of the bytes of the codes) are converted back to the plain order first."""
    if preshuffled:
        _require_mx(granularity)
        if trans_a or not trans_b or trans_c:
            raise ValueError("MX GEMM supports the NT layout only (trans_a=False, trans_b=True, trans_c=False)")
        k = a.shape[-1] * _per_byte(fmt_of(a))
        a_scale_inv = unshuffle_scales_impl(a_scale_inv, a.shape[0], k // BLOCK)
        b_scale_inv = unshuffle_scales_impl(b_scale_inv, b.shape[0], b.shape[-1] * _per_byte(fmt_of(b)) // BLOCK)
        if fmt_of(a) == _lib.FMT_E2M1 and fmt_of(b) == _lib.FMT_E2M1 and k % GEMM_K_ALIGN == 0 and b.shape[0] % 16 == 0:
            # the GEMM fetches every 16-byte piece of b from its pre-shuffled place: the codes are not rearranged
            return gemm_mx_nt_impl(a, a_scale_inv, b, b_scale_inv, out_dtype, b_shuffled=True)
        b = shuffle_codes_impl(b, inverse=True)     # (a contraction length the GEMM has to pad: plain codes first)
    return gemm_fp8_impl(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity, default_backend)


def grouped_gemm_fp8_impl(a, b, a_scale_inv, b_scale_inv, group_lens, group_offs, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, granularity=None, num_cu=None, default_backend=None):
    """grouped_gemm_fp8_impl of the reference (zbpp_gemm.py:590-603);
    ``group_offs`` and ``num_cu`` are accepted and unused (the tile schedule
    is derived from ``group_lens`` on the device)."""
    _require_mx(granularity)
    if trans_a or not trans_b:
        raise ValueError("MX grouped GEMM supports the NT layout only (trans_a=False, trans_b=True)")
    return grouped_gemm_mx_nt_impl(a, a_scale_inv, b, b_scale_inv, group_lens, out_dtype)


def grouped_gemm_fp8_variable_k_impl(a, b, a_scale_inv, b_scale_inv, group_lens, group_offs, trans_a=True, trans_b=False, trans_c=True, out_dtype=torch.bfloat16, granularity=None, num_cu=None, default_backend=None, total_m=None):
    """grouped_gemm_fp8_variable_k_impl of the reference (zbpp_gemm.py:710-724):
    ``a`` = X col-wise copy ``[k, W]``, ``b`` = dY col-wise copy ``[n, W]``
    (both transposed, segment-padded); with ``trans_c=True`` (weights stored
    ``[n, k]``, i.e. trans_b=True in the forward) returns ``[G, n, k]``.
    ``total_m`` (ours, optional) is the token count; without it the padded width is taken from the operands."""
    _require_mx(granularity)
    if not trans_a or trans_b:
        raise ValueError("variable-K grouped GEMM expects trans_a=True, trans_b=False")
    if total_m is None:
        # The reference's call (13 arguments) does not carry the token count.  The kernels need it only for the
        # padded width of the transposed operands, which the operand states itself: any count with that padded
        # width describes the same buffers (the groups come from group_lens, on the device).
        G = _check_group_lens(group_lens, a.device)
        per = _per_byte(fmt_of(a))
        width = a.shape[0] * a.shape[2] * per if a.dim() == 3 else a.shape[-1] * per
        total_m = max(width - (_lib.SEG_ALIGN - 1) * max(G, 1), 0)
        if padded_width(total_m, G) != width:
            raise ValueError(f"the operands' last dim ({width}) is not a padded width for {G} groups")
    if trans_c:
        return grouped_gemm_mx_wgrad_impl(b, b_scale_inv, a, a_scale_inv, group_lens, total_m, out_dtype)
    return grouped_gemm_mx_wgrad_impl(a, a_scale_inv, b, b_scale_inv, group_lens, total_m, out_dtype)
