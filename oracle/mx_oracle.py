"""CPU oracle for the MX (microscaling) low-precision linear path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``primus_amd/`` may import this file;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and only as the checker.

What it restates
----------------
The arithmetic of this path lives in the third-party package ``primus_turbo``
(AMD-AGI/Primus-Turbo, pinned at commit 22e544d56820674fcc4c8faf64651af99a5cd686
by /root/reference/.github/workflows/ci.yaml:43), which is not vendored in the
reference tree.  The oracle therefore restates the published OCP Microscaling
Formats (MX) v1.0 algorithm, anchored on the reference's call sites:

* block size 32, E8M0 scales, E4M3 / E2M1 elements:
  primus/backends/megatron/core/fp8_utils.py:162-168,
  primus/backends/megatron/core/fp4_utils.py:144-150
* row-wise copy = ``axis=-1``; column-wise copy = ``axis=-2`` which yields the
  TRANSPOSED quantised tensor:
  primus/backends/megatron/core/extensions/primus_turbo.py:321-354
* weights use 2-D 32x32 blocks, experts are independent matrices:
  primus/backends/megatron/core/extensions/primus_turbo.py:313-317,
  primus/backends/megatron/core/optimizer/weight_deosc.py:29-33,136-174
* every GEMM is NT with both operands quantised along the contraction dim
  (fwd / dgrad / wgrad operand table):
  primus/backends/megatron/core/extensions/primus_turbo_mxfp4_local.py:316-331,
  :432-444, :447-459
* grouped GEMM takes tokens-per-expert (``group_lens``), empty experts allowed:
  primus/backends/megatron/core/extensions/primus_turbo.py:2122-2129

Parity status
-------------
* ``cast_e4m3`` : pinned against ``torch.float8_e4m3fn`` (library routine) and
  brute-force nearest-value search.
* ``cast_e2m1`` : pinned by brute-force nearest-value search over the 8-entry
  E2M1 table (ties to even code).
* ``e8m0_scale_byte`` : pinned against the closed forms of the three published
  scale rules in exact rational arithmetic, for every non-negative bf16 amax.
* which of the three scale rules the shipped Primus-Turbo quantiser uses, its
  ``amax == 0`` byte, its NaN/Inf handling and the FP4 nibble order are
  **parity unpinned** (the package is absent); the rule is an explicit
  ``scale_mode`` argument everywhere, default ``OCP_FLOOR``.
* GEMM / grouped GEMM / wgrad: dequantise -> fp32 matmul -> bf16, pinned by
  invariants (G=1 == dense, permutation of experts, exactly representable
  integer products) in tests/.

* ``glu_with_probs_ref`` / ``glu_with_probs_bwd_ref`` (gated activation times
  router probability with a row mask; call site primus_turbo.py:1954-1980,
  unfused arithmetic experts.py:100-118): float64 closed forms, pinned against
  torch's float64 ``silu`` / ``gelu`` and autograd (library routines) and by
  the identities act(x) - act(-x) = x.  Whether the Primus-Turbo kernels round
  once (as here, like Megatron's fused weighted SwiGLU) or after every step,
  and which GELU flavour ``geglu_with_probs`` uses, is **parity unpinned**.

* ``cast_e2m1_sr`` / ``quantize_mx_rowwise_sr`` / ``quantize_mx_colwise_segmented_sr``
  (stochastic rounding of MXFP4 gradients, rowwise_use_sr / colwise_use_sr at
  primus_turbo_mxfp4_local.py:272-288): written as a search in the E2M1 value
  table; pinned by enumeration of all 2^16 random values per input (result is
  one of the two neighbours, the upper one for exactly ceil(frac * 2^16) of
  them, so the mean is within 2^-16 of a grid step of the input; grid points
  never move; saturation at 6) and by uniformity checks of the counter hash.
  Primus-Turbo's random stream cannot be reproduced (package absent, and a
  different generator by construction): which elements round up is **parity
  unpinned**; only the distribution is comparable.

* ``hadamard16_rows`` (the transposed copies' random Hadamard transform,
  colwise_use_rht at primus_turbo_mxfp4_local.py:234-250,272-288): pinned
  against ``scipy.linalg.hadamard(16)`` in float64 (library routine; the
  float32 butterflies agree with it to rounding and exactly on small integers),
  by orthogonality (transforming twice with zero signs returns the input, the
  inner product of two transformed columns equals the untransformed one) and by
  the sign-vector definition.  The reference states neither the transform size
  nor the sign vector (they live in Primus-Turbo's C++ op): **parity unpinned**.

* ``rmsnorm_rstd`` / ``rmsnorm_ref`` / ``rmsnorm_bwd_ref`` (RMSNorm in front of the
  column-parallel linear, ``rmsnorm(x, layer_norm_weight, eps)`` at
  primus_turbo.py:1689-1700): y = (x * rstd) * w in float32 with one rounding, the
  sum of squares in the fixed order the HIP kernel documents (so rstd and y are
  reproduced bit for bit); pinned against float64 closed forms, against torch's
  ``rms_norm`` (library routine, to one bf16 ulp) and its autograd, and by the
  invariants rms(y / w) = 1 and scale invariance of y in x.  Whether Primus-Turbo's
  kernel rounds once or after the normalisation and again after the weight
  (as torch's composite does) is **parity unpinned** (package absent).

* ``cast_e5m2`` / ``quantize_tensorwise`` / ``tensorwise_gemm_nt_ref`` (tensor-wise "current" FP8
  scaling, the non-MX recipe behind the same operators; restated in the reference itself at
  primus_turbo_float8_local.py:194-207 and :215-306): scale = fp8_max / max(amax, 1e-12) and
  scale_inv = 1 / scale in float32, q = cast(clamp(x * scale)).  ``cast_e5m2`` is pinned against
  ``torch.float8_e5m2`` (library routine) over every bf16 value and over float32 samples next to the
  rounding boundaries; the quantiser against the reference's formula evaluated with torch ops.  The
  reference's experimental "decomposed" variant multiplies in bf16 and its shipping variant calls a
  Primus-Turbo C++ op whose source is absent: the float32 product used here is **parity unpinned**
  against that op.

* ``pad_groups`` / ``unpad_groups`` (expert groups padded with zero rows to the quantisation alignment,
  experts.py:196-209 and :262-264; alignment from primus_turbo.py:2344-2353): index work, written with numpy
  slices per group; pinned in tests/ against the reference's own sequence (split per expert, append zero rows,
  concatenate) written as a row-by-row Python loop, and by unpad(pad(x)) == x.  The rows behind the last group's
  padding in a buffer sized for the worst case (zero rows counted into the last group) have no counterpart in
  the reference, whose buffer has the exact size because it reads the counts on the host.

* ``quantize_blockwise`` / ``quantize_blockwise_2d`` / ``blockwise_gemm_nt_ref`` (the 128-blockwise FP8 recipe:
  operand flow at primus_turbo_float8_local.py:1019-1087, admitted by rocm_arg_validation.py:145): per block the
  formula the reference restates for its tensor-wise quantiser (:194-207), scale = fp8_max / max(amax, 1e-12),
  codes = cast(clamp(x * scale)), scale_inv = 1 / scale in float32; the GEMM adds the K blocks' float32 partial
  products times both blocks' scale_inv.  Pinned in tests/ against the same formula evaluated with torch ops on
  reshaped blocks and torch's float8 casts (library routines), by "one block == the tensor-wise quantiser", block
  independence and the dequantisation error bound; the GEMM against float64 arithmetic on the decoded operands.
  The Primus-Turbo ops behind ``quant_fp8_blockwise_impl`` are absent: whether they use this formula or another
  (e.g. amax / fp8_max without the clamp at 1e-12) is **parity unpinned**.

* ``shuffle_codes_16x16`` / ``shuffle_e8m0`` and their inverses (the "pre-shuffled" MXFP4 layouts, the
  ``shuffle_*`` flags of ``quantize_mxfp4_dual`` and ``gemm_fp4_impl(preshuffled=True)``,
  primus_turbo_mxfp4_local.py:147-161, :184-198, :319-331; the reference calls it the AITER preshuffle fast
  path, :39-99): pure byte permutations.  The permutation itself lives in the third-party AITER package
  (ROCm/aiter; no version is pinned in the reference tree: it comes in through Primus-Turbo), which is absent:
  restated here from its published ``shuffle_weight(x, layout=(16, 16))`` (16 rows x 32 bytes blocks, stored as
  two halves of 16 rows x 16 bytes) and ``e8m0_shuffle`` (scales padded to 256 x 8, then
  ``view(m/32, 2, 16, n/8, 2, 4).permute(0, 3, 5, 2, 4, 1)``).  Written below as explicit index arithmetic;
  pinned in tests/ against the view / permute formulation evaluated by torch (a library routine doing the
  permutation another way), by inverse(shuffle(x)) == x and by the scale shapes the reference's own shape
  function states for the shuffled outputs (:184-187, :192-195: rows to 256, blocks to 8).  Whether Primus-Turbo's
  C++ op writes exactly these byte orders is **parity unpinned**.

All scale arithmetic is integer arithmetic on fp32 bit patterns (no log2), so
results are reproducible bit-for-bit on any host.
"""

from __future__ import annotations

import numpy as np

BLOCK = 32

# element formats
FMT_E4M3 = 0
FMT_E2M1 = 1
FMT_E5M2 = 2  # tensor-wise scaled operands only

# E8M0 scale rules
SCALE_OCP_FLOOR = 0  # OCP MX v1.0: floor(log2 amax) - emax_elem
SCALE_RCEIL = 1  # 2^ceil(log2(amax / max_normal))
SCALE_EVEN = 2  # round amax to the element mantissa width first, then floor

# emax of the element format (exponent of its largest normal)
_EMAX = {FMT_E4M3: 8, FMT_E2M1: 2}
# mantissa (fp32 field) of the largest normal: 448 = 1.75*2^8, 6 = 1.5*2^2
_MAXMAN = {FMT_E4M3: 0x600000, FMT_E2M1: 0x400000}
# explicit mantissa bits of the element format
_MBITS = {FMT_E4M3: 3, FMT_E2M1: 1}
_MAXNORM = {FMT_E4M3: 448.0, FMT_E2M1: 6.0}

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


# --------------------------------------------------------------------------
# bf16 <-> fp32 helpers (bf16 carried as uint16 bit patterns)
# --------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """Exact widening of bf16 bit patterns (uint16) to float32."""
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even narrowing of float32 to bf16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    out = (r >> np.uint32(16)).astype(np.uint16)
    out[nan] = ((u[nan] >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
    return out


def to_bf16_bits(x) -> np.ndarray:
    """Accept a torch bf16 tensor, a uint16 array or a float array."""
    try:
        import torch

        if isinstance(x, torch.Tensor):
            if x.dtype != torch.bfloat16:
                x = x.to(torch.bfloat16)
            return x.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)
    except ImportError:  # pragma: no cover
        pass
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return x
    return f32_to_bf16_bits(x.astype(np.float32))


# --------------------------------------------------------------------------
# E8M0 block scale
# --------------------------------------------------------------------------
def e8m0_scale_byte(amax_bits: np.ndarray, fmt: int, scale_mode: int = SCALE_OCP_FLOOR) -> np.ndarray:
    """E8M0 byte for a block whose finite amax has fp32 bit pattern ``amax_bits``.

    byte = clamp(E - emax_elem + bump, 0, 254) where E is the biased fp32
    exponent field of amax (after the EVEN pre-rounding, if selected) and
    bump is 1 only for RCEIL when amax's mantissa exceeds the mantissa of the
    format's largest normal.  amax == 0 gives byte 0.  Non-finite blocks are
    handled by the caller (byte 255).
    """
    b = amax_bits.astype(np.int64)
    if scale_mode == SCALE_EVEN:
        b = b + (1 << (23 - _MBITS[fmt] - 1))
    e = b >> 23
    bump = np.zeros_like(e)
    if scale_mode == SCALE_RCEIL:
        bump = ((b & 0x7FFFFF) > _MAXMAN[fmt]).astype(np.int64)
    byte = np.clip(e - _EMAX[fmt] + bump, 0, 254)
    return byte.astype(np.uint8)


def inv_scale_f32(byte: np.ndarray) -> np.ndarray:
    """2^(127 - byte) as float32 (always a normal number for byte in [0, 253]);
    0.0 for the NaN byte 255 so finite lanes of a non-finite block become +-0."""
    b = byte.astype(np.int64)
    bits = (np.clip(254 - b, 0, 254) << 23).astype(np.uint32)
    out = bits.view(np.float32).copy()
    out[b == 255] = 0.0
    # byte 254 (scale 2^127) is unreachable from bf16 data (largest byte is 253)
    return out


def scale_f32(byte: np.ndarray) -> np.ndarray:
    """2^(byte - 127) as float32 (float64 exponentiation, then exact narrowing);
    NaN for byte 255."""
    b = np.where(byte == 255, 127, byte).astype(np.float64)
    out = np.exp2(b - 127.0).astype(np.float32)
    out[byte == 255] = np.nan
    return out


# --------------------------------------------------------------------------
# element casts (saturating, round-to-nearest-even), integer arithmetic
# --------------------------------------------------------------------------
def cast_e4m3(v: np.ndarray) -> np.ndarray:
    """float32 -> OCP FP8 E4M3 (fn) code, RNE, saturating at +-448, sign kept
    on zero results, NaN -> sign|0x7F, +-Inf saturates like any large value."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    u = v.view(np.uint32)
    sign = ((u >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    a_bits = u & np.uint32(0x7FFFFFFF)
    nan = a_bits > np.uint32(0x7F800000)
    a = np.minimum(a_bits.view(np.float32), np.float32(448.0))
    a = np.where(nan, np.float32(0.0), a).astype(np.float32)
    ab = a.view(np.uint32).astype(np.int64)
    # normal range of e4m3: >= 2^-6
    rounded = (ab + 0x7FFFF + ((ab >> 20) & 1)) >> 20  # (exp32 << 3) | m3 after carry
    code_n = rounded - ((127 - 7) << 3)
    # subnormal range: multiples of 2^-9
    code_s = np.rint(a.astype(np.float64) * 512.0).astype(np.int64)
    code = np.where(a >= np.float32(2.0**-6), code_n, code_s)
    code = np.minimum(code, 0x7E)
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def cast_e2m1(v: np.ndarray) -> np.ndarray:
    """float32 -> FP4 E2M1 code (4 bits: s e e m), RNE (ties to even code),
    saturating at +-6, sign kept on zero results.  NaN saturates to sign|7."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    u = v.view(np.uint32)
    sign = ((u >> np.uint32(28)) & np.uint32(0x8)).astype(np.uint8)
    a_bits = u & np.uint32(0x7FFFFFFF)
    nan = a_bits > np.uint32(0x7F800000)
    a = np.minimum(a_bits.view(np.float32), np.float32(6.0))
    a = np.where(nan, np.float32(6.0), a).astype(np.float32)
    ab = a.view(np.uint32).astype(np.int64)
    rounded = (ab + 0x1FFFFF + ((ab >> 22) & 1)) >> 22  # (exp32 << 1) | m1
    code_n = rounded - ((127 - 1) << 1)
    code_s = np.rint(a.astype(np.float64) * 2.0).astype(np.int64)
    code = np.where(a >= np.float32(1.0), code_n, code_s)
    code = np.minimum(code, 7)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def decode_e4m3(code: np.ndarray) -> np.ndarray:
    c = code.astype(np.int64)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 0x7
    val = np.where(e == 0, m * 2.0**-9, (8 + m) * np.exp2(e.astype(np.float64) - 10.0))
    val = np.where((c & 0x7F) == 0x7F, np.nan, val)
    return (s * val).astype(np.float32)


def decode_e2m1(code: np.ndarray) -> np.ndarray:
    c = code.astype(np.int64)
    s = np.where(c & 0x8, -1.0, 1.0)
    return (s * E2M1_VALUES[c & 0x7]).astype(np.float32)


def pack_fp4(codes: np.ndarray) -> np.ndarray:
    """Pack 4-bit codes along the last axis: element 2i -> bits 3:0, element
    2i+1 -> bits 7:4 (the ``float4_e2m1fn_x2`` convention)."""
    assert codes.shape[-1] % 2 == 0
    lo = codes[..., 0::2] & 0xF
    hi = codes[..., 1::2] & 0xF
    return (lo | (hi << 4)).astype(np.uint8)


def unpack_fp4(packed: np.ndarray) -> np.ndarray:
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0xF
    out[..., 1::2] = packed >> 4
    return out


# --------------------------------------------------------------------------
# MX quantise / dequantise
# --------------------------------------------------------------------------
def _block_scale_bytes(xb_blocks: np.ndarray, fmt: int, scale_mode: int) -> np.ndarray:
    """xb_blocks: uint16 bf16 bits, reduction over the last axis."""
    mag = (xb_blocks & np.uint16(0x7FFF)).astype(np.uint32)
    amax = mag.max(axis=-1)  # bf16 magnitudes order like unsigned ints
    nonfinite = amax >= 0x7F80
    byte = e8m0_scale_byte(amax << np.uint32(16), fmt, scale_mode)
    byte[nonfinite] = 255
    return byte


def _cast_scaled(xb: np.ndarray, byte_per_elem: np.ndarray, fmt: int) -> np.ndarray:
    x = bf16_bits_to_f32(xb)
    inv = inv_scale_f32(byte_per_elem)
    with np.errstate(invalid="ignore", over="ignore"):
        v = (x * inv).astype(np.float32)  # exact: power-of-two factor; inf*0 -> nan
    finite = (xb & np.uint16(0x7FFF)) < np.uint16(0x7F80)
    if fmt == FMT_E4M3:
        code = cast_e4m3(v)
        # non-finite inputs (NaN or Inf) become NaN codes with the input's sign
        sign = ((xb >> np.uint16(8)) & np.uint16(0x80)).astype(np.uint8)
        code = np.where(finite, code, sign | np.uint8(0x7F)).astype(np.uint8)
    else:
        code = cast_e2m1(v)
        sign = ((xb >> np.uint16(12)) & np.uint16(0x8)).astype(np.uint8)
        code = np.where(finite, code, sign | np.uint8(0x7)).astype(np.uint8)
    return code


def quantize_mx_rowwise(x, fmt: int = FMT_E4M3, scale_mode: int = SCALE_OCP_FLOOR):
    """x[..., K] bf16 -> (codes[..., K] (fp8) or [..., K/2] (fp4, packed),
    scales[..., K/32]); blocks of 32 along the last axis (``axis=-1``,
    primus_turbo.py:321-331)."""
    xb = to_bf16_bits(x)
    K = xb.shape[-1]
    assert K % BLOCK == 0, "last dim must be a multiple of 32"
    blocks = xb.reshape(xb.shape[:-1] + (K // BLOCK, BLOCK))
    byte = _block_scale_bytes(blocks, fmt, scale_mode)
    code = _cast_scaled(blocks, np.broadcast_to(byte[..., None], blocks.shape), fmt)
    code = code.reshape(xb.shape)
    if fmt == FMT_E2M1:
        code = pack_fp4(code)
    return code, byte


def quantize_mx_colwise(x, fmt: int = FMT_E4M3, scale_mode: int = SCALE_OCP_FLOOR):
    """``axis=-2`` quantisation: blocks of 32 along the second-to-last axis and
    a TRANSPOSED result (primus_turbo.py:346-354):
    x[..., M, C] -> codes[..., C, M] (or [..., C, M/2]), scales[..., C, M/32].
    Defined as row-wise quantisation of the transposed input."""
    xb = to_bf16_bits(x)
    xt = np.ascontiguousarray(np.swapaxes(xb, -1, -2))
    return quantize_mx_rowwise(xt, fmt, scale_mode)


def quantize_mx_2d(x, fmt: int = FMT_E4M3, scale_mode: int = SCALE_OCP_FLOOR):
    """2-D 32x32 block quantisation for weights (``use_2d_block=True``,
    primus_turbo.py:313-317; grid definition weight_deosc.py:29-33): one scale
    per 32x32 tile of each [N, K] matrix (leading dims are independent
    matrices).  Returns the row-wise copy and the transposed copy, each with
    its per-row scale array (the tile scale replicated):
      (codes[..., N, K], scales[..., N, K/32], codesT[..., K, N], scalesT[..., K, N/32]).
    """
    xb = to_bf16_bits(x)
    N, K = xb.shape[-2], xb.shape[-1]
    assert N % BLOCK == 0 and K % BLOCK == 0
    lead = xb.shape[:-2]
    t = xb.reshape(lead + (N // BLOCK, BLOCK, K // BLOCK, BLOCK))
    t = np.moveaxis(t, -2, -3)  # [..., N/32, K/32, 32, 32]
    byte = _block_scale_bytes(t.reshape(t.shape[:-2] + (BLOCK * BLOCK,)), fmt, scale_mode)
    code_t = _cast_scaled(t, np.broadcast_to(byte[..., None, None], t.shape), fmt)
    code = np.moveaxis(code_t, -3, -2).reshape(xb.shape)
    codeT = np.ascontiguousarray(np.swapaxes(code, -1, -2))
    s_row = np.repeat(byte, BLOCK, axis=-2)  # [..., N, K/32]
    s_col = np.repeat(np.swapaxes(byte, -1, -2), BLOCK, axis=-2)  # [..., K, N/32]
    if fmt == FMT_E2M1:
        code = pack_fp4(code)
        codeT = pack_fp4(codeT)
    return code, s_row, codeT, s_col


def dequantize_mx(codes: np.ndarray, scales: np.ndarray, fmt: int = FMT_E4M3) -> np.ndarray:
    """Inverse of the row-wise layout: float32[..., K]."""
    if fmt == FMT_E2M1:
        vals = decode_e2m1(unpack_fp4(codes))
    else:
        vals = decode_e4m3(codes)
    s = np.repeat(scale_f32(scales), BLOCK, axis=-1)
    with np.errstate(invalid="ignore", over="ignore"):
        return (vals * s).astype(np.float32)


# --------------------------------------------------------------------------
# ragged (per-expert) column-wise layout used by the wgrad GEMM
# --------------------------------------------------------------------------
SEG_ALIGN = 128


def segment_layout(group_lens, align: int = SEG_ALIGN):
    """Offsets of each group's rows in the token-major tensor (``offs``) and in
    the padded transposed tensor (``poffs``); every group's padded length is
    its length rounded up to ``align``."""
    lens = np.asarray(group_lens, dtype=np.int64)
    offs = np.concatenate([[0], np.cumsum(lens)])
    plen = (lens + align - 1) // align * align
    poffs = np.concatenate([[0], np.cumsum(plen)])
    return offs, poffs


def padded_width(total_rows: int, num_groups: int, align: int = SEG_ALIGN) -> int:
    """Capacity (in elements along the contraction dim) of the padded
    transposed tensor, computable without reading ``group_lens``."""
    return (total_rows + (align - 1) * max(num_groups, 1)) // align * align


def quantize_mx_colwise_segmented(x, group_lens, fmt: int = FMT_E4M3, scale_mode: int = SCALE_OCP_FLOOR):
    """Column-wise (transposed) quantisation whose 32-blocks restart at every
    expert boundary, for the ragged-contraction wgrad GEMM
    (zbpp_gemm.py:633-639 describes the segment-aware requirement).

    x[sum(M_g), C] -> codes[C, W], scales[C, W/32] with
    W = padded_width(sum(M_g), G).  Group g occupies columns
    [poffs[g], poffs[g] + M_g); the tail up to the next multiple of 128 holds
    zero codes and a scale computed from the zero-padded block (byte 0 for an
    all-padding block).  Columns past poffs[G] are zero / byte 0.
    """
    xb = to_bf16_bits(x)
    lens = np.asarray(group_lens, dtype=np.int64)
    total, C = xb.shape
    assert lens.sum() == total
    offs, poffs = segment_layout(lens)
    W = padded_width(total, len(lens))
    xp = np.zeros((W, C), dtype=np.uint16)
    for g in range(len(lens)):
        xp[poffs[g] : poffs[g] + lens[g]] = xb[offs[g] : offs[g + 1]]
    return quantize_mx_colwise(xp, fmt, scale_mode)


# --------------------------------------------------------------------------
# stochastic rounding to E2M1 (gradients of the MXFP4 recipe)
# --------------------------------------------------------------------------
_E2M1_GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float64)


def _sr_mix(x: np.ndarray) -> np.ndarray:
    """32-bit integer finaliser (xor-shift / odd-multiply rounds), a bijection on uint32."""
    x = x.astype(np.uint64)
    m = np.uint64(0xFFFFFFFF)
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & m
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & m
    x ^= x >> np.uint64(16)
    return x


def sr_word(counter: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """32 random bits per 64-bit counter value: two rounds of the finaliser over the
    counter, the 64-bit seed and the stream id.  Returned as uint32."""
    c = np.asarray(counter, dtype=np.uint64)
    m = np.uint64(0xFFFFFFFF)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    h = _sr_mix((c & m) ^ np.uint64(seed & 0xFFFFFFFF))
    t = (h + ((c >> np.uint64(32)) * np.uint64(0x9E3779B9)) + np.uint64(seed >> 32)
         + np.uint64((int(stream) * 0x85EBCA6B) & 0xFFFFFFFF)) & m
    return _sr_mix(t).astype(np.uint32)


def cast_e2m1_sr(v: np.ndarray, rnd16: np.ndarray) -> np.ndarray:
    """float32 (already divided by the block scale, finite) -> E2M1 code with stochastic rounding.

    |v| lies between two neighbouring values lo <= |v| < hi of the E2M1 table.  With
    T = floor((|v| - lo) / (hi - lo) * 2^22) the result is hi when T + 64 * rnd16 >= 2^22 and lo
    otherwise, i.e. hi with probability ceil(T / 64) / 2^16 over a uniform 16-bit ``rnd16``;
    values at or above 6 give 6.  The sign bit is the input's."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    sign = ((v.view(np.uint32) >> np.uint32(28)) & np.uint32(0x8)).astype(np.uint8)
    w = np.abs(v).astype(np.float64)
    idx = np.searchsorted(_E2M1_GRID, w, side="right") - 1          # largest table entry <= w
    idx = np.clip(idx, 0, 7)
    lo = _E2M1_GRID[idx]
    hi = _E2M1_GRID[np.minimum(idx + 1, 7)]
    step = np.where(idx < 7, hi - lo, 1.0)
    frac = np.where(idx < 7, (w - lo) / step, 0.0)
    T = np.floor(frac * float(1 << 22)).astype(np.int64)
    up = (T + (rnd16.astype(np.int64) << 6)) >= (1 << 22)
    code = np.minimum(idx + up.astype(np.int64), 7)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def quantize_mx_rowwise_sr(x, seed: int, scale_mode: int = SCALE_OCP_FLOOR, stream: int = 0):
    """``quantize_mx_rowwise(x, FMT_E2M1)`` with stochastically rounded codes: same scales; the
    random word of the element pair (row r, columns 2j and 2j+1) is
    ``sr_word(r * K/2 + j, seed, stream)``, low half for the even column."""
    xb = to_bf16_bits(x)
    assert xb.ndim == 2
    R, K = xb.shape
    assert K % BLOCK == 0
    blocks = xb.reshape(R, K // BLOCK, BLOCK)
    byte = _block_scale_bytes(blocks, FMT_E2M1, scale_mode)
    byte_el = np.broadcast_to(byte[..., None], blocks.shape).reshape(R, K)
    xf = bf16_bits_to_f32(xb)
    with np.errstate(invalid="ignore", over="ignore"):
        v = (xf * inv_scale_f32(byte_el)).astype(np.float32)
    counter = (np.arange(R, dtype=np.uint64)[:, None] * np.uint64(K // 2) + np.arange(K // 2, dtype=np.uint64)[None, :])
    words = sr_word(counter, seed, stream)                               # [R, K/2]
    rnd16 = np.stack([words & np.uint32(0xFFFF), words >> np.uint32(16)], axis=-1).reshape(R, K)
    finite_block = byte_el != 255
    code = cast_e2m1_sr(np.where(finite_block, v, np.float32(0)), rnd16)
    # blocks holding NaN / Inf (scale byte 255) are coded as by the round-to-nearest path
    rne = _cast_scaled(xb, byte_el, FMT_E2M1)
    code = np.where(finite_block, code, rne).astype(np.uint8)
    return pack_fp4(code), byte


def _segment_padded(x, group_lens):
    """bf16 bits of x[sum(M_g), C] laid out as [W, C] with every group at its padded offset."""
    xb = to_bf16_bits(x)
    lens = np.asarray(group_lens, dtype=np.int64)
    total, C = xb.shape
    assert lens.sum() == total
    offs, poffs = segment_layout(lens)
    W = padded_width(total, len(lens))
    xp = np.zeros((W, C), dtype=np.uint16)
    for g in range(len(lens)):
        xp[poffs[g] : poffs[g] + lens[g]] = xb[offs[g] : offs[g + 1]]
    return xp


def hadamard16_rows(xb: np.ndarray, signs: int) -> np.ndarray:
    """Randomised Hadamard transform over groups of 16 consecutive rows of bf16 bits ``xb[W, C]``
    (W a multiple of 16): y = (1/4) H16 (s * x) per group, H16 Sylvester-ordered, s_i = -1 where bit i
    of ``signs`` is set.  Four float32 butterfly stages with strides 1, 2, 4, 8 (new[i] = old[i] +
    old[i+s], new[i+s] = old[i] - old[i+s]), then * 0.25 and one rounding to bf16."""
    W, C = xb.shape
    assert W % 16 == 0
    v = bf16_bits_to_f32(xb).reshape(W // 16, 16, C).astype(np.float32)
    s = np.array([-1.0 if (signs >> i) & 1 else 1.0 for i in range(16)], dtype=np.float32)
    v = v * s[None, :, None]
    with np.errstate(invalid="ignore", over="ignore"):
        for st in (1, 2, 4, 8):
            out = np.empty_like(v)
            for i in range(16):
                if i & st:
                    continue
                out[:, i] = v[:, i] + v[:, i + st]
                out[:, i + st] = v[:, i] - v[:, i + st]
            v = out
        v = v * np.float32(0.25)
    return f32_to_bf16_bits(v.reshape(W, C))


def quantize_mx_colwise_segmented_fp4(x, group_lens, scale_mode: int = SCALE_OCP_FLOOR, sr_seed=None, rht_signs=None):
    """The transposed, segment-padded MXFP4 copy with the recipe's options: optional Hadamard
    transform along the (padded) token axis first, then round-to-nearest or stochastic rounding."""
    xp = _segment_padded(x, group_lens)
    if rht_signs is not None:
        xp = hadamard16_rows(xp, rht_signs)
    xt = np.ascontiguousarray(xp.T)
    if sr_seed is None:
        return quantize_mx_rowwise(xt, FMT_E2M1, scale_mode)
    return quantize_mx_rowwise_sr(xt, sr_seed, scale_mode, stream=1)


def quantize_mx_colwise_segmented_sr(x, group_lens, seed: int, scale_mode: int = SCALE_OCP_FLOOR):
    """``quantize_mx_colwise_segmented(x, group_lens, FMT_E2M1)`` with stochastic rounding: the
    row-wise routine applied to the transposed, segment-padded tensor ``[C, W]`` with stream 1."""
    return quantize_mx_colwise_segmented_fp4(x, group_lens, scale_mode, sr_seed=seed)


# --------------------------------------------------------------------------
# GEMMs: dequantise -> fp32 matmul -> bf16
# --------------------------------------------------------------------------
def _matmul_nt_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    return np.matmul(a.astype(np.float32), b.astype(np.float32).T).astype(np.float32)


def gemm_nt_ref(a_codes, a_scales, b_codes, b_scales, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, out_bf16=True):
    """C[M, N] = dq(A)[M, K] . dq(B)[N, K]^T, fp32 accumulate."""
    a = dequantize_mx(a_codes, a_scales, a_fmt)
    b = dequantize_mx(b_codes, b_scales, b_fmt)
    c = _matmul_nt_f32(a, b)
    return f32_to_bf16_bits(c) if out_bf16 else c


def grouped_gemm_nt_ref(a_codes, a_scales, b_codes, b_scales, group_lens, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, out_bf16=True):
    """Forward / dgrad grouped GEMM: rows of A are split by ``group_lens``;
    B is [G, N, K].  Empty groups contribute no rows."""
    lens = np.asarray(group_lens, dtype=np.int64)
    offs = np.concatenate([[0], np.cumsum(lens)])
    N = b_codes.shape[1]
    out = np.zeros((a_codes.shape[0], N), dtype=np.float32)
    for g in range(len(lens)):
        if lens[g] == 0:
            continue
        sl = slice(offs[g], offs[g + 1])
        out[sl] = gemm_nt_ref(a_codes[sl], a_scales[sl], b_codes[g], b_scales[g], a_fmt, b_fmt, out_bf16=False)
    return f32_to_bf16_bits(out) if out_bf16 else out


def grouped_gemm_wgrad_ref(a_codes, a_scales, b_codes, b_scales, group_lens, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, out_bf16=True):
    """Variable-K (wgrad) grouped GEMM on the segmented transposed layout:
    A = dY^T codes [N, W], B = X^T codes [K, W]; dW[g] = A[:, seg_g] . B[:, seg_g]^T.
    Empty groups give an all-zero dW[g]."""
    lens = np.asarray(group_lens, dtype=np.int64)
    _, poffs = segment_layout(lens)
    a_per = 2 if a_fmt == FMT_E2M1 else 1
    b_per = 2 if b_fmt == FMT_E2M1 else 1
    G = len(lens)
    out = np.zeros((G, a_codes.shape[0], b_codes.shape[0]), dtype=np.float32)
    for g in range(G):
        lo, hi = int(poffs[g]), int(poffs[g + 1])
        if hi == lo:
            continue
        out[g] = gemm_nt_ref(
            a_codes[:, lo // a_per : hi // a_per],
            a_scales[:, lo // BLOCK : hi // BLOCK],
            b_codes[:, lo // b_per : hi // b_per],
            b_scales[:, lo // BLOCK : hi // BLOCK],
            a_fmt,
            b_fmt,
            out_bf16=False,
        )
    return f32_to_bf16_bits(out) if out_bf16 else out


# --------------------------------------------------------------------------
# end-to-end linear (what ops.gemm_fp8 / grouped_gemm_fp8 compute)
# --------------------------------------------------------------------------
def linear_fwd_ref(x, w, fmt_x=FMT_E4M3, fmt_w=FMT_E4M3, scale_mode=SCALE_OCP_FLOOR, w_2d=True):
    """Y = Q(X) . Q(W)^T for bf16 x[M, K], w[N, K] (primus_turbo.py:1095-1103)."""
    xq, xs = quantize_mx_rowwise(x, fmt_x, scale_mode)
    if w_2d:
        wq, ws, _, _ = quantize_mx_2d(w, fmt_w, scale_mode)
    else:
        wq, ws = quantize_mx_rowwise(w, fmt_w, scale_mode)
    return gemm_nt_ref(xq, xs, wq, ws, fmt_x, fmt_w)


def linear_bwd_ref(x, w, dy, fmt=FMT_E4M3, scale_mode=SCALE_OCP_FLOOR, group_lens=None):
    """(dX, dW) of the dense or grouped linear on bf16 inputs.
    dX = Q_row(dY) . Q_colT(W)^T (contraction N); dW = Q_colT(dY) . Q_colT(X)^T
    (contraction M, segment-aware).  Weight copies use 2-D blocks."""
    xb, wb, dyb = to_bf16_bits(x), to_bf16_bits(w), to_bf16_bits(dy)
    dense = group_lens is None
    if dense:
        group_lens = [xb.shape[0]]
        wb = wb[None]
    dyq, dys = quantize_mx_rowwise(dyb, fmt, scale_mode)
    _, _, wqT, wsT = quantize_mx_2d(wb, fmt, scale_mode)
    dx = grouped_gemm_nt_ref(dyq, dys, wqT, wsT, group_lens, fmt, fmt)
    dyT, dysT = quantize_mx_colwise_segmented(dyb, group_lens, fmt, scale_mode)
    xT, xsT = quantize_mx_colwise_segmented(xb, group_lens, fmt, scale_mode)
    dw = grouped_gemm_wgrad_ref(dyT, dysT, xT, xsT, group_lens, fmt, fmt)
    if dense:
        dw = dw[0]
    return dx, dw


# --------------------------------------------------------------------------
# gated activation x router probability (swiglu_with_probs / geglu_with_probs)
# --------------------------------------------------------------------------
def _erfc(x: np.ndarray) -> np.ndarray:
    from math import erfc

    return np.vectorize(erfc, otypes=[np.float64])(x)


def _act64(g: np.ndarray, activation: str):
    """act(g) and act'(g) in float64."""
    if activation == "silu":
        s = 1.0 / (1.0 + np.exp(-g))
        return g * s, s * (1.0 + g * (1.0 - s))
    if activation == "gelu":
        c = 0.5 * _erfc(-g / np.sqrt(2.0))   # = Phi(g); erfc keeps the negative tail free of cancellation
        return g * c, c + g * np.exp(-0.5 * g * g) / np.sqrt(2.0 * np.pi)
    raise ValueError(activation)


def glu_with_probs_ref(x, probs, row_mask=None, activation: str = "silu", out_bf16: bool = True):
    """y[m, j] = act(x[m, j]) * x[m, F + j] * probs[m]; masked rows are zero.
    ``x``: bf16 [M, 2F] (torch tensor, uint16 bits or floats); float64 arithmetic,
    one rounding to bf16 (returned as bits) unless ``out_bf16`` is False."""
    xf = bf16_bits_to_f32(to_bf16_bits(x)).astype(np.float64)
    f = xf.shape[1] // 2
    p = np.asarray(probs, dtype=np.float64).reshape(-1, 1)
    with np.errstate(over="ignore"):
        a, _ = _act64(xf[:, :f], activation)
    y = a * xf[:, f:] * p
    if row_mask is not None:
        y = np.where(np.asarray(row_mask).astype(bool).reshape(-1, 1), y, 0.0)
    return f32_to_bf16_bits(y.astype(np.float32)) if out_bf16 else y


def glu_with_probs_bwd_ref(dy, x, probs, row_mask=None, activation: str = "silu"):
    """(dx [M, 2F], dprobs [M]) in float64 for bf16 ``dy`` [M, F] and ``x`` [M, 2F]."""
    xf = bf16_bits_to_f32(to_bf16_bits(x)).astype(np.float64)
    d = bf16_bits_to_f32(to_bf16_bits(dy)).astype(np.float64)
    f = xf.shape[1] // 2
    p = np.asarray(probs, dtype=np.float64).reshape(-1, 1)
    with np.errstate(over="ignore"):
        a, da = _act64(xf[:, :f], activation)
    u = xf[:, f:]
    dx = np.concatenate([d * p * u * da, d * p * a], axis=1)
    dp = (d * a * u).sum(axis=1)
    if row_mask is not None:
        m = np.asarray(row_mask).astype(bool)
        dx = np.where(m.reshape(-1, 1), dx, 0.0)
        dp = np.where(m, dp, 0.0)
    return dx, dp


# --------------------------------------------------------------------------
# RMSNorm in front of the column-parallel linear (primus_turbo.py:1689-1700)
# --------------------------------------------------------------------------
_NORM_THREADS = 256


def rmsnorm_rstd(x, eps: float) -> np.ndarray:
    """rstd[m] = 1 / sqrt(mean_j x[m, j]^2 + eps) in float32, summed in the order of the HIP kernel:
    lane t of 256 adds the squares of its 8-element chunks (columns 8t + 2048 i ...) one element at a
    time, the 64 lanes of a wave are combined by an xor butterfly from distance 32 down to 1, the four
    waves are added in order.  (Squares of bf16 values are exact in float32.)"""
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    rows, k = xf.shape
    assert k % 8 == 0
    chunks = -(-k // (_NORM_THREADS * 8))
    pad = np.zeros((rows, chunks * _NORM_THREADS * 8), dtype=np.float32)
    pad[:, :k] = xf
    sq = (pad * pad).reshape(rows, chunks, _NORM_THREADS, 8)
    lane = np.zeros((rows, _NORM_THREADS), dtype=np.float32)
    for c in range(chunks):
        for e in range(8):
            lane = lane + sq[:, c, :, e]
    v = lane.reshape(rows, 4, 64)
    for s_ in (32, 16, 8, 4, 2, 1):
        v = v + v[:, :, np.arange(64) ^ s_]
    part = v[:, :, 0]
    total = ((part[:, 0] + part[:, 1]) + part[:, 2]) + part[:, 3]
    mean = total / np.float32(k)
    return (np.float32(1.0) / np.sqrt(mean + np.float32(eps), dtype=np.float32)).astype(np.float32)


def rmsnorm_ref(x, w, eps: float):
    """(y bits [rows, k], rstd [rows]): y = (x * rstd) * w, float32 products in that order, one rounding."""
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    wf = bf16_bits_to_f32(to_bf16_bits(w)).reshape(1, -1)
    rstd = rmsnorm_rstd(x, eps)
    y = (xf * rstd.reshape(-1, 1)) * wf
    return f32_to_bf16_bits(y.astype(np.float32)), rstd


def rmsnorm_bwd_ref(dy, x, w, eps: float):
    """(dx [rows, k], dw [k]) in float64 from the closed form: with g = dy * w, xh = x * rstd,
    dx = (g - xh * mean_j(g * xh)) * rstd and dw = sum_m dy * xh."""
    xf = bf16_bits_to_f32(to_bf16_bits(x)).astype(np.float64)
    d = bf16_bits_to_f32(to_bf16_bits(dy)).astype(np.float64)
    wf = bf16_bits_to_f32(to_bf16_bits(w)).astype(np.float64).reshape(1, -1)
    rstd = 1.0 / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + eps)
    xh = xf * rstd
    g = d * wf
    dx = (g - xh * (g * xh).mean(axis=1, keepdims=True)) * rstd
    return dx, (d * xh).sum(axis=0)


# --------------------------------------------------------------------------
# Tensor-wise ("current") FP8 scaling (primus_turbo_float8_local.py:194-207, :215-306)
# --------------------------------------------------------------------------
_FP8_MAX = {FMT_E4M3: 448.0, FMT_E5M2: 57344.0}


def cast_e5m2(v: np.ndarray) -> np.ndarray:
    """float32 -> FP8 E5M2 code, RNE, saturating at +-57344, sign kept on zero results, NaN -> sign|0x7F."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    u = v.view(np.uint32)
    sign = ((u >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    a_bits = u & np.uint32(0x7FFFFFFF)
    nan = a_bits > np.uint32(0x7F800000)
    a = np.minimum(a_bits.view(np.float32), np.float32(57344.0))
    a = np.where(nan, np.float32(0.0), a).astype(np.float32)
    ab = a.view(np.uint32).astype(np.int64)
    # normal range of e5m2: >= 2^-14; two mantissa bits are kept
    rounded = (ab + 0xFFFFF + ((ab >> 21) & 1)) >> 21  # (exp32 << 2) | m2 after carry
    code_n = rounded - ((127 - 15) << 2)
    # subnormal range: multiples of 2^-16
    code_s = np.rint(a.astype(np.float64) * 65536.0).astype(np.int64)
    code = np.where(a >= np.float32(2.0**-14), code_n, code_s)
    code = np.minimum(code, 0x7B)
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def decode_e5m2(code: np.ndarray) -> np.ndarray:
    c = code.astype(np.int64)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 2) & 0x1F
    m = c & 0x3
    val = np.where(e == 0, m * 2.0**-16, (4 + m) * np.exp2(e.astype(np.float64) - 17.0))
    val = np.where(e == 31, np.where(m == 0, np.inf, np.nan), val)
    return (s * val).astype(np.float32)


def tensor_amax(x) -> np.float32:
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    return np.float32(np.abs(xf).max()) if xf.size else np.float32(0.0)


def quantize_tensorwise(x, fmt: int = FMT_E4M3):
    """(codes uint8 of the shape of x, scale_inv float32): one scale for the whole tensor,
    scale = fp8_max / max(amax, 1e-12), codes = cast(clamp(x * scale, +-fp8_max)), scale_inv = 1 / scale,
    float32 arithmetic.  A NaN or Inf in the tensor turns every code into NaN (0x7F)."""
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    amax = tensor_amax(x)
    with np.errstate(divide="ignore", invalid="ignore"):
        scale = np.float32(_FP8_MAX[fmt]) / np.maximum(amax, np.float32(1e-12))
        scale_inv = np.float32(1.0) / scale
    if not np.isfinite(amax):
        return np.full(xf.shape, 0x7F, dtype=np.uint8), np.float32(scale_inv)
    y = (xf * scale).astype(np.float32)
    codes = cast_e5m2(y) if fmt == FMT_E5M2 else cast_e4m3(y)
    return codes, np.float32(scale_inv)


def decode_fp8(codes: np.ndarray, fmt: int) -> np.ndarray:
    return decode_e5m2(codes) if fmt == FMT_E5M2 else decode_e4m3(codes)


def tensorwise_gemm_nt_ref(a_codes, a_scale_inv, b_codes, b_scale_inv, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, out_bf16=True):
    """c = (decode(a) . decode(b)^T) * a_scale_inv * b_scale_inv: float32 accumulation, the two factors applied
    to the sum, one rounding to bf16 (gemm_fp8_impl with tensor-wise granularity,
    primus_turbo_float8_local.py:239-250)."""
    acc = _matmul_nt_f32(decode_fp8(a_codes, a_fmt), decode_fp8(b_codes, b_fmt))
    c = (acc * (np.float32(a_scale_inv) * np.float32(b_scale_inv))).astype(np.float32)
    return f32_to_bf16_bits(c) if out_bf16 else c


# --------------------------------------------------------------------------
# expert groups padded to the quantisation alignment
# --------------------------------------------------------------------------
def padded_rows_bound(rows: int, num_groups: int, align: int) -> int:
    """Largest sum of padded group lengths that ``num_groups`` counts summing to ``rows`` can produce."""
    return (rows + num_groups * (align - 1)) // align * align


def pad_groups(x: np.ndarray, group_lens, align: int, out_rows=None):
    """``(out, padded_lens)``: every group's rows followed by zero rows up to a multiple of ``align``
    (experts.py:196-209).  ``out_rows`` None gives the exact size, which is the reference's result; a larger
    buffer ends in zero rows that are counted into the last group."""
    lens = [max(int(n), 0) for n in group_lens]
    padded = [(n + align - 1) // align * align for n in lens]
    total = sum(padded)
    out_rows = total if out_rows is None else int(out_rows)
    assert out_rows >= total
    out = np.zeros((out_rows,) + x.shape[1:], dtype=x.dtype)
    src = dst = 0
    for n, m in zip(lens, padded):
        out[dst:dst + n] = x[src:src + n]
        src += n
        dst += m
    padded[-1] += out_rows - total
    return out, np.asarray(padded, dtype=np.int64)


def unpad_groups(y: np.ndarray, group_lens, align: int, rows=None) -> np.ndarray:
    """Inverse of ``pad_groups`` (experts.py:262-264): the first ``len`` rows of every padded group, back to back;
    rows of the result behind ``sum(group_lens)`` are zero."""
    lens = [max(int(n), 0) for n in group_lens]
    rows = sum(lens) if rows is None else int(rows)
    out = np.zeros((rows,) + y.shape[1:], dtype=y.dtype)
    src = dst = 0
    for n in lens:
        out[dst:dst + n] = y[src:src + n]
        dst += n
        src += (n + align - 1) // align * align
    return out


# --------------------------------------------------------------------------
# the 128-blockwise FP8 recipe
# --------------------------------------------------------------------------
BW_BLOCK = 128


def _quantize_blocks(xf: np.ndarray, amax: np.ndarray, fmt: int):
    """codes of xf and scale_inv per entry of amax (broadcastable to xf): the tensor-wise formula per block."""
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        scale = (np.float32(_FP8_MAX[fmt]) / np.maximum(amax.astype(np.float32), np.float32(1e-12))).astype(np.float32)
        scale_inv = (np.float32(1.0) / scale).astype(np.float32)
        y = (xf * scale).astype(np.float32)
    codes = cast_e5m2(y) if fmt == FMT_E5M2 else cast_e4m3(y)
    codes = np.where(np.isfinite(np.broadcast_to(amax, xf.shape)), codes, np.uint8(0x7F)).astype(np.uint8)
    return codes, scale_inv


def quantize_blockwise(x, fmt: int = FMT_E4M3, axis: int = -1, block: int = BW_BLOCK):
    """quant_fp8_blockwise_impl(x, dtype, axis, block_size) (primus_turbo_float8_local.py:1019, :1053-1059):
    1-D blocks of ``block`` along ``axis`` of the 2-D ``x``.
    axis -1 / 1: ``(codes [rows, cols], scale_inv [rows, cols / block])``; cols must be a multiple of the block.
    axis -2 / 0: blocks along the rows, returned TRANSPOSED and zero-padded as the NT GEMM consumes the copy:
    ``(codes [cols, rows_pad], scale_inv [cols, rows_pad / block])``; a block that reaches past the last row takes its
    scale from the rows it has."""
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    rows, cols = xf.shape
    if axis in (-2, 0):
        pad = (-rows) % block
        xt = np.concatenate([xf, np.zeros((pad, cols), np.float32)]).T.copy()      # [cols, rows_pad]
        return quantize_blockwise(f32_to_bf16_bits(xt), fmt, -1, block)
    assert cols % block == 0
    blocks = xf.reshape(rows, cols // block, block)
    amax = np.abs(blocks).max(axis=2, keepdims=True)
    codes, scale_inv = _quantize_blocks(blocks, amax, fmt)
    return codes.reshape(rows, cols), scale_inv.reshape(rows, cols // block)


def quantize_blockwise_2d(w, fmt: int = FMT_E4M3, block: int = BW_BLOCK):
    """quant_fp8_blockwise_for_weight_impl (primus_turbo_float8_local.py:1020, :1060): one scale per block x block
    tile of ``w [n, k]``.  ``(codes [n, k], scale_inv [n / block, k / block], codes_T [k, n], scale_inv_T)``."""
    wf = bf16_bits_to_f32(to_bf16_bits(w))
    n, k = wf.shape
    assert n % block == 0 and k % block == 0
    tiles = wf.reshape(n // block, block, k // block, block)
    amax = np.abs(tiles).max(axis=(1, 3), keepdims=True)
    codes, scale_inv = _quantize_blocks(tiles, amax, fmt)
    codes = codes.reshape(n, k)
    scale_inv = scale_inv.reshape(n // block, k // block)
    return codes, scale_inv, codes.T.copy(), scale_inv.T.copy()


def blockwise_gemm_nt_ref(a_codes, a_sinv, b_codes, b_sinv, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, block: int = BW_BLOCK, out_bf16=True):
    """c[m, n] = sum over K blocks of a_sinv[m, kb] * b_sinv[n (or n / block), kb] * (a[m, kb] . b[n, kb]) in float32
    (gemm_fp8_impl with blockwise granularity, primus_turbo_float8_local.py:1022-1033).  ``b_sinv`` has one row per
    row of b or one per ``block`` rows (weights)."""
    a = decode_fp8(a_codes, a_fmt)
    b = decode_fp8(b_codes, b_fmt)
    m, k = a.shape
    n = b.shape[0]
    sb = np.repeat(b_sinv, block, axis=0) if b_sinv.shape[0] != n else b_sinv
    acc = np.zeros((m, n), np.float32)
    for kb in range(k // block):
        sl = slice(kb * block, (kb + 1) * block)
        part = _matmul_nt_f32(a[:, sl], b[:, sl])
        acc = (acc + part * (a_sinv[:, kb][:, None] * sb[:, kb][None, :]).astype(np.float32)).astype(np.float32)
    return f32_to_bf16_bits(acc) if out_bf16 else acc


def quantize_blockwise_segmented(x, group_lens, fmt: int = FMT_E4M3, block: int = BW_BLOCK):
    """The copy with blocks along the rows for a tensor whose rows are split into groups
    (quant_fp8_blockwise_segment_m_row_col_impl, zbpp_gemm.py:633, :785), in the layout the wgrad GEMM consumes:
    transposed and segment-padded, ``(codes [cols, W], scale_inv [cols, W / block])`` with ``W = padded_width(rows,
    G, block)``; group g owns columns ``[poff_g, poff_g + len_g)``, so the blocks restart at every group.  Padding is
    zero codes; the scale_inv of a block that holds nothing is the one of an all-zero block."""
    xf = bf16_bits_to_f32(to_bf16_bits(x))
    rows, cols = xf.shape
    lens = [max(int(n), 0) for n in group_lens]
    W = padded_width(rows, len(lens), block)
    codes = np.zeros((cols, W), np.uint8)
    empty = np.float32(1.0) / (np.float32(_FP8_MAX[fmt]) / np.float32(1e-12))
    sinv = np.full((cols, W // block), empty, np.float32)
    src = dst = 0
    for n in lens:
        if n:
            c, s = quantize_blockwise(f32_to_bf16_bits(xf[src:src + n]), fmt, 0, block)
            codes[:, dst:dst + c.shape[1]] = c
            sinv[:, dst // block:dst // block + s.shape[1]] = s
        src += n
        dst += (n + block - 1) // block * block
    return codes, sinv


def grouped_blockwise_gemm_nt_ref(a_codes, a_sinv, b_codes, b_sinv, group_lens, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, out_bf16=True):
    """Rows of a split by group_lens, b [G, n, k] with b_sinv [G, n / 128, k / 128] (grouped_gemm_fp8_impl with blockwise
    granularity, zbpp_gemm.py:608-630)."""
    outs, pos = [], 0
    for g, n in enumerate(max(int(v), 0) for v in group_lens):
        outs.append(blockwise_gemm_nt_ref(a_codes[pos:pos + n], a_sinv[pos:pos + n], b_codes[g], b_sinv[g], a_fmt, b_fmt,
                                          out_bf16=out_bf16))
        pos += n
    dt = np.uint16 if out_bf16 else np.float32
    return np.concatenate(outs) if outs else np.zeros((0, b_codes.shape[1]), dt)


def grouped_blockwise_wgrad_ref(a_codes, a_sinv, b_codes, b_sinv, group_lens, a_fmt=FMT_E4M3, b_fmt=FMT_E4M3, block: int = BW_BLOCK,
                                out_bf16=True):
    """c[g] = a[:, seg_g] . b[:, seg_g]^T on the segment-padded transposed copies (grouped_gemm_fp8_variable_k_impl,
    zbpp_gemm.py:757-800); a group without tokens yields zeros."""
    outs, pos = [], 0
    for n in (max(int(v), 0) for v in group_lens):
        w = (n + block - 1) // block * block
        if w:
            outs.append(blockwise_gemm_nt_ref(a_codes[:, pos:pos + w], a_sinv[:, pos // block:(pos + w) // block],
                                              b_codes[:, pos:pos + w], b_sinv[:, pos // block:(pos + w) // block], a_fmt, b_fmt,
                                              out_bf16=out_bf16))
        else:
            outs.append(np.zeros((a_codes.shape[0], b_codes.shape[0]), np.uint16 if out_bf16 else np.float32))
        pos += w
    return np.stack(outs)


# --------------------------------------------------------------------------
# pre-shuffled MXFP4 layouts (byte permutations; see the header)
# --------------------------------------------------------------------------
def _shuffle_codes_index(rows: int, row_bytes: int) -> np.ndarray:
    """dst flat byte offset of source byte (r, b): blocks of 16 rows x 32 bytes, each stored as
    [half of 16 bytes][row in block][byte]."""
    if rows % 16 or row_bytes % 32:
        raise ValueError("the shuffled code layout needs rows % 16 == 0 and row bytes % 32 == 0")
    r = np.arange(rows, dtype=np.int64)[:, None]
    b = np.arange(row_bytes, dtype=np.int64)[None, :]
    block = (r // 16) * (row_bytes // 32) + b // 32
    return block * 512 + ((b % 32) // 16) * 256 + (r % 16) * 16 + b % 16


def shuffle_codes_16x16(codes: np.ndarray) -> np.ndarray:
    """``codes`` uint8 [rows, row_bytes] (packed FP4: two elements a byte) -> the same shape, shuffled."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    idx = _shuffle_codes_index(*codes.shape)
    out = np.empty(codes.size, dtype=np.uint8)
    out[idx.ravel()] = codes.ravel()
    return out.reshape(codes.shape)


def unshuffle_codes_16x16(shuffled: np.ndarray) -> np.ndarray:
    shuffled = np.ascontiguousarray(shuffled, dtype=np.uint8)
    idx = _shuffle_codes_index(*shuffled.shape)
    return shuffled.ravel()[idx.ravel()].reshape(shuffled.shape)


def shuffled_scale_shape(rows: int, blocks: int):
    return (rows + 255) // 256 * 256, (blocks + 7) // 8 * 8


def _shuffle_scale_index(rows: int, blocks: int, ld: int) -> np.ndarray:
    """dst flat offset of scale (m, n) in the padded [.., ld] array: 32 rows x 8 blocks form one 256-byte group
    stored as [block % 4][row % 16][(block / 4) % 2][(row / 16) % 2]."""
    m = np.arange(rows, dtype=np.int64)[:, None]
    n = np.arange(blocks, dtype=np.int64)[None, :]
    group = (m // 32) * (ld // 8) + n // 8
    return group * 256 + (n % 4) * 64 + (m % 16) * 4 + ((n // 4) % 2) * 2 + (m // 16) % 2


def shuffle_e8m0(scales: np.ndarray) -> np.ndarray:
    """``scales`` uint8 [rows, blocks] -> [ceil(rows / 256) * 256, ceil(blocks / 8) * 8], zero bytes in the padding."""
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    rows, blocks = scales.shape
    pr, pb = shuffled_scale_shape(rows, blocks)
    out = np.zeros(pr * pb, dtype=np.uint8)
    out[_shuffle_scale_index(rows, blocks, pb).ravel()] = scales.ravel()
    return out.reshape(pr, pb)


def unshuffle_e8m0(shuffled: np.ndarray, rows: int, blocks: int) -> np.ndarray:
    shuffled = np.ascontiguousarray(shuffled, dtype=np.uint8)
    if tuple(shuffled.shape) != shuffled_scale_shape(rows, blocks):
        raise ValueError("shuffled scales have the wrong shape")
    return shuffled.ravel()[_shuffle_scale_index(rows, blocks, shuffled.shape[1]).ravel()].reshape(rows, blocks)
