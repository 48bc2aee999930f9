/*
 * mxlinear.h -- C ABI of the MI355X (gfx950) MX low-precision linear path.
 *
 * The reference (AMD-AGI/Primus) reaches this path through the Python operator
 * surface of the external package `primus_turbo`; the entry points below are
 * what a binding for that surface needs, one per kernel family.  Each
 * declaration cites the reference call site it serves.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer on the current HIP device unless the
 *     name ends in _host; `stream` is a hipStream_t passed as void*.
 *   - calls are asynchronous on `stream`, re-entrant, keep no state between
 *     calls, never allocate, never synchronise and never read device memory
 *     from the host (group_lens stays on the device).
 *   - return value: MXL_OK (0) or a negative MXL_E* code; nothing throws.
 *   - bf16 tensors are row-major and contiguous.
 *   - "codes" are FP8 E4M3 bytes (fmt MXL_FMT_E4M3) or packed FP4 E2M1 nibbles,
 *     two per byte, element 2i in bits 3:0 (fmt MXL_FMT_E2M1); "scales" are
 *     E8M0 bytes, one per 32 elements along the contraction dim, row-major
 *     [rows, K/32].
 */
#ifndef MXLINEAR_H
#define MXLINEAR_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXL_OK 0
#define MXL_EINVAL (-1)  /* bad shape / alignment / enum / null pointer */
#define MXL_ELAUNCH (-2) /* HIP reported an error at launch */
#define MXL_ENODEV (-3)  /* current device is not gfx950 */
#define MXL_ESCRATCH (-4) /* the problem needs more scratch memory than an allocation-free entry point owns */
#define MXL_ESTREAM (-5)  /* an allocation-free entry point was called on a stream it is not bound to */

#define MXL_FMT_E4M3 0
#define MXL_FMT_E2M1 1
#define MXL_FMT_E5M2 2   /* tensor-wise scaled entry points only */

/* E8M0 scale rule (explicit because the reference's kernel library is not in
 * its tree): OCP MX v1.0 floor rule, round-up rule, AITER/Quark "even" rule. */
#define MXL_SCALE_OCP_FLOOR 0
#define MXL_SCALE_RCEIL 1
#define MXL_SCALE_EVEN 2

/* gated activations of the expert MLP and the dtype of the router probabilities */
#define MXL_ACT_SILU 0
#define MXL_ACT_GELU 1
#define MXL_PROBS_F32 0
#define MXL_PROBS_BF16 1

#define MXL_BLOCK 32      /* MX block size (fp8_utils.py:48, fp4_utils.py:79) */
#define MXL_SEG_ALIGN 128 /* padding of each expert segment in the transposed layout */
#define MXL_MAX_GROUPS 1024

int mxl_version(void);
const char* mxl_error_string(int code);

/* Width (elements along the token dim) of the segment-padded transposed
 * layout for `total_rows` tokens in `num_groups` experts; depends on sizes
 * only, never on group_lens. */
int64_t mxl_padded_width(int64_t total_rows, int num_groups);

/* MX quantisation of a bf16 matrix x[rows, cols].
 *
 * Serves QuantizedTensor.quantize(x, axis=-1 / axis=-2)
 * (primus_turbo.py:321-354) and quantize_mxfp4_dual
 * (primus_turbo_mxfp4_local.py:147-161).
 *
 *   q_row / s_row : row-wise copy, blocks along cols: codes [rows, cols] (or
 *                   cols/2 bytes for FP4), scales [rows, cols/32].  Pass NULL
 *                   for both to skip it.
 *   q_colT / s_colT: column-wise copy stored TRANSPOSED, blocks along rows:
 *                   codes [cols, W] (W/2 bytes for FP4), scales [cols, W/32]
 *                   with W = mxl_padded_width(rows, max(num_groups,1)).
 *                   Blocks restart at every group boundary; group g occupies
 *                   columns [poff_g, poff_g + len_g) where poff is the prefix
 *                   sum of the lens rounded up to 128; padding holds zero
 *                   codes.  Pass NULL for both to skip it.
 *   group_lens    : int64[num_groups] on the device, sum == rows; NULL (and
 *                   num_groups 0) means one group of `rows` rows.
 *   row_ld        : number of columns of the row-wise copy, >= cols and a
 *                   multiple of 32 (0 means cols).  Columns past `cols` are
 *                   padding: zero codes, scale byte 0.  The GEMMs want the
 *                   contraction dim in multiples of 128, so a caller pads here
 *                   (the reference pads its MXFP4 operands to 128 as well,
 *                   primus_turbo_mxfp4_local.py:119-124).
 * Requires cols % 32 == 0.
 */
int mxl_quantize(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt, int scale_mode,
                 const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                 void* s_colT, void* stream);

/* mxl_quantize with options (`flags`):
 *
 *   MXL_QF_KCHUNK  K-chunk-major code layout for both copies: instead of codes[rows, ld] the codes are stored
 *                  as [ld / 128][rows][128 elements] (128 or 64 bytes), i.e. the 128 elements of a row that
 *                  one GEMM K slot consumes stay together and consecutive rows follow each other.  A GEMM
 *                  tile's K slot is then one contiguous block (256 rows x 128 bytes) wherever a ragged
 *                  expert starts, and the quantiser writes 16 KiB pieces instead of 128-byte ones.  Needs
 *                  row_ld % 128 == 0.  The transposed copy becomes [W / 128][cols][128].  Scales keep their
 *                  row-major layout.  The GEMM entry points take such operands with MXL_GF_KCHUNK.  This is
 *                  the role the reference's pre-shuffled layouts play for its kernels (use_preshuffle,
 *                  primus_turbo_mxfp4_local.py:184-198); the arrangement itself is this library's own.
 *   MXL_QF_KSTEP   K-step-major layout of codes AND scales for both copies (excludes
 *                  MXL_QF_KCHUNK): codes [ld / 64][rows][64] -- the 64 elements one MFMA K step consumes --
 *                  and scales [ceil(ld / 512)][rows][16], i.e. the 16 scale bytes (8 K steps) of a row stay
 *                  together and consecutive rows follow each other.  Every request of the ring GEMM kernel
 *                  (MXL_GF_KSTEP) then reads whole consecutive cache lines: 64 rows of a K step are 4 KiB,
 *                  the scales of 256 rows for 8 K steps are 4 KiB.  Needs row_ld % 128 == 0; a scale array
 *                  holds ceil(ld / 512) * rows * 16 bytes (bytes past ld / 32 of a row are not written).
 *                  E2M1 codes: an activation copy is written in steps of 128 elements, [ld / 128][rows][64 bytes]
 *                  (the byte geometry of an FP8 copy; the operand format of the FP4 x FP4 ring GEMM), scales as
 *                  above.  A weight (mxl_quantize_weight_2d_ex) is written in steps of 64 elements,
 *                  [ld / 64][rows][32 bytes], the partner of FP8 activations, unless MXL_QF_KSTEP128 is set too:
 *                  then in steps of 128 elements like the activations, the partner of E2M1 activations.
 *
 * and, for fmt = MXL_FMT_E2M1 only, the options of the MXFP4 recipe's dual quantiser, quantize_mxfp4_dual
 * (primus_turbo_mxfp4_local.py:133-161; per-operand settings :234-288):
 *
 *   MXL_QF_SR      stochastic rounding of the codes of both copies (rowwise_use_sr / colwise_use_sr;
 *                  config flag mxfp4_gradient_stochastic_rounding,
 *                  primus/configs/modules/megatron/primus_turbo.yaml:21-24).  Scales are those of
 *                  mxl_quantize; each element becomes one of its two neighbours on the E2M1 grid, the
 *                  upper one with probability equal to its fractional position between them (the
 *                  dequantised value is unbiased), saturating at +-6.  The random bits are a
 *                  counter-based hash of `sr_seed` and the element's position in the output:
 *                  reproducible and independent of the launch geometry; the two copies draw from
 *                  different streams.
 *   MXL_QF_RHT_COL randomised Hadamard transform of the transposed copy (colwise_use_rht): every 16
 *                  consecutive token positions of an expert's segment are replaced by
 *                  (1/4) H16 (s * x) before quantisation (H16 Sylvester-ordered, s_i = -1 where bit i
 *                  of `rht_signs` is set; fp32 butterflies, one rounding to bf16).  Requires q_colT.
 *                  Both operands of a wgrad GEMM must use the same `rht_signs`; the product is then
 *                  unchanged up to rounding.  The row-wise copy is never transformed.  Groups of 16
 *                  start at the expert's segment start, so a partially filled last group holds
 *                  transformed data in all 16 positions (the padding rows enter as zeros) and the
 *                  remaining padding holds +-0 codes. */
#define MXL_QF_SR 1u
#define MXL_QF_RHT_COL 2u
#define MXL_QF_KCHUNK 4u
#define MXL_QF_KSTEP 8u
#define MXL_QF_KSTEP128 16u
int mxl_quantize_ex(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt, int scale_mode,
                    const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                    void* s_colT, uint32_t flags, uint64_t sr_seed, uint32_t rht_signs, void* stream);

/* 2-D (32x32 tile) MX quantisation of `batch` independent weight matrices
 * w[batch, n, k] (weights use ScalingRecipe(use_2d_block=True):
 * primus_turbo.py:313-317; grid definition weight_deosc.py:29-33,136-174).
 * Row-wise copy: codes [batch, n, k], scales [batch, n, k/32]; transposed
 * copy: codes [batch, k, n], scales [batch, k, n/32] (either pair may be
 * NULL).  The tile scale is replicated so both copies carry per-row scales.
 * k_ld / n_ld are the padded pitches of the two copies (>= k / >= n, multiples
 * of 32, n_ld at most n rounded up to 128; 0 means no padding): codes
 * [batch, n, k_ld] and [batch, k, n_ld], padding = zero codes, scale byte 0.
 * Requires n % 32 == 0 and k % 32 == 0.  q_colT may be NULL while s_colT is not (and q_row is given): then only the
 * SCALES of the transposed copy are written -- with 2-D blocks its codes are the row-wise codes transposed, which
 * the GEMM can read as they lie (MXL_GF_B_TRANSPOSED). */
int mxl_quantize_weight_2d(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld,
                           int64_t n_ld, int fmt, int scale_mode, void* q_row, void* s_row, void* q_colT, void* s_colT,
                           void* stream);
/* The same with `flags` (MXL_QF_KCHUNK: both copies K-chunk-major over the flattened batch, i.e.
 * [k_ld / 128][batch * n][128] and [n_ld / 128][batch * k][128]; needs k_ld % 128 == 0 resp. n_ld % 128 == 0). */
int mxl_quantize_weight_2d_ex(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld,
                              int64_t n_ld, int fmt, int scale_mode, void* q_row, void* s_row, void* q_colT,
                              void* s_colT, uint32_t flags, void* stream);

/* Row-wise dequantise to bf16 (QuantizedTensor.dequantize(),
 * weight_deosc.py:155-168): out[rows, k] = decode(codes) * 2^(scale-127).  fmt: MXL_FMT_E4M3, MXL_FMT_E2M1 or
 * MXL_FMT_E5M2 (the codes of the tensor-wise and blockwise recipes; their scale bytes are 127). */
int mxl_dequantize(const void* codes, const void* scales, int64_t rows, int64_t k, int fmt,
                   void* out_bf16, void* stream);

/* Dense NT GEMM on pre-quantised operands (gemm_fp8_impl / gemm_fp4_impl:
 * primus_turbo_float8_local.py:239-250, primus_turbo_mxfp4_local.py:319-331):
 *   c[m, n] (bf16) = dq(a)[m, k] . dq(b)[n, k]^T, fp32 accumulation.
 * Requires k % 128 == 0 (scale rows must be dword aligned; callers get there
 * with the row_ld / k_ld padding of the quantisers) and n % 32 == 0.  The contraction length (k here, the
 * padded token width in mxl_grouped_gemm_wgrad) may not exceed 2^23.  group_lens of the grouped entry points
 * are clamped on the device to what the buffers hold (negative counts to 0, the running sum to total_m). */
int mxl_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                const void* b_scales, int b_fmt, void* c_bf16, int64_t m, int64_t n, int64_t k,
                void* stream);

/* Grouped NT GEMM for forward and dgrad (grouped_gemm_fp8_impl,
 * zbpp_gemm.py:590-603; call site primus_turbo.py:2122-2129):
 *   rows of a[total_m, k] are split by group_lens (int64[num_groups], device);
 *   b is [num_groups, n, k]; c[total_m, n] (bf16).  Empty groups are skipped;
 *   group_lens is consumed on the device. */
int mxl_grouped_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                        const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                        int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream);

/* Grouped variable-K GEMM for wgrad (grouped_gemm_fp8_variable_k_impl,
 * zbpp_gemm.py:710-724): operands in the segment-padded transposed layout
 * written by mxl_quantize(..., q_colT, s_colT):
 *   a = dY^T codes [n, W], b = X^T codes [k, W], W = mxl_padded_width(total_m, G);
 *   c[g, n, k] (bf16) = a[:, seg_g] . b[:, seg_g]^T; an empty group yields zeros.
 * Requires n % 32 == 0 and k % 32 == 0.  num_groups == 0 / group_lens NULL
 * means one dense group (dense wgrad). */
int mxl_grouped_gemm_wgrad(const void* a_codes, const void* a_scales, int a_fmt,
                           const void* b_codes, const void* b_scales, int b_fmt, void* c_bf16,
                           const int64_t* group_lens, int num_groups, int64_t total_m, int64_t n,
                           int64_t k, void* stream);

/* The three GEMMs with `flags`.  MXL_GF_KCHUNK: both operands' CODES are K-chunk-major, as written by the
 * quantisers with MXL_QF_KCHUNK -- [k / 128][rows][128 elements] over all rows of the operand (total_m rows
 * of a and num_groups * n rows of b in the forward / dgrad GEMM; n rows of a and k rows of b over the padded
 * token width in wgrad).  Scales stay row-major.  Same results bit for bit; an operand must stay below 4 GiB. */
#define MXL_GF_KCHUNK 1u
/* MXL_GF_KSTEP (instead of MXL_GF_KCHUNK): codes and scales of both operands are K-step-major, as written by the
 * quantisers with MXL_QF_KSTEP.  FP8-format operands, FP8 rows against E2M1 weights in 64-element steps (forward /
 * dgrad), or E2M1 against E2M1 in 128-element steps (MXL_QF_KSTEP128 weights); at most 256 groups; anything else
 * returns MXL_EINVAL.  Served by the 4-slot ring kernel.  Same results bit for bit.
 * In every layout the kernels request whole 256-row tiles, also where a group or the operand ends earlier; a request for
 * a row behind the operand's last row is dropped by the buffer descriptor's range check (the row offset of every request
 * sits where that check sees it), so operands need no readable memory behind them. */
#define MXL_GF_KSTEP 4u
/* mxl_grouped_gemm_wgrad_ex / _scaled only, together with MXL_GF_KCHUNK or MXL_GF_KSTEP (the latter: E4M3 x E4M3,
 * E2M1 x E2M1 and, scaled, E4M3 | E5M2 x E4M3): c_bf16 points to FLOAT32 [g, n, k] and the
 * result is ADDED to it in fp32 (no rounding to bf16).  This is the gradient-accumulation fusion of the reference
 * (fuse_bgrad_accum_pattern = "megatron": the GEMM's beta = 1 epilogue adds into weight.main_grad,
 * primus_turbo.py:166-240, 243-275) -- available here for the MX recipes too.  With no tokens nothing is added. */
#define MXL_GF_ACCUM_F32 2u
/* mxl_grouped_gemm_nt_ex / _scaled only, together with MXL_GF_KSTEP: b_codes are the K-step-major codes of the TRANSPOSED
 * matrices -- of [num_groups, k, n] quantised along n, i.e. [n_ld / 64][num_groups * k][64 bytes] with n_ld = n rounded up
 * to 128 -- while b_scales stay the scales of [num_groups, n, k / 32].  This is the dgrad GEMM reading the ROW-WISE copy
 * of the weight, so that no transposed copy of the weight's codes has to be written or cached (the reference keeps a
 * second quantised copy for it, _maybe_create_quantized_weight_buffers, primus_turbo.py:278-358).  Meaningful where a
 * transposed copy is the same codes transposed: 2-D 32 x 32 block scales (mxl_quantize_weight_2d_ex writes the transposed
 * copy's scales alone when q_colT is NULL and s_colT is not) or tensor-wise scaling.  E4M3 weights with E4M3 (or,
 * scaled, E5M2) rows; or E2M1 weights with E2M1 rows, both in 128-element steps (MXL_QF_KSTEP128: b_codes are then
 * [n_ld / 128][num_groups * k][64 bytes]).  At most 256 groups; k % 128 == 0.  Bit-identical to the GEMM on the
 * transposed copy. */
#define MXL_GF_B_TRANSPOSED 8u
/* mxl_grouped_gemm_nt_ex only, alone (row-major operands): b_codes are E2M1 codes in the pre-shuffled byte order of
 * mxl_shuffle_codes -- what gemm_fp4_impl(..., preshuffled=True) of the reference is handed for its second operand
 * (primus_turbo_mxfp4_local.py:319-331; the first operand's codes are plain there).  E2M1 x E2M1, block scales in
 * the plain row-major layout, n % 16 == 0.  Same results bit for bit as on the plain codes. */
#define MXL_GF_B_SHUFFLED 16u
int mxl_grouped_gemm_nt_ex(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                           const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                           int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream);
int mxl_grouped_gemm_wgrad_ex(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                              const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                              int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream);

/* Grouped GEMM on UNQUANTISED bf16 operands, tokens-per-expert consumed on the device: ops.grouped_gemm, which the
 * reference's grouped linear calls when no low-precision recipe is active
 * (primus/backends/megatron/core/extensions/primus_turbo.py:2210-2216; the first / last layers of an FP4 run:
 * primus/backends/megatron/core/fp4_utils.py:155-165).  fp32 accumulation, one rounding to bf16.
 *   mxl_grouped_gemm_bf16: c[total_m, n] (bf16): the rows of a[total_m, k] are split by group_lens and group g is
 *     multiplied by b[g] = [n, k] (c = a . b_g^T: forward of an NT linear) or, with MXL_BF_B_KN, by b[g] = [k, n]
 *     (c = a . b_g: the dgrad of an NT linear with a = dy, k = its n; or the forward of trans_b = False).
 *     Requires k % 32 == 0, n % 8 == 0, 16-byte aligned pointers.
 *   mxl_grouped_gemm_bf16_wgrad: c[num_groups, m_out, n_out] = sum over the tokens t of group g of
 *     p[t, m_out] * q[t, n_out]  (p = dy, q = x gives the [n, k] weight gradient); a group without tokens yields zeros.
 *     bf16 output, or with MXL_BF_ACCUM_F32 c is float32 and the result is ADDED to it (the main_grad fusion).
 *     Requires m_out % 8 == 0, n_out % 8 == 0; an operand stays below 4 GiB.
 * Output tiles are 256 columns wide and 256 or 128 rows high.  Without a tile flag the library picks: forward / dgrad
 * 256 rows when total_m / num_groups is at least 256, else 128; the weight gradient 128.  MXL_BF_TILE_128 /
 * MXL_BF_TILE_256 state the choice (a caller who knows its groups are few and long, or many and short).  The result does not depend on the tile height beyond fp32 summation order -- it is the
 * same: every output element adds its products in the same order in both. */
#define MXL_BF_B_KN 1u
#define MXL_BF_ACCUM_F32 2u
#define MXL_BF_TILE_128 4u
#define MXL_BF_TILE_256 8u
int mxl_grouped_gemm_bf16(const void* a_bf16, const void* b_bf16, void* c_bf16, const int64_t* group_lens, int num_groups,
                          int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream);
int mxl_grouped_gemm_bf16_wgrad(const void* p_bf16, const void* q_bf16, void* c, const int64_t* group_lens, int num_groups,
                                int64_t total_m, int64_t m_out, int64_t n_out, uint32_t flags, void* stream);

/* Gated activation of the expert MLP fused with the router probability and the row mask
 * (swiglu_with_probs / geglu_with_probs behind fused_bias_act_with_probs, primus_turbo.py:1954-1980;
 * the unfused arithmetic is experts.py:100-118):
 *   y[m, j] = act(x[m, j]) * x[m, F + j] * probs[m]     for bf16 x[rows, 2F], y[rows, F],
 * computed in fp32, rounded once to bf16.  row_mask (one byte per row, may be NULL = all rows live):
 * a row with mask 0 yields zeros (tokens_per_expert_to_mask marks the rows past the routed tokens
 * of a worst-case sized buffer).  probs is fp32 or bf16 per probs_dtype.  Requires f % 8 == 0. */
int mxl_glu_probs_fwd(const void* x_bf16, const void* probs, int probs_dtype, const uint8_t* row_mask,
                      int64_t rows, int64_t f, int act, void* y_bf16, void* stream);

/* Backward of the above: dx[rows, 2F] (bf16) and dprobs[rows] (fp32) from dy[rows, F]; masked rows
 * get zero gradients. */
int mxl_glu_probs_bwd(const void* dy_bf16, const void* x_bf16, const void* probs, int probs_dtype,
                      const uint8_t* row_mask, int64_t rows, int64_t f, int act, void* dx_bf16,
                      void* dprobs_f32, void* stream);

/* The same activation feeding the MX quantiser directly: what mxl_quantize would produce for
 * y = mxl_glu_probs_fwd(x, ...) (bit for bit), without y ever reaching memory.  It saves one bf16
 * write and one bf16 read of [rows, f] between fc1 and fc2 of the expert MLP; the reference runs
 * the activation and the quantisation inside gemm_fp8 as two kernels (experts.py:225-240,
 * primus_turbo.py:2122-2129).  x is [rows, 2 f]; the other arguments are those of mxl_quantize with
 * cols = f.  A row-wise copy must be requested (q_row / s_row not NULL).  flags: 0 or MXL_QF_KCHUNK. */
int mxl_glu_probs_quantize(const void* x_bf16, const void* probs, int probs_dtype, const uint8_t* row_mask,
                           int64_t rows, int64_t f, int64_t row_ld, int act, int fmt, int scale_mode,
                           const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                           void* s_colT, uint32_t flags, void* stream);

/* ---- tensor-wise ("current") FP8 scaling: the non-MX recipe that the same operators serve -------------------
 * One fp32 scale per tensor (the arithmetic the reference restates in _quantize_fp8_tensorwise,
 * primus_turbo_float8_local.py:194-207, and hands to gemm_fp8_impl at :239-250):
 *   amax = max |x|,  scale = fp8_max / max(amax, 1e-12),  q = cast_fp8(clamp(x * scale, +-fp8_max)),
 *   scale_inv = 1 / scale,      fp8_max = 448 (E4M3), 57344 (E5M2: gradients of the HYBRID format),
 * all in fp32 (bf16 -> fp32 is exact), round to nearest even.  A NaN or Inf anywhere in the tensor makes every
 * code NaN. */

/* amax_f32[0] = max |x[i]| over n bf16 values (0 for n == 0); x 16-byte aligned. */
int mxl_amax(const void* x_bf16, int64_t n, void* amax_f32, void* stream);

/* mxl_quantize with the tensor's scale instead of block scales: codes in the same layouts (row-wise copy,
 * transposed segment-padded copy, row-major or K-chunk-major), fmt = MXL_FMT_E4M3 or MXL_FMT_E5M2, the scale
 * taken from amax_f32 (device, written by mxl_amax on the same stream).  s_row / s_colT receive the E8M0
 * byte 127 (2^0) for every block, so that the codes can be handed to the GEMMs below unchanged, and
 * scale_inv_f32[0] (device, may be NULL) receives 1 / scale. */
int mxl_quantize_tensorwise(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt,
                            const void* amax_f32, const int64_t* group_lens, int num_groups, void* q_row, void* s_row,
                            void* q_colT, void* s_colT, void* scale_inv_f32, uint32_t flags, void* stream);

/* The same for weights [batch, n, k] (both copies, layouts of mxl_quantize_weight_2d); one scale for the whole
 * tensor, amax_f32 taken over all of it. */
int mxl_quantize_weight_tensorwise(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld, int64_t n_ld,
                                   int fmt, const void* amax_f32, void* q_row, void* s_row, void* q_colT, void* s_colT,
                                   void* scale_inv_f32, uint32_t flags, void* stream);

/* The GEMMs with a per-tensor factor: c = (a . b^T) * alpha_a[0] * alpha_b[0] on the FP8 values of the codes, the
 * factors read on the device (the scale_inv outputs above), applied in fp32 before the rounding to bf16.  The operands
 * are what the two quantisers above write: their block scales are the unit byte by construction, so the scale arrays
 * are NOT read (they may be null); an operand with other block scales belongs to mxl_grouped_gemm_nt / _wgrad.
 * Operand formats: E4M3 x E4M3, E5M2 (a) x E4M3 (b), and E5M2 x E5M2, in every layout. */
int mxl_grouped_gemm_nt_scaled(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                               const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                               int num_groups, int64_t total_m, int64_t n, int64_t k, const float* alpha_a,
                               const float* alpha_b, uint32_t flags, void* stream);
int mxl_grouped_gemm_wgrad_scaled(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                  const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                  int num_groups, int64_t total_m, int64_t n, int64_t k, const float* alpha_a,
                                  const float* alpha_b, uint32_t flags, void* stream);

/* RMSNorm in front of the column-parallel linear (rmsnorm(x, layer_norm_weight, eps) in
 * PrimusTurboLayerNormColumnParallelLinear.forward_internal, primus_turbo.py:1689-1700):
 *   rstd[m] = 1 / sqrt(mean_j x[m, j]^2 + eps),   y[m, j] = (x[m, j] * rstd[m]) * w[j]
 * for bf16 x[rows, k], w[k]; fp32 arithmetic, y rounded once to bf16, rstd[rows] fp32 (kept for the backward).
 * y_bf16 may be NULL: then only rstd is written (what mxl_rmsnorm_quantize needs).  Requires k % 8 == 0 and
 * k <= 16384.  The sum of squares is taken in a fixed order, so results do not depend on the launch. */
int mxl_rmsnorm_fwd(const void* x_bf16, const void* w_bf16, float eps, int64_t rows, int64_t k, void* y_bf16,
                    void* rstd_f32, void* stream);

/* Backward of the above: dx[rows, k] (bf16) and dw[k] (bf16; zeros for rows == 0) from dy[rows, k].  The column
 * sums of dw go through `workspace`, at least mxl_rmsnorm_bwd_workspace_bytes(rows, k) bytes of device
 * memory, 16-byte aligned, owned by the caller (the library allocates nothing); its contents need no
 * initialisation and are dead after the call's kernels have run. */
int64_t mxl_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t k);
int mxl_rmsnorm_bwd(const void* dy_bf16, const void* x_bf16, const void* w_bf16, const void* rstd_f32, int64_t rows,
                    int64_t k, void* dx_bf16, void* dw_bf16, void* workspace, int64_t workspace_bytes, void* stream);

/* mxl_rmsnorm_bwd for callers that cannot allocate or hand over a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  Same arguments minus the
 * workspace, same kernels, same results bit for bit; the partial column sums go through a static device array of
 * mxl_rmsnorm_bwd_noalloc_max_bytes() = 8 MiB that every GPU the library runs on holds until the process ends.
 * A problem with mxl_rmsnorm_bwd_workspace_bytes(rows, k) above that returns MXL_ESCRATCH (e.g. k = 4096 with
 * more than 512 rows; k <= 1024 always fits).  Calls no hipMalloc / hipFree or other allocating routine.  All
 * calls on one GPU share the array, so two calls in flight at once would corrupt each other: per device the entry
 * point is BOUND TO ONE STREAM (calls on one stream are ordered) and returns MXL_ESTREAM, launching nothing, for any
 * other.  mxl_rmsnorm_bwd_noalloc_bind(stream) binds the current device's array to `stream` (and looks its address up,
 * once per device); the first call on an unbound device binds its own stream.  Rebinding is the caller's statement
 * that the work of the previous stream is finished or ordered in front of the new stream's.  A call on an unbound
 * device while `stream` is being captured returns MXL_ESTREAM: bind before the capture begins (a captured call
 * replays on whatever stream launches the graph; ordering replays against other users of the array is the caller's).
 * Nothing in the array has to be cleared between calls (every word read was written by the same call). */
int64_t mxl_rmsnorm_bwd_noalloc_max_bytes(void);
int mxl_rmsnorm_bwd_noalloc_bind(void* stream);
int mxl_rmsnorm_bwd_noalloc(const void* dy_bf16, const void* x_bf16, const void* w_bf16, const void* rstd_f32, int64_t rows,
                            int64_t k, void* dx_bf16, void* dw_bf16, void* stream);

/* The normalisation feeding the MX quantiser directly: what mxl_quantize would produce for
 * y = mxl_rmsnorm_fwd(x, w, ...) (bit for bit) from x, w and rstd (mxl_rmsnorm_fwd with y_bf16 = NULL), without
 * y reaching memory: the quantised copies are all the following GEMMs read.  The reference runs rmsnorm and the
 * quantisation inside gemm_fp8 / gemm_fp4 as separate kernels (primus_turbo.py:1689-1741).  The other arguments
 * are those of mxl_quantize with cols = k (k % 32 == 0); a row-wise copy must be requested.  flags: 0 or
 * MXL_QF_KCHUNK. */
int mxl_rmsnorm_quantize(const void* x_bf16, const void* w_bf16, const void* rstd_f32, int64_t rows, int64_t k,
                         int64_t row_ld, int fmt, int scale_mode, const int64_t* group_lens, int num_groups,
                         void* q_row, void* s_row, void* q_colT, void* s_colT, uint32_t flags, void* stream);

/* Expert groups padded to the quantisation alignment without a host read of the counts.  Replaces the
 * tokens_per_expert.tolist() + per-expert split / zero-append of the reference's expert MLP
 * (primus/backends/megatron/core/transformer/experts.py:196-209) and its inverse (:262-264); the alignment is the
 * reference's pad_multiple (primus/backends/megatron/core/extensions/primus_turbo.py:2344-2353: 32 for MX, else 16).
 *
 *   x           : [rows, row_bytes] bytes, rows of the groups back to back (sum(group_lens) == rows; rows of x the
 *                 counts do not cover are dropped)
 *   group_lens  : int64[num_groups] on the device, 1 <= num_groups <= 1024; negative counts read as 0
 *   out         : [out_rows, row_bytes]; group g starts at the sum of the padded lengths before it, holds its rows
 *                 and then zero rows up to a multiple of align; every row behind the last group's padding is a zero
 *                 row as well.  out_rows >= mxl_padded_rows_bound(rows, num_groups, align), the largest total the
 *                 counts can produce, since the host does not know them.
 *   padded_lens : int64[num_groups] (may be NULL): ceil(len / align) * align, the last one enlarged by the rows
 *                 behind its padding so that the lengths sum to out_rows exactly.
 *
 * mxl_unpad_groups is the inverse (and the gradient of mxl_pad_groups, as mxl_pad_groups is of it): row i of group
 * g of `out` [rows, row_bytes] is row i of that group in the padded `y` [padded_rows, row_bytes]; rows of `out`
 * behind sum(group_lens) are zero.  Any row_bytes >= 1; rows move 16 bytes per lane when pointers and row_bytes
 * are multiples of 16. */
int64_t mxl_padded_rows_bound(int64_t rows, int num_groups, int align);
int mxl_pad_groups(const void* x, int64_t rows, int64_t row_bytes, const int64_t* group_lens, int num_groups, int align,
                   void* out, int64_t out_rows, int64_t* padded_lens, void* stream);
int mxl_unpad_groups(const void* y, int64_t padded_rows, int64_t row_bytes, const int64_t* group_lens, int num_groups,
                     int align, void* out, int64_t rows, void* stream);

/* The 128-blockwise FP8 recipe (ScalingGranularity.BLOCKWISE with block_size 128: admitted by the reference's argument
 * validation, primus/backends/megatron/patches/args/rocm_arg_validation.py:145; operand flow of its
 * FP8LinearBlockwiseFunction, primus/backends/megatron/core/extensions/primus_turbo_float8_local.py:993-1089).
 * fmt is MXL_FMT_E4M3 or MXL_FMT_E5M2; every scale is an fp32 scale_inv = 1 / (fp8_max / max(amax, 1e-12)) of its block,
 * codes = cast(clamp(x * scale)), fp32 arithmetic (the formula the reference restates at :194-207, per block).
 *
 * mxl_quantize_blockwise replaces quant_fp8_blockwise_impl(x, dtype, axis, block_size = 128) (:1019, :1053-1059) and, with
 * group_lens, quant_fp8_blockwise_segment_m_row_col_impl (primus/backends/megatron/core/extensions/zbpp_gemm.py:633, :785):
 *   x          : bf16 [rows, cols], cols % 128 == 0, 16-byte aligned
 *   group_lens : int64[num_groups] on the device (<= 1024 groups) or NULL / 0: the rows of x are split into groups
 *   q_row      : [rows, cols] codes, 1 x 128 blocks along the columns (axis = 1 / -1); sinv_row fp32 [rows, cols / 128]
 *   q_colT     : the copy with 128 x 1 blocks along the rows (axis = 0 / -2), stored TRANSPOSED as the NT GEMM consumes
 *                it: [cols, W] codes, sinv_colT fp32 [cols, W / 128].  Without groups W = rows rounded up to 128; with
 *                groups W = mxl_padded_width(rows, num_groups) and group g owns columns [poff_g, poff_g + len_g), poff =
 *                prefix sum of the lens rounded up to 128, so the blocks restart at every group.  Padding: zero codes.
 *                Either copy may be left out (both pointers NULL).
 * mxl_quantize_blockwise_weight replaces quant_fp8_blockwise_for_weight_impl (:1020, :1060): w bf16 [batch, n, k], n and
 * k multiples of 128, one scale per 128 x 128 block; q [batch, n, k] with sinv [batch, n / 128, k / 128] and / or the
 * transposed copies q_T [batch, k, n] with sinv_T [batch, k / 128, n / 128] (the same scales, transposed).
 *
 * mxl_gemm_nt_blockwise replaces gemm_fp8_impl(..., granularity = BLOCKWISE) (:1022-1033, :1064-1087), always in NT
 * form on the copies above:  c[m, n] (bf16) = sum over kb of a_sinv[m, kb] * b_sinv[n / b_rows_per_scale, kb] *
 * (a[m, 128 kb ..] . b[n, 128 kb ..]), fp32 accumulation.  a [m, k] codes, b [n, k] codes, k % 128 == 0, n % 128 == 0;
 * b_rows_per_scale is 128 (b is a weight: b_sinv [n / 128, k / 128]) or 1 (b_sinv [n, k / 128], the wgrad GEMM, whose
 * two operands are transposed activation copies).  forward: a = q_row(X), b = q(W); dgrad: a = q_row(dY), b = q_T(W);
 * wgrad: a = q_colT(dY), b = q_colT(X), k = rows_pad.
 * mxl_grouped_gemm_nt_blockwise (grouped_gemm_fp8_impl with blockwise granularity, zbpp_gemm.py:608-630): the rows of
 * a [total_m, k] are split by group_lens, b is [num_groups, n, k] with b_sinv [num_groups, n / 128, k / 128].
 * mxl_grouped_gemm_wgrad_blockwise (grouped_gemm_fp8_variable_k_impl, zbpp_gemm.py:757-800): a = q_colT(dY) [n, W],
 * b = q_colT(X) [k, W] with their per-row factors, c [num_groups, n, k]; a group without tokens yields zeros. */
int mxl_quantize_blockwise(const void* x_bf16, int64_t rows, int64_t cols, int fmt, const int64_t* group_lens, int num_groups,
                           void* q_row, void* sinv_row, void* q_colT, void* sinv_colT, void* stream);
int mxl_quantize_blockwise_weight(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int fmt, void* q, void* sinv,
                                  void* q_T, void* sinv_T, void* stream);
int mxl_gemm_nt_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv,
                          int b_fmt, int b_rows_per_scale, void* c_bf16, int64_t m, int64_t n, int64_t k, void* stream);
int mxl_grouped_gemm_nt_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv,
                                  int b_fmt, void* c_bf16, const int64_t* group_lens, int num_groups, int64_t total_m,
                                  int64_t n, int64_t k, void* stream);
int mxl_grouped_gemm_wgrad_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv,
                                     int b_fmt, void* c_bf16, const int64_t* group_lens, int num_groups, int64_t total_m,
                                     int64_t n, int64_t k, void* stream);
/* The blockwise GEMMs run on output tiles of 128 x 256 or 256 x 256 and pick by the shape (256 rows unless that leaves
 * more of the chip idle than it gains; same bits either way).  mxl_blockwise_gemm_tile(128 / 256) forces one for every later
 * call of the process, 0 returns to the choice by shape: a measuring and testing aid without counterpart in the
 * reference.  MXL_EINVAL for any other value. */
int mxl_blockwise_gemm_tile(int rows);
/* What the choice by shape comes to (a host-side calculation, no GPU needed; no counterpart in the reference): the 256-row
 * tiles take rows [0, *tall_rows) x columns [0, *tall_cols) of an m x n output, the 128-row tiles the rest (the last rows
 * or the last columns of a dense GEMM, in a second launch; 0 x 0: everything on 128-row tiles).  mode 0: dense, 1: grouped
 * forward / dgrad (m = total rows), 2: grouped weight gradient (m, n = rows and columns of one group's matrix). */
int mxl_blockwise_gemm_plan(int64_t m, int64_t n, int mode, int num_groups, int64_t* tall_rows, int64_t* tall_cols);

/* ---- pre-shuffled MXFP4 layouts ----
 *
 * The byte orders behind the shuffle_rowwise / shuffle_colwise (codes) and shuffle_*_scale flags of the reference's
 * quantize_mxfp4_dual (primus_turbo_mxfp4_local.py:147-161; output shapes :184-198) and behind
 * gemm_fp4_impl(..., preshuffled=True) (:319-331), which the reference describes as the AITER pre-shuffle path.
 * mxl_shuffle_codes:  packed FP4 codes [rows, row_bytes], rows % 16 == 0, row_bytes % 32 == 0, same shape out: every
 *   block of 16 rows x 32 bytes becomes 512 consecutive bytes ([16-byte half][row][byte]), blocks in row-major order.
 * mxl_shuffle_scales: E8M0 bytes [rows, cols] -> [ceil(rows / 256) * 256, ceil(cols / 8) * 8] with zero bytes in the
 *   padding: every 32 rows x 8 columns become 256 consecutive bytes ([col % 4][row % 16][(col / 4) % 2][(row / 16) % 2]).
 * inverse != 0 converts back (src is the shuffled array, dst [rows, row_bytes] / [rows, cols]).  src and dst must not
 * overlap; code arrays must be 16-byte aligned.  The GEMMs read pre-shuffled weight CODES as they lie
 * (MXL_GF_B_SHUFFLED); pre-shuffled SCALES (1/16 of the bytes of the codes) are converted back first, which the
 * Python boundary does.  The byte orders are restated from AITER's published shuffle_weight(layout=(16, 16)) and
 * e8m0_shuffle; the reference tree holds neither their source nor a fixture, so the orders are parity unpinned
 * (the array shapes are pinned by primus_turbo_mxfp4_local.py:184-198). */
int mxl_shuffle_codes(const void* src, int64_t rows, int64_t row_bytes, void* dst, int inverse, void* stream);
int mxl_shuffle_scales(const void* src, int64_t rows, int64_t cols, void* dst, int inverse, void* stream);

/* ---- calibration (no counterpart in the reference: a measuring aid of this library's benchmark) ----
 *
 * mxl_calibrate_mfma launches a register-only loop of the GEMM kernels' scaled MFMA (32 x 32 x 64; a_fmt / b_fmt:
 * MXL_FMT_E4M3 or MXL_FMT_E2M1) on 256 workgroups of 4 waves, `iters` K steps of 16 MFMAs per wave, with no memory
 * traffic at all: its rate is what the matrix cores of the board sustain under its power limit, the ceiling for any
 * GEMM on it.  mxl_calibrate_mfma_flops(iters) = the floating-point operations of one such launch. */
int mxl_calibrate_mfma(int a_fmt, int b_fmt, int64_t iters, void* stream);
/* mxl_calibrate_tile_copy moves the bytes of the dual MXFP8 quantiser without its arithmetic: x [rows, cols] bf16 read
 * in 128 x 128 tiles, one byte per element written to out_row [rows, cols] and one to out_colT [cols, rows] (either may
 * be null: read + one output, or read only), tiles in the quantiser's order; rows and cols multiples of 128.  Its rate
 * is what that access pattern reaches on the board. */
int mxl_calibrate_tile_copy(const void* in_bf16, int64_t rows, int64_t cols, void* out_row, void* out_colT, void* stream);
int64_t mxl_calibrate_mfma_flops(int64_t iters);
/* The same loop for the bf16 MFMA of the unquantised grouped GEMM (32 x 32 x 16, 32 per iteration and wave). */
int mxl_calibrate_mfma_bf16(int64_t iters, void* stream);
int64_t mxl_calibrate_mfma_bf16_flops(int64_t iters);
/* mxl_calibrate_range_check makes the hardware rule observable on which the GEMM kernels' operand requests rely (a
 * request for rows past the end of an operand must read nothing): for each of num_cases triples of uint32
 * {voffset, soffset, num_records} (device array `cases`) one LDS-direct 16-byte buffer load goes through a raw
 * descriptor over `buf` with that num_records, per-lane offset and scalar offset, and out[4 i .. 4 i + 3] (uint32,
 * device) receives the four dwords that arrived -- zeros where the range check dropped them.  max_offset_host = the
 * largest voffset + soffset of the cases as the caller states it; the call is refused unless that plus 16 fits
 * buf_bytes, so no case can leave `buf` whatever the hardware decides. */
int mxl_calibrate_range_check(const void* buf, int64_t buf_bytes, const void* cases, int num_cases, void* out,
                              int64_t max_offset_host, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MXLINEAR_H */
