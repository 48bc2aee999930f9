// MX quantisers for gfx950: bf16 -> {E4M3, E2M1} codes + E8M0 block scales.
//
// One kernel family covers the three layouts the linear path needs
// (primus_turbo.py:321-354, primus_turbo_mxfp4_local.py:147-207):
//   ROW  : blocks of 32 along the columns, output in the input's orientation;
//   COL  : blocks of 32 along the rows, output TRANSPOSED, blocks restarting at
//          every expert boundary, each expert segment padded to 128;
//   TWOD : one scale per 32x32 tile (weights), both copies from one scale.
//
// A workgroup (256 threads, 4 waves) owns a 128x128 tile.  Wave w owns rows
// [32w, 32w+32) -- exactly one column-wise MX block -- and each lane loads
// 8 rows x 8 columns as eight 16-byte loads, so a 16-lane group reads 256
// contiguous bytes.  Row-block maxima are reduced over 4 adjacent lanes with
// DPP, column-block maxima in registers over the lane's 8 rows and then over
// the 4 lane groups.  The transposed codes go through an LDS tile so that the
// global stores are 128 contiguous bytes per output row.
#include "mx_device.h"

namespace mxl {

constexpr int QT = 128;       // tile edge
constexpr int QTHREADS = 256;

struct QuantArgs {
    const uint16_t* x;
    int64_t rows, cols;
    const int64_t* group_lens;
    int num_groups;
    uint8_t* q_row;
    uint8_t* s_row;
    uint8_t* q_colT;
    uint8_t* s_colT;
    int64_t row_ld;     // columns of the row-wise copy (>= cols; the excess is zero-filled padding)
    int64_t W;          // padded width of the transposed copy (elements)
    int64_t mat_rows;   // TWOD: rows per matrix (n); otherwise unused
    // fused gated activation in front (ACT >= 0): x is fc1's output [rows, 2 * cols], the tensor that is
    // quantised is act(x[:, :cols]) * x[:, cols:] * probs[row], masked rows are zero
    const void* probs;
    int probs_bf16;
    const uint8_t* row_mask;
    // fused RMSNorm in front (ACT == PRO_RMSNORM): the tensor that is quantised is (x * rstd[row]) * norm_w[col];
    // rstd travels in `probs` (fp32)
    const uint16_t* norm_w;
    // tensor-wise scaling (SMODE == SCALE_TENSOR): one fp32 scale for the whole tensor, fp8_max / max(amax, 1e-12),
    // from the tensor's abs-max on the device; its reciprocal is written to scale_inv_out (may be null).  The
    // block-scale arrays are filled with 127 (2^0), so the scaled GEMM reads the codes unchanged.
    const float* tensor_amax;
    float* scale_inv_out;
    // Code layout of both copies.  0: row-major [rows, ld].  1: K-chunk-major [ld / 128][rows][128 elements]:
    // the 128 elements of a row that one GEMM K slot consumes stay together and consecutive rows follow
    // each other, so a GEMM tile's slot is one contiguous block and this kernel writes 128 x 128-element
    // pieces contiguously.  chunk_rows_row / chunk_rows_col: rows of the whole row-wise / transposed operand.
    // 2: K-step-major (FP8 only): codes [ld / 64][rows][64], scales [ceil(ld / 512)][rows][16].
    int kchunk;
    int64_t chunk_rows_row, chunk_rows_col;
    uint64_t sr_seed;       // SR kernels: seed of the stochastic rounding
    uint32_t rht_signs;     // RHT kernels: sign bit i flips row i of every 16-row group before the transform
    int tiles_r, tiles_c;   // tile grid: row tiles (upper bound when grouped) x column tiles
    int super_c, n_super;   // 8x8-tile supertiles: count along the columns, total
};

// Workgroup -> tile.  Workgroups are dealt to the 8 XCDs round robin, so workgroup L is the
// (L / 8)-th one of XCD L % 8.  Each XCD walks whole 8x8-tile supertiles, column tile fastest:
//  - the 4-byte scale pieces that 8 neighbouring tiles write (32 contiguous bytes, along the columns
//    for the row-wise copy and along the rows for the transposed one) meet in one L2 and leave it as
//    one write instead of eight partial ones;
//  - the workgroups resident at any moment cover long contiguous row spans instead of one 256-byte
//    column slice at a power-of-two stride, which would camp on a few memory channels.
constexpr int QSUPER = 8;
__device__ __forceinline__ bool quant_tile_of_workgroup(const QuantArgs& a, int& pt, int& ct) {
    const int L = blockIdx.x, xcd = L & 7, k = L >> 3;
    const int s = (k / (QSUPER * QSUPER)) * 8 + xcd;
    if (s >= a.n_super) return false;
    const int within = k % (QSUPER * QSUPER);
    pt = (s / a.super_c) * QSUPER + within / QSUPER;
    ct = (s % a.super_c) * QSUPER + within % QSUPER;
    return pt < a.tiles_r && ct < a.tiles_c;
}

// SR (E2M1 only): codes are rounded stochastically instead of to nearest even; scales are unaffected.
// The random word of a pair of neighbouring elements is a function of the seed and of the pair's
// position in the OUTPUT (row-wise copy: row, column pair; transposed copy: column, position pair
// along the padded token axis), so the result does not depend on the tiling.
//
// RHT: the transposed copy is taken from a randomised Hadamard transform of the input along the token
// axis (colwise_use_rht of quantize_mxfp4_dual, primus_turbo_mxfp4_local.py:234-250,272-288): every
// group of 16 consecutive token positions of an expert's segment becomes (1/4) H16 (s * x), H16 the
// Sylvester matrix and s the sign vector `rht_signs`, evaluated as four fp32 butterfly stages (strides
// 1, 2, 4, 8) and rounded once to bf16; that tensor is then quantised like any other.  The transform is
// orthogonal, so a wgrad GEMM whose two operands were both transformed computes the same contraction
// while single large values are spread over 16 positions before they meet the 4-bit grid.
constexpr int PRO_RMSNORM = 2;   // value of ACT next to MXL_ACT_SILU (0) and MXL_ACT_GELU (1)
constexpr int SCALE_TENSOR = 3;  // value of SMODE next to the three E8M0 rules: per-tensor fp32 scale

template <int FMT, int SMODE> __device__ __forceinline__ uint32_t block_byte(uint32_t amax16) {
    if constexpr (SMODE == SCALE_TENSOR) {
        return 127u;
    } else {
        return scale_byte<FMT, SMODE>(amax16);
    }
}

// K-step-major scales: a row's 16 bytes of a panel (512 elements = 8 MFMA K steps of two blocks) are ordered
// [block parity][K step], so that the 8 bytes a GEMM lane needs for the panel's 8 steps are adjacent (the lanes
// 0-31 of an MFMA supply the scales of the even blocks, the lanes 32-63 those of the odd ones).  `v` = the scale
// bytes of the four blocks of 128-element tile `quarter` of the panel.
__device__ __forceinline__ void store_panel_scales(uint8_t* row16, int quarter, uint32_t v) {
    *(uint16_t*)(row16 + 2 * quarter) = (uint16_t)((v & 0xFFu) | ((v >> 8) & 0xFF00u));
    *(uint16_t*)(row16 + 8 + 2 * quarter) = (uint16_t)(((v >> 8) & 0xFFu) | ((v >> 16) & 0xFF00u));
}

template <int FMT, int SMODE, bool ROW, bool COL, bool TWOD, int ACT = -1, bool SR = false, bool RHT = false>
__global__ __launch_bounds__(QTHREADS) void mx_quant_kernel(QuantArgs a) {
    constexpr bool FP4 = (FMT == kFmtE2M1);
    constexpr bool TENSOR = (SMODE == SCALE_TENSOR);
    static_assert(TENSOR || FMT != kFmtE5M2, "E5M2 exists for tensor-wise scaling only");
    static_assert(!TENSOR || (!FP4 && !SR && !RHT && ACT < 0), "tensor-wise scaling: FP8 codes, plain input");
    static_assert(!SR || (FP4 && !TWOD && ACT < 0), "stochastic rounding exists for 1-D E2M1 quantisation only");
    static_assert(!RHT || (COL && !TWOD && ACT < 0), "the Hadamard transform applies to the transposed 1-D copy only");
    constexpr int TPITCH = FP4 ? (QT / 2 + 16) : (QT + 16);  // bytes per LDS row of the transposed tile
    __shared__ __attribute__((aligned(16))) uint8_t t_tile[COL ? QT * TPITCH : 16];
    __shared__ uint32_t srow_tile[QT];
    __shared__ uint32_t scol_tile[QT];

    const int t = threadIdx.x;
    const int w = t >> 6, l = t & 63, c16 = l & 15, rg = l >> 4;
    float tscale = 1.f;
    bool tensor_bad = false;   // abs-max is NaN or Inf: every code becomes NaN
    if (TENSOR) {
        const float amax = *a.tensor_amax;
        tensor_bad = !(amax < __uint_as_float(0x7F800000u));
        tscale = (FMT == kFmtE5M2 ? 57344.f : 448.f) / fmaxf(amax, 1e-12f);
        if (blockIdx.x == 0 && t == 0 && a.scale_inv_out) *a.scale_inv_out = 1.0f / tscale;
    }
    int pt, ct;
    if (!quant_tile_of_workgroup(a, pt, ct)) return;   // uniform over the workgroup
    const int64_t col0 = (int64_t)ct * QT;

    // ---- which source rows does this tile hold? ----
    int64_t src_row0 = 0;
    int rows_valid = 0;
    int64_t batch_off_rows = 0;  // TWOD: first row of this matrix in the flattened input
    // K-step-major scales of a grouped transposed copy: the 16-byte scale panels restart at every group
    int64_t seg_pan0 = 0;        // panels of the groups in front of this tile's group
    int seg_tile = -1;           // this tile's number inside its group's padded segment (-1: not grouped)
    if (TWOD) {
        // grid.x enumerates (matrix, row tile); matrices are independent.
        const int tiles_per_mat = (int)((a.mat_rows + QT - 1) / QT);
        const int mat = pt / tiles_per_mat, rt = pt % tiles_per_mat;
        batch_off_rows = (int64_t)mat * a.mat_rows;
        src_row0 = batch_off_rows + (int64_t)rt * QT;
        int64_t rem = a.mat_rows - (int64_t)rt * QT;
        rows_valid = rem < QT ? (int)rem : QT;
    } else if (!COL || a.group_lens == nullptr) {
        src_row0 = (int64_t)pt * QT;
        int64_t rem = a.rows - src_row0;
        rows_valid = rem <= 0 ? 0 : (rem < QT ? (int)rem : QT);
    } else {
        int64_t off = 0, ppo = 0;
        int pto = 0;
        for (int g = 0; g < a.num_groups; ++g) {
            // clamped to the rows that exist, so that lens which do not match the buffer cannot read outside it
            int64_t len = a.group_lens[g];
            len = len < 0 ? 0 : (len > a.rows - off ? a.rows - off : len);
            const int nt = (int)((len + QT - 1) / QT);
            if (pt < pto + nt) {
                const int64_t r = (int64_t)(pt - pto) * QT;
                src_row0 = off + r;
                rows_valid = (len - r) < QT ? (int)(len - r) : QT;
                seg_pan0 = ppo;
                seg_tile = pt - pto;
                break;
            }
            off += len;
            pto += nt;
            ppo += (nt + 3) / 4;
        }
        if (seg_tile < 0) {   // a padding tile behind the last group: its scales go behind the last group's panels
            seg_pan0 = ppo;
            seg_tile = pt - pto;
        }
    }

    // fused activation: the tile's 128 probabilities (and row-mask bits) are fetched once by 128 lanes and
    // handed round through LDS; fetched per lane and row they would double the number of load instructions
    __shared__ float prob_tile[ACT >= 0 ? QT : 1];
    __shared__ uint8_t live_tile[ACT >= 0 ? QT : 1];
    float my_rstd = 0.f;
    if (ACT == PRO_RMSNORM) {
        // only requested here; it is handed round after the tile's own loads have gone out
        if (t < QT && t < rows_valid) my_rstd = ((const float*)a.probs)[src_row0 + t];
    } else if (ACT >= 0) {
        if (t < QT) {
            const bool live = t < rows_valid && (a.row_mask == nullptr || a.row_mask[src_row0 + t] != 0);
            live_tile[t] = live ? 1 : 0;
            prob_tile[t] = live ? load_prob(a.probs, a.probs_bf16, src_row0 + t) : 0.f;
        }
        __syncthreads();
    }

    const int64_t col = col0 + 8 * c16;
    const bool col_ok = col < a.cols;      // source column exists
    const bool out_ok = col < a.row_ld;    // row-wise output column exists (padding is written as zeros)

    // ---- load 8 rows x 8 columns per lane ----
    uint4 d[8];
    uint4 norm_wv = make_uint4(0, 0, 0, 0);
    if (ACT == PRO_RMSNORM && col_ok) norm_wv = *(const uint4*)(a.norm_w + col);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int r = 32 * w + 8 * rg + it;
        d[it] = make_uint4(0, 0, 0, 0);
        if (col_ok && r < rows_valid) {
            if (ACT < 0) {
                d[it] = load16_streaming(a.x + (src_row0 + r) * a.cols + col);
            } else if (ACT == PRO_RMSNORM) {
                d[it] = load16_streaming(a.x + (src_row0 + r) * a.cols + col);
            } else {
                if (live_tile[r]) {
                    const uint16_t* xr = a.x + (src_row0 + r) * 2 * a.cols + col;
                    d[it] = glu8<(ACT == MXL_ACT_GELU ? MXL_ACT_GELU : MXL_ACT_SILU)>(load16_streaming(xr),
                                                                                      load16_streaming(xr + a.cols),
                                                                                      prob_tile[r]);
                }
            }
        }
    }

    if (ACT == PRO_RMSNORM) {
        if (t < QT) prob_tile[t] = my_rstd;
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = 32 * w + 8 * rg + it;
            if (col_ok && r < rows_valid) d[it] = norm8(d[it], norm_wv, prob_tile[r]);
        }
    }

    // ---- block maxima ----
    uint32_t rmax[8];  // per row: max over the lane's 8 columns, then over the 32-column block
    uint32_t cmax[4] = {0, 0, 0, 0};  // per column pair (packed): max over the lane's 8 rows
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const uint32_t p0 = d[it].x & 0x7FFF7FFFu, p1 = d[it].y & 0x7FFF7FFFu, p2 = d[it].z & 0x7FFF7FFFu,
                       p3 = d[it].w & 0x7FFF7FFFu;
        if (COL && !TWOD && !RHT) {
            cmax[0] = pk_max16(cmax[0], p0);
            cmax[1] = pk_max16(cmax[1], p1);
            cmax[2] = pk_max16(cmax[2], p2);
            cmax[3] = pk_max16(cmax[3], p3);
        }
        uint32_t m = pk_max16(pk_max16(p0, p1), pk_max16(p2, p3));
        m = hmax16(m);
        m = max(m, dpp_xor1(m));
        m = max(m, dpp_xor2(m));
        rmax[it] = m;
    }
    uint32_t tile_byte = 0;
    if (TWOD) {
        uint32_t m = rmax[0];
#pragma unroll
        for (int it = 1; it < 8; ++it) m = max(m, rmax[it]);
        m = max(m, (uint32_t)__shfl_xor((int)m, 16));
        m = max(m, (uint32_t)__shfl_xor((int)m, 32));
        tile_byte = block_byte<FMT, SMODE>(m);
        // the transposed copy's scales without its codes: the tile's byte for each of the lane's 8 columns
        if (!COL && a.s_colT != nullptr && rg == 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) ((uint8_t*)scol_tile)[(8 * c16 + j) * 4 + w] = (uint8_t)tile_byte;
        }
    } else if (COL && !RHT) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 16));
            cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 32));
        }
    }

    // ---- row-wise copy ----
    if (ROW) {
        uint2 o_even = make_uint2(0u, 0u);   // FP8: codes of the even row of a row pair, kept until its partner is done
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = 32 * w + 8 * rg + it;
            const uint32_t byte = TWOD ? tile_byte : block_byte<FMT, SMODE>(rmax[it]);
            if ((c16 & 3) == 0) ((uint8_t*)srow_tile)[r * 4 + (c16 >> 2)] = (uint8_t)byte;
            if (!FP4) {
                uint2 o;
                if (TENSOR) {
                    o.x = tensor_bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(d[it].x, d[it].y, tscale);
                    o.y = tensor_bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(d[it].z, d[it].w, tscale);
                } else if (byte != 255u) {
                    const float inv = inv_scale(byte);
                    o.x = cvt4_e4m3(d[it].x, d[it].y, inv);
                    o.y = cvt4_e4m3(d[it].z, d[it].w, inv);
                } else {
                    o.x = nonfinite4_e4m3(d[it].x, d[it].y);
                    o.y = nonfinite4_e4m3(d[it].z, d[it].w);
                }
                // Two rows at a time, 16 bytes per lane: a lane pair swaps one 8-byte piece, after which the even lane
                // holds 16 consecutive codes of the even row and the odd lane 16 of the odd row.  Half the store
                // instructions, and in the K-step-major layout (64-byte row pieces, two rows to a cache line) an
                // instruction then writes whole lines.
                if ((it & 1) == 0) {
                    o_even = o;
                } else {
                    const bool odd = (c16 & 1) != 0;
                    const uint2 send = odd ? o_even : o;
                    const uint2 recv = make_uint2(dpp_xor1(send.x), dpp_xor1(send.y));
                    const uint4 out = odd ? make_uint4(recv.x, recv.y, o.x, o.y) : make_uint4(o_even.x, o_even.y, recv.x, recv.y);
                    const int rr = odd ? r : r - 1;
                    const int cc = c16 & ~1;          // the pair's first 8-column piece
                    if (out_ok && rr < rows_valid) {
                        const int64_t at = a.kchunk == 2 ? ((int64_t)(2 * ct + (cc >> 3)) * a.chunk_rows_row + src_row0 + rr) * (QT / 2) + 8 * (cc & 7)
                                         : a.kchunk  ? ((int64_t)ct * a.chunk_rows_row + src_row0 + rr) * QT + 8 * cc
                                                     : (src_row0 + rr) * a.row_ld + col0 + 8 * cc;
                        store16_streaming(a.q_row + at, out);
                    }
                }
            } else {
                uint32_t o;
                if (SR && byte != 255u) {
                    const float inv = inv_scale(byte);
                    const uint64_t key = (uint64_t)(src_row0 + r) * (uint64_t)(a.cols >> 1) + (uint64_t)(col >> 1);
                    o = sr2_e2m1(d[it].x, inv, sr_word(key, a.sr_seed, 0)) |
                        (sr2_e2m1(d[it].y, inv, sr_word(key + 1, a.sr_seed, 0)) << 8) |
                        (sr2_e2m1(d[it].z, inv, sr_word(key + 2, a.sr_seed, 0)) << 16) |
                        (sr2_e2m1(d[it].w, inv, sr_word(key + 3, a.sr_seed, 0)) << 24);
                } else if (byte != 255u) {
                    const float sc = fwd_scale(byte);
                    o = cvt2_e2m1(d[it].x, sc) | (cvt2_e2m1(d[it].y, sc) << 8) | (cvt2_e2m1(d[it].z, sc) << 16) |
                        (cvt2_e2m1(d[it].w, sc) << 24);
                } else {
                    o = nonfinite2_e2m1(d[it].x) | (nonfinite2_e2m1(d[it].y) << 8) | (nonfinite2_e2m1(d[it].z) << 16) |
                        (nonfinite2_e2m1(d[it].w) << 24);
                }
                if (out_ok && r < rows_valid) {
                    // element offsets; K-step-major: 64 elements (32 bytes) of a row per K step
                    const int64_t at = a.kchunk == 2 ? ((int64_t)(2 * ct + (c16 >> 3)) * a.chunk_rows_row + src_row0 + r) * (QT / 2) + 8 * (c16 & 7)
                                     : a.kchunk ? ((int64_t)ct * a.chunk_rows_row + src_row0 + r) * QT + 8 * c16
                                                : (src_row0 + r) * a.row_ld + col;
                    store4_streaming(a.q_row + at / 2, o);
                }
            }
        }
    }

    // ---- Hadamard transform along the rows, in place (the row-wise copy above used the plain input) ----
    if (RHT) {
        // a 16-row group = the 8 rows of this lane and the 8 rows of the lane 16 further (rg ^ 1)
        const uint32_t upper = rg & 1;
        uint32_t* tw = (uint32_t*)d;
#pragma unroll
        for (int j2 = 0; j2 < 4; ++j2) {
            float lo[8], hi[8];
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const uint32_t flip = ((a.rht_signs >> (8 * upper + it)) & 1u) ? 0x80008000u : 0u;
                const uint32_t v = tw[it * 4 + j2] ^ flip;
                lo[it] = bf16_lo(v);
                hi[it] = bf16_hi(v);
            }
#pragma unroll
            for (int st = 1; st < 8; st <<= 1) {
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    if (it & st) continue;
                    const float a0 = lo[it], b0 = lo[it + st], a1 = hi[it], b1 = hi[it + st];
                    lo[it] = a0 + b0;
                    lo[it + st] = a0 - b0;
                    hi[it] = a1 + b1;
                    hi[it + st] = a1 - b1;
                }
            }
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const float o0 = __shfl_xor(lo[it], 16), o1 = __shfl_xor(hi[it], 16);
                const float r0 = upper ? (o0 - lo[it]) : (lo[it] + o0);
                const float r1 = upper ? (o1 - hi[it]) : (hi[it] + o1);
                tw[it * 4 + j2] = pack_bf16(r0 * 0.25f, r1 * 0.25f);
            }
        }
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            cmax[0] = pk_max16(cmax[0], d[it].x & 0x7FFF7FFFu);
            cmax[1] = pk_max16(cmax[1], d[it].y & 0x7FFF7FFFu);
            cmax[2] = pk_max16(cmax[2], d[it].z & 0x7FFF7FFFu);
            cmax[3] = pk_max16(cmax[3], d[it].w & 0x7FFF7FFFu);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 16));
            cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 32));
        }
    }

    // ---- column-wise (transposed) copy into the LDS tile ----
    if (COL) {
        const uint32_t* dw = (const uint32_t*)d;  // dw[it*4 + j]: columns 2j, 2j+1 of row `it`
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t amax = (j & 1) ? (cmax[j >> 1] >> 16) : (cmax[j >> 1] & 0xFFFFu);
            const uint32_t byte = TWOD ? tile_byte : block_byte<FMT, SMODE>(amax);
            const int c = 8 * c16 + j;
            if (rg == 0) ((uint8_t*)scol_tile)[c * 4 + w] = (uint8_t)byte;
            // the lane's 8 rows of column j, as 4 packed (row 2i, row 2i+1) pairs
            uint32_t pr[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t lo = dw[(2 * i) * 4 + (j >> 1)], hi = dw[(2 * i + 1) * 4 + (j >> 1)];
                pr[i] = (j & 1) ? ((lo >> 16) | (hi & 0xFFFF0000u)) : ((lo & 0xFFFFu) | (hi << 16));
            }
            if (!FP4) {
                uint2 o;
                if (TENSOR) {
                    o.x = tensor_bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(pr[0], pr[1], tscale);
                    o.y = tensor_bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(pr[2], pr[3], tscale);
                } else if (byte != 255u) {
                    const float inv = inv_scale(byte);
                    o.x = cvt4_e4m3(pr[0], pr[1], inv);
                    o.y = cvt4_e4m3(pr[2], pr[3], inv);
                } else {
                    o.x = nonfinite4_e4m3(pr[0], pr[1]);
                    o.y = nonfinite4_e4m3(pr[2], pr[3]);
                }
                *(uint2*)(t_tile + c * TPITCH + 32 * w + 8 * rg) = o;
            } else {
                uint32_t o;
                if (SR && byte != 255u) {
                    const float inv = inv_scale(byte);
                    const uint64_t pos = (uint64_t)pt * QT + (uint64_t)(32 * w + 8 * rg);   // along the padded token axis
                    const uint64_t key = (uint64_t)(col0 + c) * (uint64_t)(a.W >> 1) + (pos >> 1);
                    o = sr2_e2m1(pr[0], inv, sr_word(key, a.sr_seed, 1)) |
                        (sr2_e2m1(pr[1], inv, sr_word(key + 1, a.sr_seed, 1)) << 8) |
                        (sr2_e2m1(pr[2], inv, sr_word(key + 2, a.sr_seed, 1)) << 16) |
                        (sr2_e2m1(pr[3], inv, sr_word(key + 3, a.sr_seed, 1)) << 24);
                } else if (byte != 255u) {
                    const float sc = fwd_scale(byte);
                    o = cvt2_e2m1(pr[0], sc) | (cvt2_e2m1(pr[1], sc) << 8) | (cvt2_e2m1(pr[2], sc) << 16) |
                        (cvt2_e2m1(pr[3], sc) << 24);
                } else {
                    o = nonfinite2_e2m1(pr[0]) | (nonfinite2_e2m1(pr[1]) << 8) | (nonfinite2_e2m1(pr[2]) << 16) |
                        (nonfinite2_e2m1(pr[3]) << 24);
                }
                *(uint32_t*)(t_tile + c * TPITCH + (32 * w + 8 * rg) / 2) = o;
            }
        }
    }
    __syncthreads();

    // ---- scales: one dword (4 blocks) per row / per column of the tile ----
    if (ROW && t < QT && t < rows_valid) {
        const int64_t sld = a.row_ld / 32;
        const int64_t nb = (a.row_ld - col0) / 32;  // valid blocks in this tile row
        uint8_t* dst = a.s_row + (src_row0 + t) * sld + col0 / 32;
        const uint32_t v = srow_tile[t];
        if (a.kchunk >= 2) {
            store_panel_scales(a.s_row + ((int64_t)(ct >> 2) * a.chunk_rows_row + src_row0 + t) * 16, ct & 3, v);
        } else if (nb >= 4 && (sld & 3) == 0) {
            *(uint32_t*)dst = v;
        } else {
            for (int b = 0; b < 4 && b < nb; ++b) dst[b] = (uint8_t)(v >> (8 * b));
        }
    }
    if (COL || (TWOD && a.s_colT != nullptr)) {
        const int64_t out_rows_base = TWOD ? (batch_off_rows / a.mat_rows) * a.cols : 0;  // TWOD: matrix * k
        const int64_t m0 = TWOD ? (src_row0 - batch_off_rows) : (int64_t)pt * QT;          // position along W
        if (t < QT && col0 + t < a.cols) {
            uint8_t* dst = a.s_colT + (out_rows_base + col0 + t) * (a.W / 32) + m0 / 32;
            const uint32_t v = scol_tile[t];
            const int64_t nb = (a.W - m0) / 32;
            if (a.kchunk >= 2) {
                const int64_t mt = seg_tile >= 0 ? (int64_t)seg_tile : m0 / QT;
                store_panel_scales(a.s_colT + ((seg_pan0 + mt / 4) * a.chunk_rows_col + out_rows_base + col0 + t) * 16, (int)(mt & 3), v);
            } else if (nb >= 4 && ((a.W / 32) & 3) == 0) {
                *(uint32_t*)dst = v;
            } else {
                for (int b = 0; b < 4 && b < nb; ++b) dst[b] = (uint8_t)(v >> (8 * b));
            }
        }
        if (!COL) return;                        // (scales only)
        constexpr int ROWB = FP4 ? QT / 2 : QT;  // bytes per transposed tile row
        constexpr int LPR = ROWB / 16;           // lanes per row
        const int64_t wbytes = FP4 ? a.W / 2 : a.W;
        const int64_t m0b = FP4 ? m0 / 2 : m0;
        const int64_t avail = wbytes - m0b;      // bytes left in the output row (TWOD tails)
#pragma unroll
        for (int i = 0; i < QT / (QTHREADS / LPR); ++i) {
            const int c = t / LPR + i * (QTHREADS / LPR);
            const int ch = t % LPR;
            if (col0 + c < a.cols && 16 * ch < avail) {
                const uint4 v = *(const uint4*)(t_tile + c * TPITCH + 16 * ch);
                const int64_t at = (FP4 && a.kchunk == 2)
                                       ? ((2 * (m0 / QT) + (ch >> 1)) * a.chunk_rows_col + out_rows_base + col0 + c) * (QT / 4) + 16 * (ch & 1)
                                   : a.kchunk == 2
                                       ? ((2 * (m0 / QT) + (ch >> 2)) * a.chunk_rows_col + out_rows_base + col0 + c) * (QT / 2) + 16 * (ch & 3)
                                   : a.kchunk ? ((m0 / QT) * a.chunk_rows_col + out_rows_base + col0 + c) * ROWB + 16 * ch
                                              : (out_rows_base + col0 + c) * wbytes + m0b + 16 * ch;
                store16_streaming(a.q_colT + at, v);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// dequantise: codes + scales -> bf16 (row-wise layout)
// ---------------------------------------------------------------------------
__device__ __forceinline__ float dec_e4m3(uint32_t c) {
    // exact decode through fp32 bit assembly
    const uint32_t s = (c & 0x80u) << 24, e = (c >> 3) & 0xFu, m = c & 7u;
    float v;
    if (e == 0)
        v = (float)m * 0.001953125f;  // m * 2^-9
    else if ((c & 0x7Fu) == 0x7Fu)
        v = __uint_as_float(0x7FC00000u);
    else
        v = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return __uint_as_float(__float_as_uint(v) | s);
}
// E5M2 is the upper byte of an IEEE half: exact through the half -> float conversion (NaN and infinity included)
__device__ __forceinline__ float dec_e5m2(uint32_t c) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)(c << 8));
}
__device__ __forceinline__ float dec_e2m1(uint32_t c) {
    const uint32_t s = (c & 8u) << 28, e = (c >> 1) & 3u, m = c & 1u;
    const uint32_t bits = e ? (((e + 126u) << 23) | (m << 22)) : (m ? 0x3F000000u : 0u);
    return __uint_as_float(bits | s);
}

template <int FMT>
__global__ __launch_bounds__(256) void mx_dequant_kernel(const uint8_t* q, const uint8_t* s, uint16_t* out,
                                                         int64_t nblocks) {
    // one lane per 8 elements; 4 lanes per MX block
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t blk = i >> 2;
    if (blk >= nblocks) return;
    const uint32_t byte = s[blk];
    // fp32 holds 2^(byte-127) exactly (subnormal for byte 0); multiply in two steps to stay exact
    const float sc = (byte == 255u) ? __uint_as_float(0x7FC00000u) : fwd_scale(byte);
    float v[8];
    if (FMT == kFmtE4M3 || FMT == kFmtE5M2) {
        const uint2 c = *(const uint2*)(q + i * 8);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v[k] = FMT == kFmtE5M2 ? dec_e5m2((c.x >> (8 * k)) & 0xFFu) : dec_e4m3((c.x >> (8 * k)) & 0xFFu);
            v[4 + k] = FMT == kFmtE5M2 ? dec_e5m2((c.y >> (8 * k)) & 0xFFu) : dec_e4m3((c.y >> (8 * k)) & 0xFFu);
        }
    } else {
        const uint32_t c = *(const uint32_t*)(q + i * 4);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = dec_e2m1((c >> (4 * k)) & 0xFu);
    }
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v2bf h = {(__bf16)(v[2 * k] * sc), (__bf16)(v[2 * k + 1] * sc)};
        o[k] = __builtin_bit_cast(uint32_t, h);
    }
    *(uint4*)(out + i * 8) = make_uint4(o[0], o[1], o[2], o[3]);
}

// ---------------------------------------------------------------------------
// host-side dispatch
// ---------------------------------------------------------------------------
template <int FMT, int SMODE, bool TWOD, int ACT = -1, bool SR = false, bool RHT = false>
static int launch_quant(QuantArgs& a, int64_t tiles_r, int64_t tiles_c, hipStream_t st) {
    const int64_t super_r = (tiles_r + QSUPER - 1) / QSUPER, super_c = (tiles_c + QSUPER - 1) / QSUPER;
    const int64_t n_super = super_r * super_c;
    const int64_t wgs = (n_super + 7) / 8 * 8 * QSUPER * QSUPER;
    if (tiles_r > 0x7FFFFFFF || tiles_c > 0x7FFFFFFF || wgs > 0x7FFFFFFF) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    a.tiles_r = (int)tiles_r;
    a.tiles_c = (int)tiles_c;
    a.super_c = (int)super_c;
    a.n_super = (int)n_super;
    const dim3 grid((unsigned)wgs);
    const bool row = a.q_row != nullptr, col = a.q_colT != nullptr;
    if (row && col)
        hipLaunchKernelGGL((mx_quant_kernel<FMT, SMODE, true, true, TWOD, ACT, SR, RHT>), grid, dim3(QTHREADS), 0, st, a);
    else if (row && !RHT)
        hipLaunchKernelGGL((mx_quant_kernel<FMT, SMODE, true, false, TWOD, ACT, SR, false>), grid, dim3(QTHREADS), 0, st,
                           a);
    else if (ACT < 0 && col)
        hipLaunchKernelGGL((mx_quant_kernel<FMT, SMODE, false, true, TWOD, -1, SR, RHT>), grid, dim3(QTHREADS), 0, st, a);
    else
        return MXL_EINVAL;   // the fused activation always feeds a forward GEMM: a row-wise copy is part of it
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

template <bool TWOD, int ACT = -1>
static int dispatch_quant(int fmt, int smode, QuantArgs& a, int64_t tiles_r, int64_t tiles_c, hipStream_t st) {
#define MXL_Q(F, S) \
    if (fmt == F && smode == S) return launch_quant<F, S, TWOD, ACT>(a, tiles_r, tiles_c, st);
    MXL_Q(MXL_FMT_E4M3, MXL_SCALE_OCP_FLOOR)
    MXL_Q(MXL_FMT_E4M3, MXL_SCALE_RCEIL)
    MXL_Q(MXL_FMT_E4M3, MXL_SCALE_EVEN)
    MXL_Q(MXL_FMT_E2M1, MXL_SCALE_OCP_FLOOR)
    MXL_Q(MXL_FMT_E2M1, MXL_SCALE_RCEIL)
    MXL_Q(MXL_FMT_E2M1, MXL_SCALE_EVEN)
#undef MXL_Q
    return MXL_EINVAL;
}

// the MXFP4 recipe's options (1-D E2M1 only): stochastic rounding, Hadamard transform of the transposed copy
template <bool SR, bool RHT>
static int dispatch_quant_fp4(int smode, QuantArgs& a, int64_t tiles_r, int64_t tiles_c, hipStream_t st) {
    if (smode == MXL_SCALE_OCP_FLOOR)
        return launch_quant<MXL_FMT_E2M1, MXL_SCALE_OCP_FLOOR, false, -1, SR, RHT>(a, tiles_r, tiles_c, st);
    if (smode == MXL_SCALE_RCEIL) return launch_quant<MXL_FMT_E2M1, MXL_SCALE_RCEIL, false, -1, SR, RHT>(a, tiles_r, tiles_c, st);
    if (smode == MXL_SCALE_EVEN) return launch_quant<MXL_FMT_E2M1, MXL_SCALE_EVEN, false, -1, SR, RHT>(a, tiles_r, tiles_c, st);
    return MXL_EINVAL;
}

// tensor-wise scaling: E4M3 or E5M2 codes, 1-D (activations, gradients) or batched-matrix (weights) tiling
template <bool TWOD>
static int dispatch_quant_tensor(int fmt, QuantArgs& a, int64_t tiles_r, int64_t tiles_c, hipStream_t st) {
    if (fmt == MXL_FMT_E4M3) return launch_quant<MXL_FMT_E4M3, SCALE_TENSOR, TWOD>(a, tiles_r, tiles_c, st);
    if (fmt == MXL_FMT_E5M2) return launch_quant<MXL_FMT_E5M2, SCALE_TENSOR, TWOD>(a, tiles_r, tiles_c, st);
    return MXL_EINVAL;
}

// abs-max of a bf16 tensor: non-negative floats order like their bit patterns, so an integer atomic max on the
// fp32 pattern does it (a NaN pattern is larger than every number and wins).  One atomic per workgroup.
__global__ __launch_bounds__(256) void amax_kernel(const uint16_t* x, int64_t n8, int64_t n, uint32_t* out) {
    __shared__ uint32_t part[4];
    uint32_t m = 0;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
        const uint4 v = load16_streaming(x + i * 8);
        m = pk_max16(m, pk_max16(pk_max16(v.x & 0x7FFF7FFFu, v.y & 0x7FFF7FFFu), pk_max16(v.z & 0x7FFF7FFFu, v.w & 0x7FFF7FFFu)));
    }
    m = hmax16(m);
    if (blockIdx.x == 0 && threadIdx.x == 0)
        for (int64_t i = n8 * 8; i < n; ++i) m = max(m, (uint32_t)(x[i] & 0x7FFFu));   // tail of fewer than 8 elements
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, s));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = max(max(part[0], part[1]), max(part[2], part[3]));
        atomicMax(out, m << 16);   // bf16 pattern -> fp32 pattern
    }
}

__global__ void amax_init_kernel(uint32_t* out) { *out = 0u; }

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_amax(const void* x_bf16, int64_t n, void* amax_f32, void* stream) {
    if (n < 0 || !amax_f32 || (n > 0 && !x_bf16) || ((uintptr_t)x_bf16 & 15) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipStream_t st = (hipStream_t)stream;
    // a fill kernel, not a memset: callers may be capturing the stream into a graph
    hipLaunchKernelGGL(amax_init_kernel, dim3(1), dim3(1), 0, st, (uint32_t*)amax_f32);
    if (hipGetLastError() != hipSuccess) return MXL_ELAUNCH;
    if (n == 0) return MXL_OK;
    const int64_t n8 = n / 8;
    int64_t grid = (n8 + 256 * 8 - 1) / (256 * 8);   // about 8 loads per lane
    grid = grid < 1 ? 1 : grid > 4096 ? 4096 : grid;
    hipLaunchKernelGGL(amax_kernel, dim3((unsigned)grid), dim3(256), 0, st, (const uint16_t*)x_bf16, n8, n, (uint32_t*)amax_f32);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int64_t mxl_padded_width(int64_t total_rows, int num_groups) {
    if (num_groups < 1) num_groups = 1;
    return (total_rows + (int64_t)(MXL_SEG_ALIGN - 1) * num_groups) / MXL_SEG_ALIGN * MXL_SEG_ALIGN;
}

// code layout selected by the flags: 0 row-major, 1 K-chunk-major, 2 K-step-major, 3 K-step-major with steps of 128
// elements (E2M1 only: 64-byte rows, i.e. K-chunk-major codes with K-step-major scale panels), -1 contradictory flags
static int qf_layout(uint32_t flags) {
    if ((flags & MXL_QF_KCHUNK) && (flags & MXL_QF_KSTEP)) return -1;
    if ((flags & MXL_QF_KSTEP128) && !(flags & MXL_QF_KSTEP)) return -1;
    return (flags & MXL_QF_KSTEP128) ? 3 : (flags & MXL_QF_KSTEP) ? 2 : (flags & MXL_QF_KCHUNK) ? 1 : 0;
}

static int quantize_1d(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt, int scale_mode,
                       const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT, void* s_colT,
                       int act, const void* probs, int probs_dtype, const uint8_t* row_mask, void* stream,
                       bool sr = false, uint64_t sr_seed = 0, bool rht = false, uint32_t rht_signs = 0,
                       int kchunk = 0, const void* norm_w = nullptr, const void* tensor_amax = nullptr,
                       void* scale_inv_out = nullptr) {
    if (row_ld == 0) row_ld = cols;
    if (kchunk < 0) return MXL_EINVAL;                  // contradictory layout flags
    if (kchunk == 2 && fmt == MXL_FMT_E2M1) kchunk = 3;  // E2M1 activations: the K step is 128 elements (64-byte rows)
    if (kchunk == 3 && fmt != MXL_FMT_E2M1) return MXL_EINVAL;
    if (kchunk && q_row && row_ld % QT != 0) return MXL_EINVAL;   // whole 128-element chunks
    if ((sr || rht) && (fmt != MXL_FMT_E2M1 || act >= 0)) return MXL_EINVAL;
    if (rht && !q_colT) return MXL_EINVAL;   // the transform belongs to the transposed copy
    if (row_ld < cols || row_ld % MXL_BLOCK != 0) return MXL_EINVAL;
    if ((!x_bf16 && rows > 0) || rows < 0 || cols <= 0 || cols % MXL_BLOCK != 0) return MXL_EINVAL;
    if ((q_row == nullptr) != (s_row == nullptr) || (q_colT == nullptr) != (s_colT == nullptr)) return MXL_EINVAL;
    if (!q_row && !q_colT) return MXL_EINVAL;
    if (num_groups < 0 || num_groups > MXL_MAX_GROUPS || (num_groups > 0) != (group_lens != nullptr)) return MXL_EINVAL;
    QuantArgs a;
    a.x = (const uint16_t*)x_bf16;
    a.rows = rows;
    a.cols = cols;
    a.group_lens = group_lens;
    a.num_groups = num_groups;
    a.q_row = (uint8_t*)q_row;
    a.s_row = (uint8_t*)s_row;
    a.q_colT = (uint8_t*)q_colT;
    a.s_colT = (uint8_t*)s_colT;
    a.row_ld = row_ld;
    a.W = mxl_padded_width(rows, num_groups);
    a.mat_rows = 0;
    a.probs = probs;
    a.probs_bf16 = probs_dtype == MXL_PROBS_BF16;
    a.row_mask = row_mask;
    a.norm_w = (const uint16_t*)norm_w;
    a.tensor_amax = (const float*)tensor_amax;
    a.scale_inv_out = (float*)scale_inv_out;
    a.sr_seed = sr_seed;
    a.rht_signs = rht_signs & 0xFFFFu;
    a.kchunk = kchunk;
    a.chunk_rows_row = rows;
    a.chunk_rows_col = cols;
    const int64_t gx = q_colT ? a.W / QT : (rows + QT - 1) / QT;
    const int64_t gy = ((q_row ? row_ld : cols) + QT - 1) / QT;
    if (tensor_amax) {
        if (sr || rht || act >= 0) return MXL_EINVAL;
        if (gx == 0) return MXL_OK;   // nothing to quantise (scale_inv_out is then left unwritten)
        return dispatch_quant_tensor<false>(fmt, a, gx, gy, (hipStream_t)stream);
    }
    if (gx == 0) return MXL_OK;
    if (sr && rht) return dispatch_quant_fp4<true, true>(scale_mode, a, gx, gy, (hipStream_t)stream);
    if (sr) return dispatch_quant_fp4<true, false>(scale_mode, a, gx, gy, (hipStream_t)stream);
    if (rht) return dispatch_quant_fp4<false, true>(scale_mode, a, gx, gy, (hipStream_t)stream);
    if (act == MXL_ACT_SILU) return dispatch_quant<false, MXL_ACT_SILU>(fmt, scale_mode, a, gx, gy, (hipStream_t)stream);
    if (act == MXL_ACT_GELU) return dispatch_quant<false, MXL_ACT_GELU>(fmt, scale_mode, a, gx, gy, (hipStream_t)stream);
    if (act == PRO_RMSNORM) return dispatch_quant<false, PRO_RMSNORM>(fmt, scale_mode, a, gx, gy, (hipStream_t)stream);
    return dispatch_quant<false>(fmt, scale_mode, a, gx, gy, (hipStream_t)stream);
}

extern "C" int mxl_quantize(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt, int scale_mode,
                            const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                            void* s_colT, void* stream) {
    return quantize_1d(x_bf16, rows, cols, row_ld, fmt, scale_mode, group_lens, num_groups, q_row, s_row, q_colT, s_colT,
                       -1, nullptr, MXL_PROBS_F32, nullptr, stream);
}

extern "C" int mxl_quantize_ex(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt, int scale_mode,
                               const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                               void* s_colT, uint32_t flags, uint64_t sr_seed, uint32_t rht_signs, void* stream) {
    if (flags & ~(uint32_t)(MXL_QF_SR | MXL_QF_RHT_COL | MXL_QF_KCHUNK | MXL_QF_KSTEP | MXL_QF_KSTEP128)) return MXL_EINVAL;
    return quantize_1d(x_bf16, rows, cols, row_ld, fmt, scale_mode, group_lens, num_groups, q_row, s_row, q_colT,
                       s_colT, -1, nullptr, MXL_PROBS_F32, nullptr, stream, (flags & MXL_QF_SR) != 0, sr_seed,
                       (flags & MXL_QF_RHT_COL) != 0, rht_signs, qf_layout(flags));
}

extern "C" int mxl_glu_probs_quantize(const void* x_bf16, const void* probs, int probs_dtype, const uint8_t* row_mask,
                                      int64_t rows, int64_t f, int64_t row_ld, int act, int fmt, int scale_mode,
                                      const int64_t* group_lens, int num_groups, void* q_row, void* s_row, void* q_colT,
                                      void* s_colT, uint32_t flags, void* stream) {
    if (act != MXL_ACT_SILU && act != MXL_ACT_GELU) return MXL_EINVAL;
    if (probs_dtype != MXL_PROBS_F32 && probs_dtype != MXL_PROBS_BF16) return MXL_EINVAL;
    if (rows > 0 && !probs) return MXL_EINVAL;
    if (flags & ~(uint32_t)(MXL_QF_KCHUNK | MXL_QF_KSTEP | MXL_QF_KSTEP128)) return MXL_EINVAL;
    return quantize_1d(x_bf16, rows, f, row_ld, fmt, scale_mode, group_lens, num_groups, q_row, s_row, q_colT, s_colT, act,
                       probs, probs_dtype, row_mask, stream, false, 0, false, 0, qf_layout(flags));
}

extern "C" int mxl_rmsnorm_quantize(const void* x_bf16, const void* w_bf16, const void* rstd_f32, int64_t rows, int64_t k,
                                    int64_t row_ld, int fmt, int scale_mode, const int64_t* group_lens, int num_groups,
                                    void* q_row, void* s_row, void* q_colT, void* s_colT, uint32_t flags, void* stream) {
    if (!w_bf16 || (rows > 0 && !rstd_f32)) return MXL_EINVAL;
    if (flags & ~(uint32_t)(MXL_QF_KCHUNK | MXL_QF_KSTEP | MXL_QF_KSTEP128)) return MXL_EINVAL;
    return quantize_1d(x_bf16, rows, k, row_ld, fmt, scale_mode, group_lens, num_groups, q_row, s_row, q_colT, s_colT,
                       PRO_RMSNORM, rstd_f32, MXL_PROBS_F32, nullptr, stream, false, 0, false, 0,
                       qf_layout(flags), w_bf16);
}

static int quantize_weight_2d(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld, int64_t n_ld, int fmt,
                              int scale_mode, void* q_row, void* s_row, void* q_colT, void* s_colT, int kchunk,
                              void* stream, const void* tensor_amax = nullptr, void* scale_inv_out = nullptr) {
    if (k_ld == 0) k_ld = k;
    if (n_ld == 0) n_ld = n;
    if (kchunk < 0 || (kchunk == 3 && fmt != MXL_FMT_E2M1)) return MXL_EINVAL;
    if (kchunk && ((q_row && k_ld % QT != 0) || (q_colT && n_ld % QT != 0))) return MXL_EINVAL;   // whole chunks
    if (k_ld < k || n_ld < n || k_ld % MXL_BLOCK != 0 || n_ld % MXL_BLOCK != 0) return MXL_EINVAL;
    if (n_ld > (n + QT - 1) / QT * QT) return MXL_EINVAL;  // padding of the transposed copy stays inside the last tile
    if (!w_bf16 || batch <= 0 || n <= 0 || k <= 0 || n % MXL_BLOCK != 0 || k % MXL_BLOCK != 0) return MXL_EINVAL;
    // (the transposed copy's scales may be asked for without its codes, next to a row-wise copy)
    if ((q_row == nullptr) != (s_row == nullptr) || (q_colT != nullptr && s_colT == nullptr)) return MXL_EINVAL;
    if (s_colT != nullptr && q_colT == nullptr && q_row == nullptr) return MXL_EINVAL;
    if (!q_row && !q_colT) return MXL_EINVAL;
    QuantArgs a;
    a.x = (const uint16_t*)w_bf16;
    a.rows = batch * n;
    a.cols = k;
    a.group_lens = nullptr;
    a.num_groups = 0;
    a.q_row = (uint8_t*)q_row;
    a.s_row = (uint8_t*)s_row;
    a.q_colT = (uint8_t*)q_colT;
    a.s_colT = (uint8_t*)s_colT;
    a.row_ld = k_ld;
    a.W = n_ld;  // transposed copy of each matrix is [k, n_ld]
    a.mat_rows = n;
    a.probs = nullptr;
    a.probs_bf16 = 0;
    a.row_mask = nullptr;
    a.norm_w = nullptr;
    a.tensor_amax = (const float*)tensor_amax;
    a.scale_inv_out = (float*)scale_inv_out;
    a.sr_seed = 0;
    a.rht_signs = 0;
    a.kchunk = kchunk;
    a.chunk_rows_row = batch * n;   // the batch is one operand of batch * n rows (resp. batch * k for the transposed copy)
    a.chunk_rows_col = batch * k;
    const int64_t gx = batch * ((n + QT - 1) / QT);
    const int64_t gy = ((q_row ? k_ld : k) + QT - 1) / QT;
    if (tensor_amax) return dispatch_quant_tensor<true>(fmt, a, gx, gy, (hipStream_t)stream);
    return dispatch_quant<true>(fmt, scale_mode, a, gx, gy, (hipStream_t)stream);
}

extern "C" int mxl_quantize_weight_2d(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld,
                                      int64_t n_ld, int fmt, int scale_mode, void* q_row, void* s_row, void* q_colT,
                                      void* s_colT, void* stream) {
    return quantize_weight_2d(w_bf16, batch, n, k, k_ld, n_ld, fmt, scale_mode, q_row, s_row, q_colT, s_colT, false, stream);
}

extern "C" int mxl_quantize_weight_2d_ex(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld,
                                         int64_t n_ld, int fmt, int scale_mode, void* q_row, void* s_row, void* q_colT,
                                         void* s_colT, uint32_t flags, void* stream) {
    if (flags & ~(uint32_t)(MXL_QF_KCHUNK | MXL_QF_KSTEP | MXL_QF_KSTEP128)) return MXL_EINVAL;
    return quantize_weight_2d(w_bf16, batch, n, k, k_ld, n_ld, fmt, scale_mode, q_row, s_row, q_colT, s_colT,
                              qf_layout(flags), stream);
}

extern "C" int mxl_quantize_tensorwise(const void* x_bf16, int64_t rows, int64_t cols, int64_t row_ld, int fmt,
                                       const void* amax_f32, const int64_t* group_lens, int num_groups, void* q_row,
                                       void* s_row, void* q_colT, void* s_colT, void* scale_inv_f32, uint32_t flags,
                                       void* stream) {
    if (!amax_f32 || (fmt != MXL_FMT_E4M3 && fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if (flags & ~(uint32_t)(MXL_QF_KCHUNK | MXL_QF_KSTEP)) return MXL_EINVAL;
    return quantize_1d(x_bf16, rows, cols, row_ld, fmt, MXL_SCALE_OCP_FLOOR, group_lens, num_groups, q_row, s_row, q_colT,
                       s_colT, -1, nullptr, MXL_PROBS_F32, nullptr, stream, false, 0, false, 0,
                       qf_layout(flags), nullptr, amax_f32, scale_inv_f32);
}

extern "C" int mxl_quantize_weight_tensorwise(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int64_t k_ld,
                                              int64_t n_ld, int fmt, const void* amax_f32, void* q_row, void* s_row,
                                              void* q_colT, void* s_colT, void* scale_inv_f32, uint32_t flags,
                                              void* stream) {
    if (!amax_f32 || (fmt != MXL_FMT_E4M3 && fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if (flags & ~(uint32_t)(MXL_QF_KCHUNK | MXL_QF_KSTEP)) return MXL_EINVAL;
    return quantize_weight_2d(w_bf16, batch, n, k, k_ld, n_ld, fmt, MXL_SCALE_OCP_FLOOR, q_row, s_row, q_colT, s_colT,
                              qf_layout(flags), stream, amax_f32, scale_inv_f32);
}

extern "C" int mxl_dequantize(const void* codes, const void* scales, int64_t rows, int64_t k, int fmt,
                              void* out_bf16, void* stream) {
    if (!codes || !scales || !out_bf16 || rows < 0 || k <= 0 || k % MXL_BLOCK != 0) return MXL_EINVAL;
    const int64_t nblocks = rows * (k / MXL_BLOCK);
    if (nblocks == 0) return MXL_OK;
    const int64_t threads = nblocks * 4;
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7FFFFFFF) return MXL_EINVAL;
    if (fmt != MXL_FMT_E4M3 && fmt != MXL_FMT_E2M1 && fmt != MXL_FMT_E5M2) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    if (fmt == MXL_FMT_E5M2)
        hipLaunchKernelGGL((mx_dequant_kernel<MXL_FMT_E5M2>), dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const uint8_t*)codes, (const uint8_t*)scales, (uint16_t*)out_bf16, nblocks);
    else if (fmt == MXL_FMT_E4M3)
        hipLaunchKernelGGL((mx_dequant_kernel<MXL_FMT_E4M3>), dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const uint8_t*)codes, (const uint8_t*)scales, (uint16_t*)out_bf16, nblocks);
    else if (fmt == MXL_FMT_E2M1)
        hipLaunchKernelGGL((mx_dequant_kernel<MXL_FMT_E2M1>), dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const uint8_t*)codes, (const uint8_t*)scales, (uint16_t*)out_bf16, nblocks);
    else
        return MXL_EINVAL;
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}
