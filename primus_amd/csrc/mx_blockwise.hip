// The 128-blockwise FP8 recipe (ScalingGranularity.BLOCKWISE, block_size 128), the third recipe that the
// reference's argument validation admits (primus/backends/megatron/patches/args/rocm_arg_validation.py:145) and that
// its FP8LinearBlockwiseFunction runs (primus/backends/megatron/core/extensions/primus_turbo_float8_local.py:993-1089):
//
//   activations / gradients : one fp32 scale per 1 x 128 block along the contraction dimension
//                             (quant_fp8_blockwise_impl(x, dtype, axis, block_size), :1019, :1053-1059)
//   weights                 : one fp32 scale per 128 x 128 block (quant_fp8_blockwise_for_weight_impl, :1020, :1060)
//   GEMM                    : c[m, n] = sum over K blocks kb of  sa[m, kb] * sb[n, kb] * (a[m, kb] . b[n, kb])
//                             with fp32 accumulation (gemm_fp8_impl with granularity BLOCKWISE, :1022-1033)
//
// scale = fp8_max / max(amax, 1e-12), codes = cast(clamp(x * scale)), scale_inv = 1 / scale, all fp32: the formula the
// reference restates for its tensor-wise quantiser (:194-207) applied per block.  Arbitrary fp32 factors cannot ride on
// the MFMA's E8M0 scale inputs, so these GEMMs keep two kinds of accumulators: the MFMAs of one K block of 128 add up
// in partial tiles (from zero), which are then multiplied into the real accumulators with the block's factors.  Two
// kernels, both of 8 waves, two per SIMD: a 128 x 256 tile with all four partial tiles of a wave's 64 x 64 at once
// (small problems), and a 256 x 256 tile whose waves own 64 x 128 and keep one column of partial tiles at a time.
#include "mx_device.h"

namespace mxl {

constexpr int BW = 128;            // block edge
constexpr int BW_THREADS = 256;

typedef float bv16f __attribute__((ext_vector_type(16)));
typedef int bv8i __attribute__((ext_vector_type(8)));
typedef __bf16 bv4bf __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------------------------------------
// Quantiser.  One workgroup per 128 x 128 tile of x[rows, cols] (cols % 128 == 0; rows ragged).  The tile stays in
// registers: lane (wave w, row group rg = lane / 16, c16 = lane % 16) holds rows 32 w + 8 rg + 0..7, columns
// 8 c16 + 0..7, eight 16-byte loads that are all in flight together.  A row's largest magnitude is a maximum over the
// 16 lanes of a DPP row, a column's goes through the row groups of a wave and then through LDS over the four waves;
// the fp32 factors are computed once per row and column (a division each, by 256 of the workgroup's lanes for the tile)
// and handed round through LDS.  Row-wise codes leave as 16-byte stores (a lane pair swaps 8-byte pieces of a row
// pair); the transposed codes are converted straight into transposed order (the convert instruction takes any two
// values), collected in an LDS tile and stored as 128 contiguous bytes per output row.
//   ROW  : q_row[rows, cols], sinv_row[rows, cols / 128]
//   COL  : q_colT[cols, rows_pad], sinv_colT[cols, rows_pad / 128], rows_pad = rows rounded up to 128 (zero codes)
//   TWOD : one scale per tile for both copies: sinv_row[ceil(rows / 128), cols / 128], sinv_colT[cols / 128, ceil(rows / 128)]
// A block that holds a NaN or an infinity becomes NaN codes (0x7F) with scale_inv = 1 / (fp8_max / amax) as computed.
// ------------------------------------------------------------------------------------------------------------
struct BwQuantArgs {
    const uint16_t* x;
    int64_t rows, cols;
    uint8_t* q_row;
    float* sinv_row;
    uint8_t* q_colT;
    float* sinv_colT;
    // grouped activations (1-D blocks only): the transposed copy is segment-padded like the MX one -- group g owns the
    // columns [poff_g, poff_g + len_g) of its W = mxl_padded_width(rows, G) columns, poff = prefix sum of the lens
    // rounded up to 128 -- so that the blocks along the tokens restart at every group
    // (quant_fp8_blockwise_segment_m_row_col_impl, primus/backends/megatron/core/extensions/zbpp_gemm.py:633, :785)
    const int64_t* group_lens;
    int num_groups;
    int64_t W;
    int tiles_r, tiles_c, super_c, n_super;   // the launch's tile grid and its 8 x 8 supertiles
};

constexpr int BW_MAX_GROUPS = 1024;

// Which group holds tile `y` when every group is cut into tiles of TR rows (a group's last tile may be ragged):
// `pre` (LDS, BW_MAX_GROUPS + 1 ints) receives the prefix sum of the groups' tile counts, `red` (LDS, one word of 8
// bytes per wave of the workgroup, NT / 64 of them) is scratch.  Returns the group (or -1 behind the last tile); tile_in_group, the rows in front of the group
// and its length come back through the references.  Negative lens read as 0.  All threads of the workgroup call it.
template <int NT = 256, int TR = BW>
__device__ __forceinline__ int bw_locate(const int64_t* lens, int groups, int y, int* pre, int64_t* red, int& tile_in_group,
                                         int64_t& rows_before, int64_t& len) {
    const int t = threadIdx.x;
    if (t == 0) pre[0] = 0;
    for (int j = t; j < groups; j += NT) {
        const int64_t l = lens[j] > 0 ? lens[j] : 0;
        pre[j + 1] = (int)((l + TR - 1) / TR);
    }
    __syncthreads();
    if (t < 64) {   // in-place inclusive scan of pre[1 .. groups], a run of consecutive entries per lane
        const int per = (groups + 63) / 64, j0 = 1 + t * per;
        int sum = 0;
        for (int i = 0; i < per; ++i)
            if (j0 + i <= groups) sum += pre[j0 + i];
        int incl = sum;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(incl, d);
            if (t >= d) incl += o;
        }
        int run = incl - sum;
        for (int i = 0; i < per; ++i)
            if (j0 + i <= groups) {
                run += pre[j0 + i];
                pre[j0 + i] = run;
            }
    }
    __syncthreads();
    int g = -1;
    if (y < pre[groups]) {
        int lo = 0, hi = groups;   // first index in (0, groups] whose prefix exceeds y
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (pre[mid] > y) hi = mid;
            else lo = mid + 1;
        }
        g = lo - 1;
    }
    tile_in_group = g >= 0 ? y - pre[g] : 0;
    int64_t part = 0;
    for (int j = t; j < g; j += NT) part += lens[j] > 0 ? lens[j] : 0;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) part += __shfl_xor(part, d);
    if ((t & 63) == 0) red[t >> 6] = part;
    __syncthreads();
    rows_before = 0;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) rows_before += red[i];
    len = g >= 0 ? (lens[g] > 0 ? lens[g] : 0) : 0;
    return g;
}

constexpr int BW_TPITCH = BW + 16;   // bytes per LDS row of the transposed code tile

template <int FMT> __device__ __forceinline__ float bw_fp8_max() { return FMT == kFmtE5M2 ? 57344.f : 448.f; }
// fp8_max / max(amax, 1e-12) with the sign bit set when the block holds a NaN or an infinity (its codes are all NaN
// then, and the factor, which is never negative, is not used for them)
template <int FMT> __device__ __forceinline__ uint32_t bw_scale_word(uint32_t amax16, float& sinv) {
    const float sc = bw_fp8_max<FMT>() / fmaxf(__uint_as_float(amax16 << 16), 1e-12f);
    sinv = 1.0f / sc;
    return __float_as_uint(sc) | (amax16 >= 0x7F80u ? 0x80000000u : 0u);
}
template <int FMT> __device__ __forceinline__ uint2 bw_cvt8(uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t scale_word) {
    const float sc = __uint_as_float(scale_word & 0x7FFFFFFFu);
    const bool bad = (scale_word >> 31) != 0;
    uint2 o;
    o.x = cvt4_fp8<FMT>(p0, p1, sc);
    o.y = cvt4_fp8<FMT>(p2, p3, sc);
    o.x = bad ? 0x7F7F7F7Fu : o.x;
    o.y = bad ? 0x7F7F7F7Fu : o.y;
    return o;
}

template <int FMT, bool TWOD>
__global__ __launch_bounds__(BW_THREADS) void bw_quant_kernel(BwQuantArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t t_tile[BW * BW_TPITCH];
    __shared__ __attribute__((aligned(16))) uint32_t amax_r[BW];         // per row
    __shared__ __attribute__((aligned(16))) uint32_t amax_c[4][BW / 2];  // per wave: column pairs, packed 16-bit maxima
    __shared__ __attribute__((aligned(16))) uint32_t scale_r[BW], scale_c[BW];
    __shared__ uint32_t amax_w[4];
    __shared__ int grp_pre[BW_MAX_GROUPS + 1];
    __shared__ int64_t grp_red[4];
    const int t = threadIdx.x;
    const int w = t >> 6, l = t & 63, c16 = l & 15, rg = l >> 4, rbase = 32 * w + 8 * rg;
    // Tile order: consecutive workgroup ids land on different XCDs, and every XCD walks whole 8 x 8 supertiles (column
    // tile fastest): the 4-byte factors that 8 neighbouring tiles write into one row of sinv_row (32 contiguous bytes)
    // then meet in one L2, and the resident workgroups of an XCD cover long contiguous row spans.
    const int L = blockIdx.x, xcd = L & 7, kk = L >> 3;
    const int sup = (kk >> 6) * 8 + xcd;
    if (sup >= a.n_super) return;
    const int bx = (sup % a.super_c) * 8 + (kk & 7), by = (sup / a.super_c) * 8 + ((kk >> 3) & 7);
    if (bx >= a.tiles_c || by >= a.tiles_r) return;
    const int64_t col0 = (int64_t)bx * BW;
    // the tile's rows: rows [row0, row0 + valid) of this matrix land in columns [prow0, prow0 + 128) of the transposed copy
    const int64_t zoff = TWOD ? (int64_t)blockIdx.y : 0;          // matrix of a batch of weights
    int64_t row0 = (int64_t)by * BW, prow0 = row0, rows_pad = (a.rows + BW - 1) / BW * BW;
    int64_t valid64 = a.rows - row0 < BW ? a.rows - row0 : BW;
    if (!TWOD && a.group_lens != nullptr) {
        int tile_in_group;
        int64_t before, len;
        const int grp = bw_locate(a.group_lens, a.num_groups, by, grp_pre, grp_red, tile_in_group, before, len);
        // bw_locate counts tiles per group exactly as the padded layout counts 128-column pieces per segment
        row0 = before + (int64_t)tile_in_group * BW;
        valid64 = grp >= 0 ? len - (int64_t)tile_in_group * BW : 0;
        valid64 = valid64 > BW ? BW : valid64;
        valid64 = row0 + valid64 > a.rows ? a.rows - row0 : valid64;     // lens that claim more rows than there are
        rows_pad = a.W;
    }
    const int valid = valid64 < 0 ? 0 : (int)valid64;
    const uint16_t* xin = a.x + zoff * a.rows * a.cols;
    const int64_t kb_cols = a.cols / BW, kb_rows = rows_pad / BW;
    const bool want_row = a.q_row != nullptr, want_col = a.q_colT != nullptr;   // uniform

    // ---- load 8 rows x 8 columns per lane; rows past the end read as zero ----
    // (a row past the end fetches the tile's last row instead and drops it: eight loads without a branch between them)
    uint4 d[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) d[it] = make_uint4(0u, 0u, 0u, 0u);
    if (valid > 0) {
        const uint16_t* src = xin + row0 * a.cols + col0 + 8 * c16;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = rbase + it;
            const uint4 v = load16_streaming(src + (int64_t)(r < valid ? r : valid - 1) * a.cols);
            d[it] = r < valid ? v : make_uint4(0u, 0u, 0u, 0u);
        }
    }

    // ---- largest magnitudes (15-bit bf16 patterns) ----
    uint32_t rmax[8];                    // of the lane's rows, over the 128 columns
    uint32_t cmax[4] = {0u, 0u, 0u, 0u}; // of the lane's column pairs (packed), over its 8 rows
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const uint32_t p0 = d[it].x & 0x7FFF7FFFu, p1 = d[it].y & 0x7FFF7FFFu, p2 = d[it].z & 0x7FFF7FFFu,
                       p3 = d[it].w & 0x7FFF7FFFu;
        if (!TWOD) {
            cmax[0] = pk_max16(cmax[0], p0);
            cmax[1] = pk_max16(cmax[1], p1);
            cmax[2] = pk_max16(cmax[2], p2);
            cmax[3] = pk_max16(cmax[3], p3);
        }
        uint32_t m = hmax16(pk_max16(pk_max16(p0, p1), pk_max16(p2, p3)));
        m = max(m, dpp_xor1(m));
        m = max(m, dpp_xor2(m));
        if (!TWOD) {
            m = max(m, dpp_half_mirror(m));
            m = max(m, dpp_mirror(m));
        }
        rmax[it] = m;
    }
    uint32_t tile_word = 0u;
    if (TWOD) {
        uint32_t m = rmax[0];
#pragma unroll
        for (int it = 1; it < 8; ++it) m = max(m, rmax[it]);
#pragma unroll
        for (int dlt = 4; dlt < 64; dlt <<= 1) m = max(m, (uint32_t)__shfl_xor((int)m, dlt));
        if (l == 0) amax_w[w] = m;
        __syncthreads();
        m = max(max(amax_w[0], amax_w[1]), max(amax_w[2], amax_w[3]));
        float sinv;
        tile_word = bw_scale_word<FMT>(m, sinv);
        if (t == 0) {
            if (want_row) a.sinv_row[(zoff * kb_rows + by) * kb_cols + bx] = sinv;
            if (want_col) a.sinv_colT[(zoff * kb_cols + bx) * kb_rows + by] = sinv;
        }
    } else {
        if (want_col) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 16));
                cmax[j] = pk_max16(cmax[j], (uint32_t)__shfl_xor((int)cmax[j], 32));
            }
            if (rg == 0) *(uint4*)&amax_c[w][4 * c16] = make_uint4(cmax[0], cmax[1], cmax[2], cmax[3]);
        }
        if (want_row && c16 == 0) {
            *(uint4*)&amax_r[rbase] = make_uint4(rmax[0], rmax[1], rmax[2], rmax[3]);
            *(uint4*)&amax_r[rbase + 4] = make_uint4(rmax[4], rmax[5], rmax[6], rmax[7]);
        }
        __syncthreads();
        // one factor per row (waves 2 and 3) and per column (waves 0 and 1)
        if (t >= BW) {
            if (want_row) {
                const int r = t - BW;
                float sinv;
                scale_r[r] = bw_scale_word<FMT>(amax_r[r], sinv);
                if (r < valid) a.sinv_row[(row0 + r) * kb_cols + bx] = sinv;
            }
        } else if (want_col) {
            const uint16_t* h = (const uint16_t*)&amax_c[0][0];
            const uint32_t m = max(max((uint32_t)h[t], (uint32_t)h[BW + t]), max((uint32_t)h[2 * BW + t], (uint32_t)h[3 * BW + t]));
            float sinv;
            scale_c[t] = bw_scale_word<FMT>(m, sinv);
            a.sinv_colT[(col0 + t) * kb_rows + by] = sinv;
        }
        __syncthreads();
    }

    // ---- row-wise copy: two rows at a time, 16 bytes per lane ----
    if (want_row) {
        uint32_t sw[8];
        if (!TWOD) {
            const uint4 s0 = *(const uint4*)&scale_r[rbase], s1 = *(const uint4*)&scale_r[rbase + 4];
            sw[0] = s0.x; sw[1] = s0.y; sw[2] = s0.z; sw[3] = s0.w;
            sw[4] = s1.x; sw[5] = s1.y; sw[6] = s1.z; sw[7] = s1.w;
        }
        const bool odd = (c16 & 1) != 0;
        uint8_t* dst = a.q_row + (zoff * a.rows + row0 + rbase) * a.cols + col0 + 8 * (c16 & ~1);
        uint2 o_even = make_uint2(0u, 0u);
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const uint2 o = bw_cvt8<FMT>(d[it].x, d[it].y, d[it].z, d[it].w, TWOD ? tile_word : sw[it]);
            if ((it & 1) == 0) {
                o_even = o;
            } else {
                // even lane: 16 codes of the even row; odd lane: 16 codes of the odd row
                const uint2 send = odd ? o_even : o;
                const uint2 recv = make_uint2(dpp_xor1(send.x), dpp_xor1(send.y));
                const uint4 out = odd ? make_uint4(recv.x, recv.y, o.x, o.y) : make_uint4(o_even.x, o_even.y, recv.x, recv.y);
                const int rr = odd ? it : it - 1;
                if (rbase + rr < valid) store16_streaming(dst + (int64_t)rr * a.cols, out);
            }
        }
    }

    // ---- transposed copy: column 8 c16 + j of the lane's 8 rows = 8 bytes of output row col0 + 8 c16 + j ----
    if (want_col) {
        uint32_t sw[8];
        if (!TWOD) {
            const uint4 s0 = *(const uint4*)&scale_c[8 * c16], s1 = *(const uint4*)&scale_c[8 * c16 + 4];
            sw[0] = s0.x; sw[1] = s0.y; sw[2] = s0.z; sw[3] = s0.w;
            sw[4] = s1.x; sw[5] = s1.y; sw[6] = s1.z; sw[7] = s1.w;
        }
        const uint32_t* dw = (const uint32_t*)d;  // dw[it * 4 + j / 2]: columns j, j + 1 (j even) of row `it`
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t pr[4];   // rows (2 i, 2 i + 1) of column j
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t lo = dw[(2 * i) * 4 + (j >> 1)], hi = dw[(2 * i + 1) * 4 + (j >> 1)];
                pr[i] = (j & 1) ? ((lo >> 16) | (hi & 0xFFFF0000u)) : ((lo & 0xFFFFu) | (hi << 16));
            }
            *(uint2*)(t_tile + (8 * c16 + j) * BW_TPITCH + rbase) = bw_cvt8<FMT>(pr[0], pr[1], pr[2], pr[3], TWOD ? tile_word : sw[j]);
        }
        __syncthreads();
        // rows past the end hold zero codes (or NaN codes in a block with a NaN or an infinity)
        uint8_t* dst = a.q_colT + (zoff * a.cols + col0) * rows_pad + prow0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = (t >> 3) + 32 * i, ch = t & 7;
            store16_streaming(dst + (int64_t)c * rows_pad + 16 * ch, *(const uint4*)(t_tile + c * BW_TPITCH + 16 * ch));
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// GEMM.  c[m, n] (bf16) = sum_kb sa[m, kb] * sb[n >> sb_shift, kb] * (a[m, kb-th 128] . b[n, kb-th 128]),
// a[m_rows, k], b[n, k] FP8 codes, k % 128 == 0, n % 128 == 0; sb_shift = 0 (a factor per row of b) or 7 (per
// 128 rows: weights).
// Workgroup = 8 waves (two per SIMD) on a 128 x 256 output tile, wave (wm, wn) = 64 x 64 = 2 x 2 MFMA tiles of
// 32 x 32 with two accumulator sets of 64 registers.  K advances in blocks of 128 through a ring of three LDS stages
// (128 + 256 rows x 128 bytes = 48 KiB each) filled by LDS-direct loads two blocks ahead: a request has two K blocks
// of MFMA work (about a microsecond) to land, where a register-staged prefetch of one block left the pipe waiting
// for memory most of the time (1.1 PFLOP/s on the Llama MLP shapes).  16-byte pieces are XOR-swizzled by the row on the global side, so
// the fragment reads are conflict-free ds_read_b128.  The two waves of a SIMD cover each other: while one multiplies
// its block's partial sums into the accumulators (64 FMAs per lane), the other's MFMAs run.  The factors of a block
// are fetched one block ahead with plain loads and handed round through LDS.  Rows past the end of a group or of
// the operand are dropped by the buffer descriptor's range check (it covers the per-lane and the scalar offset) and
// read as zero.
// ------------------------------------------------------------------------------------------------------------
struct BwGemmArgs {
    const uint8_t* a;
    const float* sa;
    const uint8_t* b;
    const float* sb;
    uint16_t* c;
    int64_t m, n, k;
    int64_t ldc;        // elements between rows of c (n, unless the launch covers a range of a wider output's columns)
    int sb_shift;
    // mode 0: one dense GEMM.  mode 1 (forward / dgrad of a grouped linear): the rows of a are split by group_lens, b is
    // [num_groups, n, k] with its factors per group, a row tile belongs to one group.  mode 2 (wgrad of a grouped
    // linear): a [m, k] and b [n, k] are transposed segment-padded copies, group z = blockIdx.z contracts over its
    // segment of k only and writes c[z] (zeros for a group without tokens).
    int mode;
    const int64_t* group_lens;
    int num_groups;
};

constexpr int BWG_THREADS = 512;
constexpr int BWG_BM = 128, BWG_BN = 256;
constexpr int BWG_A = BWG_BM * BW, BWG_B = BWG_BN * BW, BWG_STAGE = BWG_A + BWG_B;      // 16 + 32 KiB
constexpr int BWG_STAGES = 3;
constexpr int BWG_FAC = (BWG_BM + BWG_BN) * 4;                                            // factors of one K block
constexpr int BW_GEMM_LDS = BWG_STAGES * (BWG_STAGE + BWG_FAC);

__device__ __forceinline__ v4i bw_rsrc(const void* base, int64_t bytes) {
    const uint64_t p = (uint64_t)base;
    const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32) & 0xFFFF);
    r[2] = __builtin_amdgcn_readfirstlane((int)n);
    r[3] = 0x00020000;
    return r;
}
// LDS-direct 16-byte load: lane i's data lands at lds_off + 16 i (M0 holds nothing else in this kernel)
__device__ __forceinline__ void bw_dma16(v4i rsrc, uint32_t lds_off, uint32_t voff, uint32_t soff) {
    asm volatile("" : "+s"(soff));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_off), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}

// SBU: b's factors are per 128 rows (a weight's 128 x 128 blocks), i.e. one value for the wave's 64 columns: the
// block's factor product is two multiplications per lane instead of 64.
template <int AFMT, int BFMT, bool SBU>
__global__ __launch_bounds__(BWG_THREADS) void bw_gemm_kernel(BwGemmArgs p) {
    constexpr int CB = BFMT == kFmtE5M2 ? 1 : 0, BL = AFMT == kFmtE5M2 ? 1 : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t bw_smem[];
    float* fac_base = (float*)(bw_smem + BWG_STAGES * BWG_STAGE);        // [stage][a: 128 | b: 256]
    __shared__ int grp_pre[BW_MAX_GROUPS + 1];
    __shared__ int64_t grp_red[BWG_THREADS / 64];
    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5, wm = w >> 2, wn = w & 3;
    const uint32_t smem_base = (uint32_t)(uintptr_t)bw_smem;
    int64_t row0 = (int64_t)blockIdx.y * BWG_BM;
    const int64_t col0 = (int64_t)blockIdx.x * BWG_BN;
    const int64_t kb_n = p.k / BW;
    int64_t m_end = p.m, b_group = 0, c_group = 0, kb0 = 0, kb1 = kb_n;
    if (p.mode == 1) {
        int tile_in_group;
        int64_t before, len;
        const int grp = bw_locate<BWG_THREADS>(p.group_lens, p.num_groups, (int)blockIdx.y, grp_pre, grp_red, tile_in_group, before, len);
        if (grp < 0) return;                     // the grid is sized for the worst case (every group with a ragged tile)
        row0 = before + (int64_t)tile_in_group * BWG_BM;
        m_end = before + len < p.m ? before + len : p.m;
        if (row0 >= m_end) return;
        b_group = grp;
    } else if (p.mode == 2) {
        // this group's segment of the contraction: [sum of the padded lens in front, + its own padded len), in blocks
        const int grp = (int)blockIdx.z;
        int64_t part = 0;
        for (int j = t; j < grp; j += BWG_THREADS) part += ((p.group_lens[j] > 0 ? p.group_lens[j] : 0) + BW - 1) / BW;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) part += __shfl_xor(part, d);
        if ((t & 63) == 0) grp_red[t >> 6] = part;
        __syncthreads();
        kb0 = 0;
#pragma unroll
        for (int i = 0; i < BWG_THREADS / 64; ++i) kb0 += grp_red[i];
        kb1 = kb0 + ((p.group_lens[grp] > 0 ? p.group_lens[grp] : 0) + BW - 1) / BW;
        kb0 = kb0 > kb_n ? kb_n : kb0;           // lens that claim more than the operands hold
        kb1 = kb1 > kb_n ? kb_n : kb1;
        c_group = grp;
    }
    const int64_t pm = m_end, pk = p.k, pn = p.n;
    const int sb_shift = p.sb_shift;
    const float* const psa = p.sa;
    const float* const psb = p.sb + b_group * (pn >> sb_shift) * kb_n;
    uint16_t* const pc_out = p.c + c_group * p.m * p.ldc;
    const int64_t ldc = p.ldc;
    // descriptors: from the tile's first row to the last row that may be read (the group's / the operand's end for a,
    // the end of the group's matrix for b); offsets inside them are 32-bit (the host bounds 256 rows x k)
    const uint8_t* const b_mat = p.b + b_group * pn * pk;
    const v4i ra = bw_rsrc(p.a + row0 * pk, (pm - row0) * pk);
    const v4i rb = bw_rsrc(b_mat + col0 * pk, (pn - col0) * pk);
    // loader geometry: a round is 512 pieces of 16 bytes = 64 rows x 128 bytes; lane i of wave w lands at chunk
    // offset 1024 w + 16 i, i.e. row 8 w + i / 8, LDS piece i % 8, and fetches global piece (i % 8) ^ ((row / 2) % 8):
    // the 16 rows that one cycle of a ds_read_b128 serves (two rows share a 256-byte bank period) then hit 16
    // different 16-byte bank groups (XOR by row % 8 left rows r and r + 8 on the same one: half of the LDS cycles
    // were bank conflicts)
    const int ld_row = t >> 3;
    const uint32_t ld_voff = (uint32_t)(ld_row * pk + 16 * ((t & 7) ^ ((ld_row >> 1) & 7)));
    const uint32_t round_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(64 * pk));
    const uint32_t wave_lds = smem_base + (uint32_t)(w * 1024);
    auto issue = [&](uint32_t koff, int stage) __attribute__((always_inline)) {
        const uint32_t base = wave_lds + (uint32_t)(stage * BWG_STAGE);
#pragma unroll
        for (int e = 0; e < 2; ++e) bw_dma16(ra, base + e * 8192, ld_voff, koff + e * round_bytes);
#pragma unroll
        for (int e = 0; e < 4; ++e) bw_dma16(rb, base + BWG_A + e * 8192, ld_voff, koff + e * round_bytes);
    };
    // Factors of a K block, one dword per lane straight into LDS (lane i of wave w lands at word 64 w + i): waves 0, 1
    // fetch a's 128 row factors, waves 2 .. 5 b's 256 (per row of b, or one per 128 rows); waves 6, 7 repeat the
    // requests of waves 4, 5 (the same bytes to the same place), so that every wave has the same number of requests in
    // flight.  Rows past the end of the group or of b are dropped by the descriptors and read as zero.
    const int fw = w < 6 ? w : w - 2;
    const bool f_a = fw < 2;
    const int frow = f_a ? fw * 64 + l : fw * 64 + l - BWG_BM;
    const v4i rfac = f_a ? bw_rsrc(psa + row0 * kb_n, (pm - row0) * kb_n * 4)
                         : bw_rsrc(psb + (col0 >> sb_shift) * kb_n, (((pn - col0) + (1 << sb_shift) - 1) >> sb_shift) * kb_n * 4);
    const uint32_t fac_voff = (uint32_t)(((f_a ? frow : (frow >> sb_shift)) * kb_n) * 4);
    const uint32_t fac_lds = smem_base + (uint32_t)(BWG_STAGES * BWG_STAGE + fw * 256);
    auto issue_fac = [&](uint32_t soff, int stage) __attribute__((always_inline)) {
        const uint32_t lds = fac_lds + (uint32_t)(stage * BWG_FAC);
        asm volatile("" : "+s"(soff));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                     :
                     : "s"(lds), "v"(fac_voff), "s"(rfac), "s"(soff)
                     : "memory");
    };

    bv16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // pipeline: two blocks ahead.  A wave's requests for a block are its six operand rounds and one factor request; at the
    // top of block kb everything but the seven requests of block kb + 1 has landed.  Requests for blocks past the range go
    // out as well, at an offset of 2 GiB, where the descriptors' range check drops them (or, under an operand that large,
    // they fetch bytes of it that nobody reads): the request count per block is then a constant, and the block's
    // instructions stay one basic block whose order can be pinned (a branch around the requests lets the compiler sink
    // the MFMAs behind every load).
    constexpr uint32_t DROP = 0x80000000u;
    const int k0 = __builtin_amdgcn_readfirstlane((int)kb0), k1 = __builtin_amdgcn_readfirstlane((int)kb1);   // (k is below 2^23)
    if (k0 < k1) {
        issue((uint32_t)(k0 * BW), 0);
        issue_fac((uint32_t)(k0 * 4), 0);
        const bool two = k0 + 1 < k1;
        issue(two ? (uint32_t)((k0 + 1) * BW) : DROP, 1);
        issue_fac(two ? (uint32_t)((k0 + 1) * 4) : DROP, 1);
    }
    // fragment addressing: lane (lr, g) reads the 16-byte pieces 4 ks + 2 h + g of its row, swizzled by the row
    const int swz = (lr >> 1) & 7;
    uint32_t piece[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int h = 0; h < 2; ++h) piece[ks][h] = (uint32_t)(16 * ((4 * ks + 2 * h + g) ^ swz));
    const uint32_t a_row = (uint32_t)((wm * 64 + lr) * BW), b_row = (uint32_t)(BWG_A + (wn * 64 + lr) * BW);
    int st = 0, st2 = 2;                          // stage of block kb, stage of block kb + 2
    for (int kb = k0; kb < k1; ++kb) {
        asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
        __syncthreads();       // block kb and its factors are in LDS for every wave; every wave has left block kb - 1
        const bool more = kb + 2 < k1;
        const uint32_t in_koff = more ? (uint32_t)__builtin_amdgcn_readfirstlane((kb + 2) * BW) : DROP;
        const uint32_t in_fac = more ? (uint32_t)__builtin_amdgcn_readfirstlane((kb + 2) * 4) : DROP;
        const uint32_t in_base = wave_lds + (uint32_t)(st2 * BWG_STAGE);
        const float* fac = fac_base + st * (BWG_BM + BWG_BN);
        const uint8_t* stg = bw_smem + st * BWG_STAGE;
        auto frag = [&](uint32_t row_off, int ks) __attribute__((always_inline)) {
            const uint4 lo = *(const uint4*)(stg + row_off + piece[ks][0]);
            const uint4 hi = *(const uint4*)(stg + row_off + piece[ks][1]);
            return bv8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        };
        const float sbu = SBU ? fac[BWG_BM + wn * 64] : 0.f;
        float sa[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) sa[i] = fac[wm * 64 + i * 32 + lr];
        __builtin_amdgcn_sched_barrier(0);
        // fragment reads in the order the MFMAs want them (tile (0, 0) first)
        bv8i fa8[2][2], fb8[2][2];      // [fragment][ks]
        fb8[0][0] = frag(b_row, 0);
        fa8[0][0] = frag(a_row, 0);
        __builtin_amdgcn_sched_barrier(0);
        fb8[0][1] = frag(b_row, 1);
        fa8[0][1] = frag(a_row, 1);
        __builtin_amdgcn_sched_barrier(0);
        fb8[1][0] = frag(b_row + 32 * BW, 0);
        fb8[1][1] = frag(b_row + 32 * BW, 1);
        fa8[1][0] = frag(a_row + 32 * BW, 0);
        fa8[1][1] = frag(a_row + 32 * BW, 1);
        __builtin_amdgcn_sched_barrier(0);
        bv16f zero;
#pragma unroll
        for (int e = 0; e < 16; ++e) zero[e] = 0.f;
        // acc += part * (sa[row] * sb[col]): lane (lr, g), register e = 4 q + r of tile (i, j) is row i * 32 + lr,
        // column j * 32 + 8 q + 4 g + r of the wave's 64 x 64
        auto scale_in = [&](const bv16f& part, int i, int j) __attribute__((always_inline)) {
            const float sab = sa[i] * sbu;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (SBU) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = fmaf(part[4 * q + e], sab, acc[i][j][4 * q + e]);
                } else {
                    const float4 sb = *(const float4*)(&fac[BWG_BM + wn * 64 + j * 32 + 8 * q + 4 * g]);
                    acc[i][j][4 * q + 0] = fmaf(part[4 * q + 0], sa[i] * sb.x, acc[i][j][4 * q + 0]);
                    acc[i][j][4 * q + 1] = fmaf(part[4 * q + 1], sa[i] * sb.y, acc[i][j][4 * q + 1]);
                    acc[i][j][4 * q + 2] = fmaf(part[4 * q + 2], sa[i] * sb.z, acc[i][j][4 * q + 2]);
                    acc[i][j][4 * q + 3] = fmaf(part[4 * q + 3], sa[i] * sb.w, acc[i][j][4 * q + 3]);
                }
            }
        };
        // request number mi of block kb + 2, one behind each of this block's first seven MFMAs: six operand rounds, the factors
#define REQ(mi)                                                                                                        \
    do {                                                                                                               \
        if ((mi) < 2) bw_dma16(ra, in_base + (mi) * 8192, ld_voff, in_koff + (mi) * round_bytes);                          \
        else if ((mi) < 6) bw_dma16(rb, in_base + BWG_A + ((mi) - 2) * 8192, ld_voff, in_koff + ((mi) - 2) * round_bytes); \
        else if ((mi) == 6) issue_fac(in_fac, st2);                                                                    \
    } while (0)
        // The four 32 x 32 tiles one after the other, two MFMAs each (the b fragment is the first operand: a lane ends up
        // with 4 consecutive output columns); the FMAs of a tile run in the shadow of the next tile's MFMAs.
        bv16f part[4];
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            const int i = tl >> 1, j = tl & 1;
            part[tl] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[j][0], fa8[i][0], zero, CB, BL, 0, 127, 0, 127);
            REQ(2 * tl);
            part[tl] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[j][1], fa8[i][1], part[tl], CB, BL, 0, 127, 0, 127);
            REQ(2 * tl + 1);
            __builtin_amdgcn_sched_barrier(0);
            if (tl > 0) scale_in(part[tl - 1], (tl - 1) >> 1, (tl - 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
        }
#undef REQ
        scale_in(part[3], 1, 1);
        st = st == BWG_STAGES - 1 ? 0 : st + 1;
        st2 = st2 == BWG_STAGES - 1 ? 0 : st2 + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // (dropped requests included: none may outlive the workgroup's LDS)
    if ((((uintptr_t)pc_out) & 15) == 0) {
        __syncthreads();   // no request of any wave still writes LDS: the stages are free
        // Output through a wave-private LDS patch of 32 rows x 128 bytes, one a fragment at a time: a lane's four
        // consecutive bf16 go in as 8 bytes and come out as 16 bytes per lane, 8 rows x 128 contiguous bytes per store
        // instruction (16-byte pieces XOR-swizzled by the row).
        uint8_t* const patch = bw_smem + w * (2 * 32 * 128);   // (one patch per a fragment, both written before the first is read back)
        const bool cols_in = col0 + wn * 64 < pn;        // (n is a multiple of 128: the wave's columns are in or out as a whole)
        const int er = l >> 3, ep = l & 7;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const bv4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                     (__bf16)acc[i][j][4 * q + 3]};
                    *(bv4bf*)(patch + i * (32 * 128) + lr * 128 + 16 * ((4 * j + q) ^ ((lr >> 1) & 7)) + 8 * g) = o;
                }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int r = 8 * u + er;
                const uint4 v = *(const uint4*)(patch + i * (32 * 128) + r * 128 + 16 * (ep ^ ((r >> 1) & 7)));
                const int64_t m = row0 + wm * 64 + i * 32 + r;
                if (cols_in && m < pm) store16_streaming(pc_out + m * ldc + col0 + wn * 64 + 8 * ep, v);
            }
        return;
    }
    // an output that is only 8-byte aligned: stored straight from the accumulator layout
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t m = row0 + wm * 64 + i * 32 + lr;
        if (m >= pm) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t col = col0 + wn * 64 + j * 32 + 8 * q + 4 * g;
                if (col >= pn) continue;     // (n is a multiple of 128: a quad is in or out as a whole)
                const bv4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                 (__bf16)acc[i][j][4 * q + 3]};
                *(bv4bf*)(pc_out + m * ldc + col) = o;
            }
    }
}

// ------------------------------------------------------------------------------------------------------------
// The same GEMM on a 256 x 256 tile, for problems with enough of them to fill the chip: a third fewer operand bytes
// per flop travel from L2 to LDS (what the 128 x 256 kernel waits for most) and half as many barriers and tiles.
// 8 waves as 4 x 2, a wave owns 64 rows x 128 columns = 2 x 4 MFMA tiles (128 accumulator registers); the partial
// sums of only ONE column of tiles (2 x 16 registers) exist at a time: for each of the four b fragments of a K block,
// 4 MFMAs (both a fragments, both halves of the block) add up from zero and are multiplied into the accumulators
// in the shadow of the following MFMAs.  Same MFMA and FMA order per output element as the 128 x 256 kernel, so the
// same bits.  Two LDS stages of 64 KiB (a K block of both operands) + factors: the requests of block kb + 1 go out
// behind the first nine MFMAs of block kb, into the stage block kb - 1 has left.
// One workgroup per tile, like the 128 x 256 kernel (a persistent form, whose last K block requests the first block of
// the workgroup's next tile, was built and measured: no faster -- workgroups in lockstep all reach their epilogues at
// once, and the burst of stores costs what the saved dispatches gain).
// ------------------------------------------------------------------------------------------------------------
constexpr int BWH_BM = 256, BWH_BN = 256;
constexpr int BWH_A = BWH_BM * BW, BWH_STAGE = (BWH_BM + BWH_BN) * BW;      // 32 + 32 KiB
constexpr int BWH_FAC = (BWH_BM + BWH_BN) * 4;
constexpr int BW_GEMM256_LDS = 2 * (BWH_STAGE + BWH_FAC);

template <int AFMT, int BFMT, bool SBU>
__global__ __launch_bounds__(BWG_THREADS) void bw_gemm256_kernel(BwGemmArgs p) {
    constexpr int CB = BFMT == kFmtE5M2 ? 1 : 0, BL = AFMT == kFmtE5M2 ? 1 : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t bw_smem[];
    float* fac_base = (float*)(bw_smem + 2 * BWH_STAGE);                 // [stage][a: 256 | b: 256]
    __shared__ int grp_pre[BW_MAX_GROUPS + 1];
    __shared__ int64_t grp_red[BWG_THREADS / 64];
    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5, wm = w >> 1, wn = w & 1;
    const uint32_t smem_base = (uint32_t)(uintptr_t)bw_smem;
    int64_t row0 = (int64_t)blockIdx.y * BWH_BM;
    const int64_t col0 = (int64_t)blockIdx.x * BWH_BN;
    const int64_t kb_n = p.k / BW;
    int64_t m_end = p.m, b_group = 0, c_group = 0, kb0 = 0, kb1 = kb_n;
    if (p.mode == 1) {
        int tile_in_group;
        int64_t before, len;
        const int grp = bw_locate<BWG_THREADS, BWH_BM>(p.group_lens, p.num_groups, (int)blockIdx.y, grp_pre, grp_red, tile_in_group, before, len);
        if (grp < 0) return;                     // the grid is sized for the worst case (every group with a ragged tile)
        row0 = before + (int64_t)tile_in_group * BWH_BM;
        m_end = before + len < p.m ? before + len : p.m;
        if (row0 >= m_end) return;
        b_group = grp;
    } else if (p.mode == 2) {
        // this group's segment of the contraction: [sum of the padded lens in front, + its own padded len), in blocks
        const int grp = (int)blockIdx.z;
        int64_t part = 0;
        for (int j = t; j < grp; j += BWG_THREADS) part += ((p.group_lens[j] > 0 ? p.group_lens[j] : 0) + BW - 1) / BW;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) part += __shfl_xor(part, d);
        if ((t & 63) == 0) grp_red[t >> 6] = part;
        __syncthreads();
        kb0 = 0;
#pragma unroll
        for (int i = 0; i < BWG_THREADS / 64; ++i) kb0 += grp_red[i];
        kb1 = kb0 + ((p.group_lens[grp] > 0 ? p.group_lens[grp] : 0) + BW - 1) / BW;
        kb0 = kb0 > kb_n ? kb_n : kb0;           // lens that claim more than the operands hold
        kb1 = kb1 > kb_n ? kb_n : kb1;
        c_group = grp;
    }
    const int64_t pm = m_end, pk = p.k, pn = p.n;
    const int sb_shift = p.sb_shift;
    const float* const psb = p.sb + b_group * (pn >> sb_shift) * kb_n;
    uint16_t* const pc_out = p.c + c_group * p.m * p.ldc;
    const int64_t ldc = p.ldc;
    // descriptors: from the tile's first row to the last row that may be read (the group's / the operand's end for a,
    // the end of the group's matrix for b); offsets inside them are 32-bit (the host bounds 256 rows x k)
    const v4i ra = bw_rsrc(p.a + row0 * pk, (pm - row0) * pk);
    const v4i rb = bw_rsrc(p.b + b_group * pn * pk + col0 * pk, (pn - col0) * pk);
    // loader geometry as in the 128 x 256 kernel: a round = 64 rows x 128 bytes, piece (i % 8) ^ ((row / 2) % 8)
    const int ld_row = t >> 3;
    const uint32_t ld_voff = (uint32_t)(ld_row * pk + 16 * ((t & 7) ^ ((ld_row >> 1) & 7)));
    const uint32_t round_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(64 * pk));
    const uint32_t wave_lds = smem_base + (uint32_t)(w * 1024);
    // factors: waves 0 .. 3 fetch a's 256 row factors, waves 4 .. 7 b's (lane i of wave w lands at word 64 w + i)
    const bool f_a = w < 4;
    const int frow = f_a ? t : t - BWH_BM;
    const uint32_t fac_voff = (uint32_t)(((f_a ? frow : (frow >> sb_shift)) * kb_n) * 4);
    const uint32_t fac_lds = smem_base + (uint32_t)(2 * BWH_STAGE + w * 256);
    const v4i rfac = f_a ? bw_rsrc(p.sa + row0 * kb_n, (pm - row0) * kb_n * 4)
                         : bw_rsrc(psb + (col0 >> sb_shift) * kb_n, (((pn - col0) + (1 << sb_shift) - 1) >> sb_shift) * kb_n * 4);
    // round e of a block: 0 .. 3 the a rows, 4 .. 7 the b rows
    auto issue_round = [&](uint32_t koff, uint32_t base, int e) __attribute__((always_inline)) {
        if (e < 4) bw_dma16(ra, base + e * 8192, ld_voff, koff + e * round_bytes);
        else bw_dma16(rb, base + BWH_A + (e - 4) * 8192, ld_voff, koff + (e - 4) * round_bytes);
    };
    auto issue_fac = [&](uint32_t soff, int stage) __attribute__((always_inline)) {
        const uint32_t lds = fac_lds + (uint32_t)(stage * BWH_FAC);
        asm volatile("" : "+s"(soff));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                     :
                     : "s"(lds), "v"(fac_voff), "s"(rfac), "s"(soff)
                     : "memory");
    };
    // fragment addressing: lane (lr, g) reads the 16-byte pieces 4 ks + 2 h + g of its row, swizzled by the row
    const int swz = (lr >> 1) & 7;
    uint32_t piece[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int h = 0; h < 2; ++h) piece[ks][h] = (uint32_t)(16 * ((4 * ks + 2 * h + g) ^ swz));
    const uint32_t a_row = (uint32_t)((wm * 64 + lr) * BW), b_row = (uint32_t)(BWH_A + (wn * 128 + lr) * BW);

    bv16f acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    const int k0 = __builtin_amdgcn_readfirstlane((int)kb0), k1 = __builtin_amdgcn_readfirstlane((int)kb1);
    if (k0 < k1) {
        const uint32_t koff = (uint32_t)__builtin_amdgcn_readfirstlane(k0 * BW);
#pragma unroll
        for (int e = 0; e < 8; ++e) issue_round(koff, wave_lds, e);
        issue_fac((uint32_t)__builtin_amdgcn_readfirstlane(k0 * 4), 0);
    }
    const bool wave_live = __builtin_amdgcn_readfirstlane((int)(row0 + wm * 64 < pm && col0 + wn * 128 < pn)) != 0;
    int st = 0;
    for (int kb = k0; kb < k1; ++kb) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // block kb and its factors are in LDS for every wave; every wave has left the other stage
        // The requests of block kb + 1 go out behind this block's MFMAs.  In the last block they go out as well, at
        // an offset of 2 GiB: past the end of what the descriptor covers they are dropped (or, under an operand that
        // large, fetch bytes of it that nobody reads) -- a branch between the MFMAs would split the block's
        // instructions into basic blocks, and the order below, which the register budget depends on, would not
        // survive that.
        const bool follows = kb + 1 < k1;
        const uint32_t in_koff = follows ? (uint32_t)__builtin_amdgcn_readfirstlane((kb + 1) * BW) : 0x80000000u;
        const uint32_t in_fac = follows ? (uint32_t)__builtin_amdgcn_readfirstlane((kb + 1) * 4) : 0x80000000u;
        const uint32_t in_base = wave_lds + (uint32_t)((st ^ 1) * BWH_STAGE);
        if (!wave_live) {
            // all of this wave's rows (or columns) lie past the end of the tile: it only keeps its share of the requests
            // going, and the wave it shares a SIMD with has the MFMA pipe to itself
#pragma unroll
            for (int e = 0; e < 8; ++e) issue_round(in_koff, in_base, e);
            issue_fac(in_fac, st ^ 1);
            st ^= 1;
            continue;
        }
        const float* fac = fac_base + st * (BWH_BM + BWH_BN);
        const uint8_t* stg = bw_smem + st * BWH_STAGE;
        auto frag = [&](uint32_t row_off, int ks) __attribute__((always_inline)) {
            const uint4 lo = *(const uint4*)(stg + row_off + piece[ks][0]);
            const uint4 hi = *(const uint4*)(stg + row_off + piece[ks][1]);
            return bv8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        };
        // fragment reads in the order the MFMAs want them: all eight waves read at once behind the barrier, and the
        // first MFMA should wait for 4 of a wave's 12 reads, not for 10
        const float sbu = SBU ? fac[BWH_BM + wn * 128] : 0.f;
        float sa[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) sa[i] = fac[wm * 64 + i * 32 + lr];
        __builtin_amdgcn_sched_barrier(0);
        bv8i fa8[2][2], fb8[2];      // [a fragment][ks], [ks]
        fb8[0] = frag(b_row, 0);
        fa8[0][0] = frag(a_row, 0);
        __builtin_amdgcn_sched_barrier(0);
        fb8[1] = frag(b_row, 1);
        fa8[0][1] = frag(a_row, 1);
        __builtin_amdgcn_sched_barrier(0);
        fa8[1][0] = frag(a_row + 32 * BW, 0);
        fa8[1][1] = frag(a_row + 32 * BW, 1);
        bv16f zero;
#pragma unroll
        for (int e = 0; e < 16; ++e) zero[e] = 0.f;
        // acc += part * (sa[row] * sb[col]): lane (lr, g), register e = 4 q + r of tile (i, j) is row i * 32 + lr,
        // column j * 32 + 8 q + 4 g + r of the wave's 64 x 128
        auto scale_in = [&](const bv16f& part, int i, int j) __attribute__((always_inline)) {
            const float sab = sa[i] * sbu;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (SBU) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = fmaf(part[4 * q + e], sab, acc[i][j][4 * q + e]);
                } else {
                    const float4 sb = *(const float4*)(&fac[BWH_BM + wn * 128 + j * 32 + 8 * q + 4 * g]);
                    acc[i][j][4 * q + 0] = fmaf(part[4 * q + 0], sa[i] * sb.x, acc[i][j][4 * q + 0]);
                    acc[i][j][4 * q + 1] = fmaf(part[4 * q + 1], sa[i] * sb.y, acc[i][j][4 * q + 1]);
                    acc[i][j][4 * q + 2] = fmaf(part[4 * q + 2], sa[i] * sb.z, acc[i][j][4 * q + 2]);
                    acc[i][j][4 * q + 3] = fmaf(part[4 * q + 3], sa[i] * sb.w, acc[i][j][4 * q + 3]);
                }
            }
        };
        // request number mi (one behind each of the block's first nine MFMAs): the eight operand rounds, then the factors
#define REQ(mi)                                            \
    do {                                                   \
        if ((mi) < 8) issue_round(in_koff, in_base, (mi)); \
        else if ((mi) == 8) issue_fac(in_fac, st ^ 1);     \
    } while (0)
        // Per b fragment j: the two MFMAs of a fragment 0, the FMAs of the previous fragment's second tile in their
        // shadow, the two MFMAs of a fragment 1 (each half of the b fragment gives its registers to the next
        // fragment's half as soon as its last MFMA has gone), the FMAs of this fragment's first tile.  The b
        // fragment is the MFMA's first operand: a lane ends up with 4 consecutive output columns.
        bv16f part0, part1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            part0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[0], fa8[0][0], zero, CB, BL, 0, 127, 0, 127);
            REQ(4 * j);
            part0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[1], fa8[0][1], part0, CB, BL, 0, 127, 0, 127);
            REQ(4 * j + 1);
            __builtin_amdgcn_sched_barrier(0);
            if (j > 0) scale_in(part1, 1, j - 1);
            __builtin_amdgcn_sched_barrier(0);
            part1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[0], fa8[1][0], zero, CB, BL, 0, 127, 0, 127);
            REQ(4 * j + 2);
            __builtin_amdgcn_sched_barrier(0);
            if (j < 3) fb8[0] = frag(b_row + (j + 1) * 32 * BW, 0);
            part1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[1], fa8[1][1], part1, CB, BL, 0, 127, 0, 127);
            REQ(4 * j + 3);
            __builtin_amdgcn_sched_barrier(0);
            if (j < 3) fb8[1] = frag(b_row + (j + 1) * 32 * BW, 1);
            scale_in(part0, 0, j);
            __builtin_amdgcn_sched_barrier(0);
        }
#undef REQ
        scale_in(part1, 1, 3);
        st ^= 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // no request of any wave (the last block's dropped ones included) still writes LDS: the stages are free
    // Output through a wave-private LDS patch of 32 rows x 256 bytes, one a fragment at a time: a lane's four
    // consecutive bf16 go in as 8 bytes and come out as 16 bytes per lane, 4 rows x 256 contiguous bytes per store
    // instruction (16-byte pieces XOR-swizzled by the row).  Stored straight from the accumulator layout, 16 bytes per
    // row and instruction, the partial lines cost a K = 4096 tile 5 % of its time.
    uint8_t* const patch = bw_smem + w * (2 * 32 * 256);     // (one patch per a fragment: the two stages hold all sixteen)
    const bool cols_in = col0 + wn * 128 < pn;       // (n is a multiple of 128: the wave's columns are in or out as a whole)
    const int er = l >> 4, ep = l & 15;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bv4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                 (__bf16)acc[i][j][4 * q + 3]};
                *(bv4bf*)(patch + i * (32 * 256) + lr * 256 + 16 * ((4 * j + q) ^ (lr & 15)) + 8 * g) = o;
            }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int r = 4 * u + er;
            const uint4 v = *(const uint4*)(patch + i * (32 * 256) + r * 256 + 16 * (ep ^ (r & 15)));
            const int64_t m = row0 + wm * 64 + i * 32 + r;
            if (cols_in && m < pm) store16_streaming(pc_out + m * ldc + col0 + wn * 128 + 8 * ep, v);
        }
}

template <bool TWOD>
static int launch_bw_quant(const BwQuantArgs& a, int fmt, int64_t row_tiles, int batch, hipStream_t st) {
    const int64_t wgs = (int64_t)(a.n_super + 7) / 8 * 8 * 64;
    if (wgs > 0x7FFFFFFF) return MXL_EINVAL;
    const dim3 grid((unsigned)wgs, (unsigned)batch);
    if (fmt == MXL_FMT_E4M3) hipLaunchKernelGGL((bw_quant_kernel<MXL_FMT_E4M3, TWOD>), grid, dim3(BW_THREADS), 0, st, a);
    else hipLaunchKernelGGL((bw_quant_kernel<MXL_FMT_E5M2, TWOD>), grid, dim3(BW_THREADS), 0, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

static int bw_quant(const void* x, int64_t rows, int64_t cols, int fmt, const int64_t* group_lens, int num_groups, int batch,
                    void* q_row, void* sinv_row, void* q_colT, void* sinv_colT, bool twod, void* stream) {
    if (rows < 0 || cols <= 0 || cols % BW != 0 || (fmt != MXL_FMT_E4M3 && fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if ((q_row == nullptr) != (sinv_row == nullptr) || (q_colT == nullptr) != (sinv_colT == nullptr)) return MXL_EINVAL;
    if (!q_row && !q_colT) return MXL_EINVAL;
    if (batch < 1 || batch > 65535 || (twod && rows % BW != 0) || (!twod && batch != 1)) return MXL_EINVAL;
    if (num_groups < 0 || num_groups > BW_MAX_GROUPS || (num_groups > 0) != (group_lens != nullptr) || (twod && num_groups)) return MXL_EINVAL;
    const int64_t W = num_groups ? mxl_padded_width(rows, num_groups) : (rows + BW - 1) / BW * BW;
    const int64_t row_tiles = W / BW;       // with groups: the 128-column pieces of the padded transposed copy
    if (row_tiles == 0) return MXL_OK;
    if (!x && rows > 0) return MXL_EINVAL;
    if (((uintptr_t)x & 15) != 0 || row_tiles > 65535) return MXL_EINVAL;
    if ((((uintptr_t)q_row | (uintptr_t)q_colT) & 15) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const int tiles_c = (int)(cols / BW), super_c = (tiles_c + 7) / 8, super_r = (int)((row_tiles + 7) / 8);
    if ((int64_t)super_c * super_r > 0x7FFFFFF) return MXL_EINVAL;
    BwQuantArgs a{(const uint16_t*)x, rows, cols, (uint8_t*)q_row, (float*)sinv_row, (uint8_t*)q_colT, (float*)sinv_colT,
                  group_lens, num_groups, W, (int)row_tiles, tiles_c, super_c, super_c * super_r};
    return twod ? launch_bw_quant<true>(a, fmt, row_tiles, batch, (hipStream_t)stream)
                : launch_bw_quant<false>(a, fmt, row_tiles, 1, (hipStream_t)stream);
}

// The dynamic LDS size is above the default limit.  The attribute belongs to the (kernel, device) pair and is set at
// the first launch on a device -- not at every launch: a launch may be recorded by a stream capture, which is no
// place for a call that changes function state.
template <int AFMT, int BFMT, bool SBU, bool TALL>
static int launch_bw_gemm(const BwGemmArgs& g, dim3 grid, hipStream_t st) {
    static std::atomic<bool> attr_set[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MXL_ELAUNCH;
    const int slot = dev & 63;
    constexpr int lds = TALL ? BW_GEMM256_LDS : BW_GEMM_LDS;
    const void* kern = TALL ? (const void*)bw_gemm256_kernel<AFMT, BFMT, SBU> : (const void*)bw_gemm_kernel<AFMT, BFMT, SBU>;
    if (!attr_set[slot].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return MXL_ELAUNCH;
        attr_set[slot].store(true, std::memory_order_release);
    }
    if (TALL) hipLaunchKernelGGL((bw_gemm256_kernel<AFMT, BFMT, SBU>), grid, dim3(BWG_THREADS), lds, st, g);
    else hipLaunchKernelGGL((bw_gemm_kernel<AFMT, BFMT, SBU>), grid, dim3(BWG_THREADS), lds, st, g);
    return MXL_OK;
}
template <int AFMT, int BFMT>
static int launch_bw_gemm_fmt(const BwGemmArgs& g, dim3 grid, bool sbu, bool tall, hipStream_t st) {
    if (tall) return sbu ? launch_bw_gemm<AFMT, BFMT, true, true>(g, grid, st) : launch_bw_gemm<AFMT, BFMT, false, true>(g, grid, st);
    return sbu ? launch_bw_gemm<AFMT, BFMT, true, false>(g, grid, st) : launch_bw_gemm<AFMT, BFMT, false, false>(g, grid, st);
}

static std::atomic<int> bw_gemm_tile_rows{0};   // 0: by the shape; 128 or 256: forced (mxl_blockwise_gemm_tile)

// Tile height of a launch.  256 x 256 tiles run about 15 % faster per flop than 128 x 256 ones (a third fewer operand
// bytes from L2 per flop), so they win unless the coarser tiles leave that much more of the chip idle -- in the last
// round of tiles, or in the ragged last tile of every group of a grouped forward (expected padding: half a tile per
// group, which a group of 512 rows pays back).  A dense GEMM may take both: most of the output on 256-row tiles in
// whole rounds, its last rows or its last columns on 128-row tiles (a second launch), whichever split has the lowest
// cost in rounds of tiles over the chip's 256 CUs (a round of 128-row tiles = 0.5 x 1.15 rounds of 256-row tiles).
// mxl_blockwise_gemm_tile overrides.
struct BwPlan {
    bool all_low;                 // everything on 128-row tiles
    int64_t low_rows, low_cols;   // otherwise: what the 128-row tiles take, the last rows or the last columns (0, 0: nothing)
};
static BwPlan bw_plan(int64_t m, int64_t n, int mode, int num_groups) {
    BwPlan pl{false, 0, 0};
    const int64_t col_tiles = (n + BWG_BN - 1) / BWG_BN, zs = mode == 2 ? num_groups : 1, cus = 256;
    auto rounds_of = [&](int64_t tiles) { return (double)((tiles + cus - 1) / cus); };
    const int64_t rt_tall = (m + BWH_BM - 1) / BWH_BM, rt_low = (m + BWG_BM - 1) / BWG_BM;
    const int forced = bw_gemm_tile_rows.load(std::memory_order_relaxed);
    if (forced == BWG_BM) {
        pl.all_low = true;
    } else if (forced == BWH_BM) {
    } else if (mode == 0) {
        double best = rounds_of(rt_tall * col_tiles);
        for (int64_t low = 1; low < rt_tall && low <= 4 * cus; ++low) {        // `low` of the 256-row tiles cut in two
            const int64_t rows = m - (rt_tall - low) * BWH_BM;
            const double cost = rounds_of((rt_tall - low) * col_tiles) + 0.575 * rounds_of((rows + BWG_BM - 1) / BWG_BM * col_tiles);
            if (cost < best) best = cost, pl.low_rows = rows, pl.low_cols = 0;
        }
        for (int64_t low = 1; low < col_tiles && low <= 4 * cus; ++low) {      // the last `low` column tiles
            const double cost = rounds_of(rt_tall * (col_tiles - low)) + 0.575 * rounds_of(rt_low * low);
            if (cost < best) best = cost, pl.low_rows = 0, pl.low_cols = n - (col_tiles - low) * BWG_BN;
        }
        if (0.575 * rounds_of(rt_low * col_tiles) <= best) pl = BwPlan{true, 0, 0};
    } else {
        const double cost_tall = rounds_of(rt_tall * col_tiles * zs), cost_low = 0.575 * rounds_of(rt_low * col_tiles * zs);
        pl.all_low = !(cost_tall < cost_low && (mode != 1 || m >= 512 * (int64_t)num_groups));
    }
    return pl;
}

static int bw_gemm(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv, int b_fmt,
                   int b_rows_per_scale, void* c_bf16, int64_t m, int64_t n, int64_t k, int mode, const int64_t* group_lens,
                   int num_groups, void* stream) {
    if (m < 0 || n <= 0 || k < 0 || n % BW != 0 || k % BW != 0) return MXL_EINVAL;
    if (b_rows_per_scale != 1 && b_rows_per_scale != BW) return MXL_EINVAL;
    if ((a_fmt != MXL_FMT_E4M3 && a_fmt != MXL_FMT_E5M2) || (b_fmt != MXL_FMT_E4M3 && b_fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if (mode != 0 && (!group_lens || num_groups < 1 || num_groups > BW_MAX_GROUPS)) return MXL_EINVAL;
    if (m == 0) return MXL_OK;
    if (!c_bf16 || ((uintptr_t)c_bf16 & 7) != 0) return MXL_EINVAL;
    if (k > 0 && (!a_codes || !a_sinv || !b_codes || !b_sinv)) return MXL_EINVAL;
    if (k == 0 && mode != 2) return MXL_EINVAL;
    if ((((uintptr_t)a_codes | (uintptr_t)b_codes) & 15) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    BwPlan plan = bw_plan(m, n, mode, num_groups);
    if (((uintptr_t)c_bf16 & 15) != 0) plan = BwPlan{true, 0, 0};      // (the 256-row kernel's epilogue stores 16 bytes per lane)
    const bool all_low = plan.all_low;
    const int64_t low_rows = plan.low_rows, low_cols = plan.low_cols;
    const int64_t zs = mode == 2 ? num_groups : 1;
    if (256 * k >= ((int64_t)1 << 31)) return MXL_EINVAL;     // byte offsets inside a tile's operand rows are 32-bit
    hipStream_t st = (hipStream_t)stream;
    const bool sbu = b_rows_per_scale == BW;
    const int sb_shift = sbu ? 7 : 0;
    // rows [r0, r1) x columns [c0, c1) of the output (a dense GEMM: any range whose c0 is a multiple of 256; grouped:
    // everything) on tiles of `tall ? 256 : 128` rows
    auto run = [&](bool tall, int64_t r0, int64_t r1, int64_t c0, int64_t c1) {
        const int64_t bm = tall ? BWH_BM : BWG_BM, rows = r1 - r0, cols = c1 - c0;
        const int64_t row_tiles = mode == 1 ? rows / bm + num_groups : (rows + bm - 1) / bm;
        if (row_tiles > 65535 || (mode == 2 && num_groups > 65535)) return (int)MXL_EINVAL;
        BwGemmArgs g{(const uint8_t*)a_codes + r0 * k, (const float*)a_sinv + r0 * (k / BW), (const uint8_t*)b_codes + c0 * k,
                     (const float*)b_sinv + (c0 >> sb_shift) * (k / BW), (uint16_t*)c_bf16 + r0 * n + c0, rows, cols, k, n, sb_shift, mode,
                     group_lens, num_groups};
        const dim3 grid((unsigned)((cols + BWG_BN - 1) / BWG_BN), (unsigned)row_tiles, (unsigned)zs);
        if (a_fmt == MXL_FMT_E4M3 && b_fmt == MXL_FMT_E4M3) return launch_bw_gemm_fmt<MXL_FMT_E4M3, MXL_FMT_E4M3>(g, grid, sbu, tall, st);
        if (a_fmt == MXL_FMT_E5M2 && b_fmt == MXL_FMT_E4M3) return launch_bw_gemm_fmt<MXL_FMT_E5M2, MXL_FMT_E4M3>(g, grid, sbu, tall, st);
        if (a_fmt == MXL_FMT_E4M3 && b_fmt == MXL_FMT_E5M2) return launch_bw_gemm_fmt<MXL_FMT_E4M3, MXL_FMT_E5M2>(g, grid, sbu, tall, st);
        return launch_bw_gemm_fmt<MXL_FMT_E5M2, MXL_FMT_E5M2>(g, grid, sbu, tall, st);
    };
    int rc;
    if (all_low) {
        rc = run(false, 0, m, 0, n);
    } else if (low_rows > 0) {
        rc = run(true, 0, m - low_rows, 0, n);
        if (rc == MXL_OK) rc = run(false, m - low_rows, m, 0, n);
    } else if (low_cols > 0) {
        rc = run(true, 0, m, 0, n - low_cols);
        if (rc == MXL_OK) rc = run(false, 0, m, n - low_cols, n);
    } else {
        rc = run(true, 0, m, 0, n);
    }
    if (rc != MXL_OK) return rc;
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_quantize_blockwise(const void* x_bf16, int64_t rows, int64_t cols, int fmt, const int64_t* group_lens,
                                      int num_groups, void* q_row, void* sinv_row, void* q_colT, void* sinv_colT, void* stream) {
    return bw_quant(x_bf16, rows, cols, fmt, group_lens, num_groups, 1, q_row, sinv_row, q_colT, sinv_colT, false, stream);
}

extern "C" int mxl_quantize_blockwise_weight(const void* w_bf16, int64_t batch, int64_t n, int64_t k, int fmt, void* q, void* sinv,
                                             void* q_T, void* sinv_T, void* stream) {
    if (batch < 1 || batch > 65535) return MXL_EINVAL;
    return bw_quant(w_bf16, n, k, fmt, nullptr, 0, (int)batch, q, sinv, q_T, sinv_T, true, stream);
}

extern "C" int mxl_blockwise_gemm_tile(int rows) {
    if (rows != 0 && rows != BWG_BM && rows != BWH_BM) return MXL_EINVAL;
    bw_gemm_tile_rows.store(rows, std::memory_order_relaxed);
    return MXL_OK;
}

extern "C" int mxl_blockwise_gemm_plan(int64_t m, int64_t n, int mode, int num_groups, int64_t* tall_rows, int64_t* tall_cols) {
    if (m <= 0 || n <= 0 || n % BW != 0 || mode < 0 || mode > 2 || (mode != 0 && num_groups < 1) || !tall_rows || !tall_cols) return MXL_EINVAL;
    const BwPlan pl = bw_plan(m, n, mode, num_groups);
    *tall_rows = pl.all_low ? 0 : m - pl.low_rows;
    *tall_cols = pl.all_low ? 0 : n - pl.low_cols;
    return MXL_OK;
}

extern "C" int mxl_gemm_nt_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv,
                                     int b_fmt, int b_rows_per_scale, void* c_bf16, int64_t m, int64_t n, int64_t k,
                                     void* stream) {
    if (k <= 0) return MXL_EINVAL;
    return bw_gemm(a_codes, a_sinv, a_fmt, b_codes, b_sinv, b_fmt, b_rows_per_scale, c_bf16, m, n, k, 0, nullptr, 0, stream);
}

extern "C" int mxl_grouped_gemm_nt_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes,
                                             const void* b_sinv, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                             int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    if (k <= 0) return MXL_EINVAL;
    return bw_gemm(a_codes, a_sinv, a_fmt, b_codes, b_sinv, b_fmt, BW, c_bf16, total_m, n, k, 1, group_lens, num_groups, stream);
}

extern "C" int mxl_grouped_gemm_wgrad_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes,
                                                const void* b_sinv, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                                int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    if (total_m < 0 || num_groups < 1) return MXL_EINVAL;
    // a: dY^T [n, W], b: X^T [k, W], W = mxl_padded_width(total_m, num_groups); c [num_groups, n, k]
    return bw_gemm(a_codes, a_sinv, a_fmt, b_codes, b_sinv, b_fmt, 1, c_bf16, n, k, mxl_padded_width(total_m, num_groups), 2,
                   group_lens, num_groups, stream);
}
