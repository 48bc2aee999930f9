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
// the MFMA's E8M0 scale inputs, so this GEMM keeps two accumulator sets: the MFMAs of one K block of 128 add up in
// the first (from zero), which is then multiplied into the second with the block's factors.  That takes registers
// the 256 x 256 kernels do not have: the tile is 128 x 128, 64 x 64 per wave.  Operands go through LDS with plain
// loads and stores, register-prefetched one K block ahead.
#include "mx_device.h"

namespace mxl {

constexpr int BW = 128;            // block edge
constexpr int BW_THREADS = 256;

typedef float bv16f __attribute__((ext_vector_type(16)));
typedef int bv8i __attribute__((ext_vector_type(8)));
typedef __bf16 bv4bf __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------------------------------------
// Quantiser.  One workgroup per 128 x 128 tile of x[rows, cols] (cols % 128 == 0; rows ragged).  The tile sits in
// LDS as bf16 with a pitch of 130 elements; thread t owns half a row (row t / 2, 64 columns) for the row-wise copy and
// half a column (column t / 2, 64 rows) for the transposed one.
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
};

constexpr int BW_PITCH = 130;

template <int FMT> __device__ __forceinline__ float bw_fp8_max() { return FMT == kFmtE5M2 ? 57344.f : 448.f; }

template <int FMT, bool TWOD>
__global__ __launch_bounds__(BW_THREADS) void bw_quant_kernel(BwQuantArgs a) {
    __shared__ uint16_t tile[BW * BW_PITCH];
    __shared__ uint32_t amax_r[BW], amax_c[BW];
    __shared__ uint32_t amax_tile;
    const int t = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.y * BW, col0 = (int64_t)blockIdx.x * BW;
    const int64_t rows_pad = (a.rows + BW - 1) / BW * BW;
    const int64_t kb_cols = a.cols / BW, kb_rows = rows_pad / BW;
    // load: 2048 pieces of 8 elements, 8 per thread; rows past the end read as zero
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int pc = i * BW_THREADS + t, r = pc >> 4, c8 = (pc & 15) * 8;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row0 + r < a.rows) v = *(const uint4*)(a.x + (row0 + r) * a.cols + col0 + c8);
        uint32_t* d = (uint32_t*)(tile + r * BW_PITCH + c8);   // pitch 130 elements: 4-byte aligned
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
    if (t == 0) amax_tile = 0u;
    __syncthreads();
    const int own = t >> 1, half = t & 1;
    // largest magnitude (15-bit bf16 pattern) of the half row and of the half column this thread owns
    uint32_t mr = 0u, mc = 0u;
    {
        const uint32_t* p = (const uint32_t*)(tile + own * BW_PITCH + half * 64);
#pragma unroll 8
        for (int i = 0; i < 32; ++i) mr = pk_absmax(mr, p[i]);
        mr = hmax16(mr);
        const uint16_t* q = tile + (half * 64) * BW_PITCH + own;
#pragma unroll 8
        for (int i = 0; i < 64; ++i) {
            const uint32_t v = q[i * BW_PITCH] & 0x7FFFu;
            mc = v > mc ? v : mc;
        }
    }
    {
        const uint32_t orr = __shfl_xor(mr, 1), occ = __shfl_xor(mc, 1);
        mr = orr > mr ? orr : mr;
        mc = occ > mc ? occ : mc;
    }
    if (half == 0) {
        amax_r[own] = mr;
        amax_c[own] = mc;
        if (TWOD) atomicMax(&amax_tile, mr);
    }
    __syncthreads();
    const float fmax = bw_fp8_max<FMT>();
    auto scale_of = [&](uint32_t amax16) { return fmax / fmaxf(__uint_as_float(amax16 << 16), 1e-12f); };
    // ---- row-wise copy: half a row, 64 codes = four 16-byte stores ----
    if (a.q_row != nullptr) {
        const uint32_t am = TWOD ? amax_tile : amax_r[own];
        const float sc = scale_of(am);
        const bool bad = am >= 0x7F80u;
        const int64_t r = row0 + own;
        if (r < a.rows) {
            const uint32_t* p = (const uint32_t*)(tile + own * BW_PITCH + half * 64);
            uint8_t* dst = a.q_row + r * a.cols + col0 + half * 64;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint4 o;
                o.x = bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(p[8 * i + 0], p[8 * i + 1], sc);
                o.y = bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(p[8 * i + 2], p[8 * i + 3], sc);
                o.z = bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(p[8 * i + 4], p[8 * i + 5], sc);
                o.w = bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(p[8 * i + 6], p[8 * i + 7], sc);
                *(uint4*)(dst + 16 * i) = o;
            }
            if (!TWOD && half == 0) a.sinv_row[r * kb_cols + blockIdx.x] = 1.0f / sc;
        }
        if (TWOD && t == 0) a.sinv_row[(int64_t)blockIdx.y * kb_cols + blockIdx.x] = 1.0f / sc;
    }
    // ---- transposed copy: half a column, 64 codes of row (col0 + own) of the output; rows past the end give zero codes ----
    if (a.q_colT != nullptr) {
        const uint32_t am = TWOD ? amax_tile : amax_c[own];
        const float sc = scale_of(am);
        const bool bad = am >= 0x7F80u;
        const uint16_t* q = tile + (half * 64) * BW_PITCH + own;
        uint8_t* dst = a.q_colT + (col0 + own) * rows_pad + row0 + half * 64;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = 16 * i + 4 * j;
                const uint32_t p0 = (uint32_t)q[(e + 0) * BW_PITCH] | ((uint32_t)q[(e + 1) * BW_PITCH] << 16);
                const uint32_t p1 = (uint32_t)q[(e + 2) * BW_PITCH] | ((uint32_t)q[(e + 3) * BW_PITCH] << 16);
                w[j] = bad ? 0x7F7F7F7Fu : cvt4_fp8<FMT>(p0, p1, sc);
            }
            *(uint4*)(dst + 16 * i) = make_uint4(w[0], w[1], w[2], w[3]);
        }
        if (!TWOD && half == 0) a.sinv_colT[(col0 + own) * kb_rows + blockIdx.y] = 1.0f / sc;
        if (TWOD && t == 0) a.sinv_colT[(int64_t)blockIdx.x * kb_rows + blockIdx.y] = 1.0f / sc;
    }
}

// ------------------------------------------------------------------------------------------------------------
// GEMM.  c[m, n] (bf16) = sum_kb sa[m, kb] * sb[n >> sb_shift, kb] * (a[m, kb-th 128] . b[n, kb-th 128]),
// a[m_rows, k], b[n, k] FP8 codes, k % 128 == 0, n % 128 == 0; sb_shift = 0 (a factor per row of b) or 7 (per
// 128 rows: weights).  Workgroup = 128 x 128 output tile, wave (wm, wn) = 64 x 64 = 2 x 2 MFMA tiles of 32 x 32.
// LDS: two stages of both operands' 128 x 128 bytes, 16-byte pieces XOR-swizzled by the row, and the factors.
// ------------------------------------------------------------------------------------------------------------
struct BwGemmArgs {
    const uint8_t* a;
    const float* sa;
    const uint8_t* b;
    const float* sb;
    uint16_t* c;
    int64_t m, n, k;
    int sb_shift;
};

constexpr int BW_GEMM_LDS = 2 * 2 * BW * BW + 2 * 2 * BW * 4;

template <int AFMT, int BFMT>
__global__ __launch_bounds__(BW_THREADS, 2) void bw_gemm_kernel(BwGemmArgs p) {
    constexpr int CB = BFMT == kFmtE5M2 ? 1 : 0, BL = AFMT == kFmtE5M2 ? 1 : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t bw_smem[];
    uint8_t (*ops)[2][BW * BW] = (uint8_t (*)[2][BW * BW])bw_smem;                     // [stage][operand][row * 128 + swizzled piece]
    float (*fac)[2][BW] = (float (*)[2][BW])(bw_smem + 2 * 2 * BW * BW);               // [stage][operand][row]
    const int t = threadIdx.x;
    const int w = t >> 6, l = t & 63, lr = l & 31, g = l >> 5, wm = w >> 1, wn = w & 1;
    const int64_t row0 = (int64_t)blockIdx.y * BW, col0 = (int64_t)blockIdx.x * BW;
    const int64_t kb_n = p.k / BW;   // (the argument block itself is only read here and in the copies below)
    // loader geometry: piece pc = i * 256 + t of an operand's 1024 pieces: row pc / 8 = 32 i + t / 8, piece t % 8.
    // Everything the loop needs from the argument block is copied to locals first (and the loader is written as
    // macros over scalars): a lambda that captures the block or an array by reference puts it on the stack.
    const uint8_t* const pa = p.a;
    const uint8_t* const pb = p.b;
    const float* const psa = p.sa;
    const float* const psb = p.sb;
    const int64_t pm = p.m, pk = p.k, pn = p.n;
    uint16_t* const pc_out = p.c;
    const int sb_shift = p.sb_shift;
    const int lrow = t >> 3, lpc = t & 7;
    const int lds_off = lrow * BW + 16 * (lpc ^ (lrow & 7));      // rows 32 i + lrow share (row & 7)
    const uint8_t* ga = pa + (row0 + lrow) * pk + lpc * 16;
    const uint8_t* gb = pb + (col0 + lrow) * pk + lpc * 16;
    const bool av0 = row0 + lrow < pm, av1 = row0 + 32 + lrow < pm, av2 = row0 + 64 + lrow < pm, av3 = row0 + 96 + lrow < pm;
    const float* gsa = psa + (row0 + (t & (BW - 1))) * kb_n;
    const float* gsb = psb + ((col0 + (t & (BW - 1))) >> sb_shift) * kb_n;
    const bool fav = t < BW && row0 + t < pm;
    const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
    uint4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
    float fr = 0.f;
#define MXL_BW_FETCH(KB)                                                                      \
    do {                                                                                      \
        const int64_t o_ = (int64_t)(KB) * BW;                                                \
        ra0 = av0 ? *(const uint4*)(ga + o_) : z4;                                            \
        ra1 = av1 ? *(const uint4*)(ga + 32 * pk + o_) : z4;                                  \
        ra2 = av2 ? *(const uint4*)(ga + 64 * pk + o_) : z4;                                  \
        ra3 = av3 ? *(const uint4*)(ga + 96 * pk + o_) : z4;                                  \
        rb0 = *(const uint4*)(gb + o_);                                                       \
        rb1 = *(const uint4*)(gb + 32 * pk + o_);                                             \
        rb2 = *(const uint4*)(gb + 64 * pk + o_);                                             \
        rb3 = *(const uint4*)(gb + 96 * pk + o_);                                             \
        fr = t < BW ? (fav ? gsa[KB] : 0.f) : gsb[KB];                                        \
    } while (0)
#define MXL_BW_STASH(ST)                                                                      \
    do {                                                                                      \
        uint8_t* oa_ = &ops[ST][0][lds_off];                                                  \
        uint8_t* ob_ = &ops[ST][1][lds_off];                                                  \
        *(uint4*)(oa_) = ra0; *(uint4*)(oa_ + 32 * BW) = ra1;                                 \
        *(uint4*)(oa_ + 64 * BW) = ra2; *(uint4*)(oa_ + 96 * BW) = ra3;                       \
        *(uint4*)(ob_) = rb0; *(uint4*)(ob_ + 32 * BW) = rb1;                                 \
        *(uint4*)(ob_ + 64 * BW) = rb2; *(uint4*)(ob_ + 96 * BW) = rb3;                       \
        fac[ST][t >> 7][t & (BW - 1)] = fr;                                                   \
    } while (0)
    bv16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    MXL_BW_FETCH(0);
    MXL_BW_STASH(0);
    __syncthreads();
    for (int64_t kb = 0; kb < kb_n; ++kb) {
        const int st = (int)(kb & 1);
        if (kb + 1 < kb_n) MXL_BW_FETCH(kb + 1);
        bv16f part[2][2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bv8i fa8[2], fb8[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                // lane (lr, g) of a 32-row fragment holds bytes 16 g .. 16 g + 15 and 32 + 16 g .. of the K step
                const int ra_ = wm * 64 + i * 32 + lr, rb_ = wn * 64 + i * 32 + lr;
                const uint4 alo = *(const uint4*)(&ops[st][0][ra_ * BW + 16 * ((4 * ks + g) ^ (ra_ & 7))]);
                const uint4 ahi = *(const uint4*)(&ops[st][0][ra_ * BW + 16 * ((4 * ks + 2 + g) ^ (ra_ & 7))]);
                const uint4 blo = *(const uint4*)(&ops[st][1][rb_ * BW + 16 * ((4 * ks + g) ^ (rb_ & 7))]);
                const uint4 bhi = *(const uint4*)(&ops[st][1][rb_ * BW + 16 * ((4 * ks + 2 + g) ^ (rb_ & 7))]);
                fa8[i] = bv8i{(int)alo.x, (int)alo.y, (int)alo.z, (int)alo.w, (int)ahi.x, (int)ahi.y, (int)ahi.z, (int)ahi.w};
                fb8[i] = bv8i{(int)blo.x, (int)blo.y, (int)blo.z, (int)blo.w, (int)bhi.x, (int)bhi.y, (int)bhi.z, (int)bhi.w};
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    bv16f zero;
#pragma unroll
                    for (int e = 0; e < 16; ++e) zero[e] = 0.f;
                    // the b fragment is the first operand: a lane ends up with 4 consecutive output columns
                    part[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[j], fa8[i], ks == 0 ? zero : part[i][j], CB, BL, 0,
                                                                               127, 0, 127);
                }
        }
        // acc += part * (sa[row] * sb[col]): lane (lr, g), register e = 4 q + r of tile (i, j) is row i * 32 + lr,
        // column j * 32 + 8 q + 4 g + r of the wave's 64 x 64
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float sa = fac[st][0][wm * 64 + i * 32 + lr];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 sb = *(const float4*)(&fac[st][1][wn * 64 + j * 32 + 8 * q + 4 * g]);
                    acc[i][j][4 * q + 0] = fmaf(part[i][j][4 * q + 0], sa * sb.x, acc[i][j][4 * q + 0]);
                    acc[i][j][4 * q + 1] = fmaf(part[i][j][4 * q + 1], sa * sb.y, acc[i][j][4 * q + 1]);
                    acc[i][j][4 * q + 2] = fmaf(part[i][j][4 * q + 2], sa * sb.z, acc[i][j][4 * q + 2]);
                    acc[i][j][4 * q + 3] = fmaf(part[i][j][4 * q + 3], sa * sb.w, acc[i][j][4 * q + 3]);
                }
        }
        if (kb + 1 < kb_n) MXL_BW_STASH(st ^ 1);   // the other stage was last read before the previous iteration's barrier
        __syncthreads();
    }
#undef MXL_BW_FETCH
#undef MXL_BW_STASH
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t m = row0 + wm * 64 + i * 32 + lr;
        if (m >= pm) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bv4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                 (__bf16)acc[i][j][4 * q + 3]};
                *(bv4bf*)(pc_out + m * pn + col0 + wn * 64 + j * 32 + 8 * q + 4 * g) = o;
            }
    }
}

template <bool TWOD>
static int launch_bw_quant(const BwQuantArgs& a, int fmt, hipStream_t st) {
    const dim3 grid((unsigned)(a.cols / BW), (unsigned)((a.rows + BW - 1) / BW));
    if (fmt == MXL_FMT_E4M3) hipLaunchKernelGGL((bw_quant_kernel<MXL_FMT_E4M3, TWOD>), grid, dim3(BW_THREADS), 0, st, a);
    else hipLaunchKernelGGL((bw_quant_kernel<MXL_FMT_E5M2, TWOD>), grid, dim3(BW_THREADS), 0, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

static int bw_quant(const void* x, int64_t rows, int64_t cols, int fmt, void* q_row, void* sinv_row, void* q_colT,
                    void* sinv_colT, bool twod, void* stream) {
    if (rows < 0 || cols <= 0 || cols % BW != 0 || (fmt != MXL_FMT_E4M3 && fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if ((q_row == nullptr) != (sinv_row == nullptr) || (q_colT == nullptr) != (sinv_colT == nullptr)) return MXL_EINVAL;
    if (!q_row && !q_colT) return MXL_EINVAL;
    if (twod && rows % BW != 0) return MXL_EINVAL;
    if (rows == 0) return MXL_OK;
    if (!x || ((uintptr_t)x & 15) != 0 || (rows + BW - 1) / BW > 65535) return MXL_EINVAL;
    if ((((uintptr_t)q_row | (uintptr_t)q_colT) & 15) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    BwQuantArgs a{(const uint16_t*)x, rows, cols, (uint8_t*)q_row, (float*)sinv_row, (uint8_t*)q_colT, (float*)sinv_colT};
    return twod ? launch_bw_quant<true>(a, fmt, (hipStream_t)stream) : launch_bw_quant<false>(a, fmt, (hipStream_t)stream);
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_quantize_blockwise(const void* x_bf16, int64_t rows, int64_t cols, int fmt, void* q_row, void* sinv_row,
                                      void* q_colT, void* sinv_colT, void* stream) {
    return bw_quant(x_bf16, rows, cols, fmt, q_row, sinv_row, q_colT, sinv_colT, false, stream);
}

extern "C" int mxl_quantize_blockwise_weight(const void* w_bf16, int64_t n, int64_t k, int fmt, void* q, void* sinv, void* q_T,
                                             void* sinv_T, void* stream) {
    return bw_quant(w_bf16, n, k, fmt, q, sinv, q_T, sinv_T, true, stream);
}

extern "C" int mxl_gemm_nt_blockwise(const void* a_codes, const void* a_sinv, int a_fmt, const void* b_codes, const void* b_sinv,
                                     int b_fmt, int b_rows_per_scale, void* c_bf16, int64_t m, int64_t n, int64_t k,
                                     void* stream) {
    if (m < 0 || n <= 0 || k <= 0 || n % BW != 0 || k % BW != 0) return MXL_EINVAL;
    if (b_rows_per_scale != 1 && b_rows_per_scale != BW) return MXL_EINVAL;
    if ((a_fmt != MXL_FMT_E4M3 && a_fmt != MXL_FMT_E5M2) || (b_fmt != MXL_FMT_E4M3 && b_fmt != MXL_FMT_E5M2)) return MXL_EINVAL;
    if (m == 0) return MXL_OK;
    if (!a_codes || !a_sinv || !b_codes || !b_sinv || !c_bf16 || (m + BW - 1) / BW > 65535) return MXL_EINVAL;
    if ((((uintptr_t)a_codes | (uintptr_t)b_codes) & 15) != 0 || ((uintptr_t)c_bf16 & 7) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    BwGemmArgs g{(const uint8_t*)a_codes, (const float*)a_sinv, (const uint8_t*)b_codes, (const float*)b_sinv, (uint16_t*)c_bf16,
                 m, n, k, b_rows_per_scale == 1 ? 0 : 7};
    const dim3 grid((unsigned)(n / BW), (unsigned)((m + BW - 1) / BW));
    hipStream_t st = (hipStream_t)stream;
    // the dynamic LDS size is above the default limit: the attribute is set at every launch (a host-side table write)
#define MXL_BW_GEMM(A, B)                                                                                                \
    do {                                                                                                                 \
        if (hipFuncSetAttribute((const void*)bw_gemm_kernel<A, B>, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                                BW_GEMM_LDS) != hipSuccess)                                                              \
            return MXL_ELAUNCH;                                                                                          \
        hipLaunchKernelGGL((bw_gemm_kernel<A, B>), grid, dim3(BW_THREADS), BW_GEMM_LDS, st, g);                          \
    } while (0)
    if (a_fmt == MXL_FMT_E4M3 && b_fmt == MXL_FMT_E4M3) MXL_BW_GEMM(MXL_FMT_E4M3, MXL_FMT_E4M3);
    else if (a_fmt == MXL_FMT_E5M2 && b_fmt == MXL_FMT_E4M3) MXL_BW_GEMM(MXL_FMT_E5M2, MXL_FMT_E4M3);
    else if (a_fmt == MXL_FMT_E4M3 && b_fmt == MXL_FMT_E5M2) MXL_BW_GEMM(MXL_FMT_E4M3, MXL_FMT_E5M2);
    else MXL_BW_GEMM(MXL_FMT_E5M2, MXL_FMT_E5M2);
#undef MXL_BW_GEMM
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}
