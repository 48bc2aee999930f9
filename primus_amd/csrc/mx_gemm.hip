// Block-scaled (MX) NT GEMMs for gfx950 on the scaled FP8/FP4 MFMA
// (v_mfma_scale_f32_32x32x64_f8f6f4): dense, grouped (ragged rows per expert,
// forward and dgrad) and grouped variable-K (wgrad).  Operand conventions
// follow the reference's NT structure (primus_turbo_mxfp4_local.py:316-331,
// :432-459): both operands are quantised along the contraction dim, scales
// are E8M0 bytes per 32 elements and are applied inside the MFMA, per K step.
//
// Schedule: persistent workgroups (one per CU) walk a tile list that is
// derived on the device from group_lens, so nothing is read back to the host
// and empty experts cost nothing.  A workgroup (4 waves, 2x2) owns a 256x256
// output tile; each wave a 128x128 sub-tile = 4x4 MFMA tiles of 32x32 with
// fp32 accumulators.  K advances 128 elements (4 MX blocks) per stage through a
// double-buffered LDS ring; 16-byte chunks are XOR-swizzled so the fragment
// reads are bank-conflict free.
//
// MFMA operand layout (measured on gfx950): lane l holds row l%32; its 32
// bytes are k = 16g + [0,16) and k = 32 + 16g + [0,16) with g = l/32; the
// scale of (row r, block kb) is taken from lane r + 32*kb, byte `opsel` of the
// scale register.  An FP4 operand instead holds k = 32g + [0,32) in its first
// four registers (low nibble first).  The kernel feeds the N-side operand as MFMA source 0 so a
// lane ends up with 4 consecutive output columns (one 8-byte bf16 store).
#include <atomic>

#include "mx_device.h"

namespace mxl {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int GTHREADS = 256;
constexpr int MODE_FWD = 0;    // rows of A ragged by group; B = [G, N, K]
constexpr int MODE_WGRAD = 1;  // contraction ragged by group; C = [G, M, N]
constexpr int GROUP_M = 4;     // tile-order super-row height (L2 locality)

struct GemmArgs {
    const uint8_t* a;   // M-side codes
    const uint8_t* sa;  // M-side scales
    const uint8_t* b;   // N-side codes
    const uint8_t* sb;  // N-side scales
    uint16_t* c;        // bf16 out
    const int64_t* group_lens;  // device, may be null (one group)
    int num_groups;     // >= 1
    int64_t total_m;    // FWD: rows of a; WGRAD: tokens (sum of lens)
    int64_t m;          // WGRAD: rows of a (fixed)   | FWD: unused
    int64_t n;          // columns of c / rows of b (per group in FWD)
    int64_t k;          // FWD: contraction length; WGRAD: padded width W
};

template <int FMT> struct Op {
    static constexpr int kb = (FMT == kFmtE2M1) ? BK / 2 : BK;  // bytes per row per K stage
    static constexpr int cpr = kb / 16;                         // 16-byte chunks per row
    static constexpr int nld = 256 * cpr / GTHREADS;            // chunk loads per thread per stage
    static constexpr int rows_per_ld = GTHREADS / cpr;          // tile rows covered by one load round
};

typedef __attribute__((address_space(3))) void* lds_ptr_t;

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int64_t bytes) {
    const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, n, 0x00020000);  // raw buffer, out-of-range reads give 0
}

// One operand stage, global -> LDS without passing through registers
// (buffer_load_dwordx4 ... lds).  The hardware writes lane i of a wave to
// LDS slot base + 16*i, so the XOR swizzle is applied on the global side:
// the lane that owns physical chunk (row, pch) fetches logical chunk
// pch ^ swz(row).  `voff` is that lane's byte offset inside the tile for load
// round 0; later rounds only add a uniform row step.  In a partial last stage
// the lanes past the end of K store zeros instead (their LDS slot is their own).
template <int FMT>
__device__ __forceinline__ void stage_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds, uint32_t voff, int64_t kbyte,
                                             int64_t ld_bytes, int kbytes_left, int logical_ch, int w, int l) {
    const bool ok = 16 * logical_ch < kbytes_left;
#pragma unroll
    for (int i = 0; i < Op<FMT>::nld; ++i) {
        uint8_t* dst = lds + (i * 4 + w) * 1024;
        const uint32_t soff = (uint32_t)(kbyte + (int64_t)i * Op<FMT>::rows_per_ld * ld_bytes);
        if (ok)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 16, voff, soff, 0, 0);
        else
            *(uint4*)(dst + 16 * l) = make_uint4(0, 0, 0, 0);
    }
}

// Scale dword (4 blocks of this K stage) of one row; blocks past the end read as 2^0.
__device__ __forceinline__ uint32_t load_scale4(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_off, int64_t blk0,
                                                int64_t blk_end, bool aligned) {
    uint32_t v;
    if (aligned && blk0 + 4 <= blk_end) {
        v = __builtin_amdgcn_raw_buffer_load_b32(rsrc, row_off, (uint32_t)blk0, 0);
    } else {
        v = 0x7F7F7F7Fu;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (blk0 + j < blk_end) {
                const uint32_t b = __builtin_amdgcn_raw_buffer_load_b8(rsrc, row_off, (uint32_t)(blk0 + j), 0);
                v = (v & ~(0xFFu << (8 * j))) | (b << (8 * j));
            }
    }
    return v;
}

// LDS -> MFMA fragment of one 32-row tile for K step ks (64 elements).
template <int FMT>
__device__ __forceinline__ v8i read_frag(const uint8_t* lds, int row, int ks, int g) {
    v8i f;
    if (FMT == kFmtE4M3) {
        const int s = swz(row);
        const uint4 lo = *(const uint4*)(lds + row * 128 + 16 * ((4 * ks + g) ^ s));
        const uint4 hi = *(const uint4*)(lds + row * 128 + 16 * ((4 * ks + 2 + g) ^ s));
        f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
        f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
    } else {
        // FP4 operands are laid out differently (measured): the lane's 32 nibbles are the
        // 32 consecutive k = 32g + [0,32) of the K step, i.e. one 16-byte chunk of the 64-byte row.
        const int s = swz(row) & 3;
        const uint4 v = *(const uint4*)(lds + row * 64 + 16 * ((2 * ks + g) ^ s));
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
        f[4] = 0; f[5] = 0; f[6] = 0; f[7] = 0;
    }
    return f;
}

template <int AFMT, int BFMT, int MODE>
__global__ __launch_bounds__(GTHREADS) void mx_gemm_kernel(GemmArgs p) {
    constexpr int A_BYTES = 256 * Op<AFMT>::kb, B_BYTES = 256 * Op<BFMT>::kb;
    constexpr int STAGE = A_BYTES + B_BYTES + 2 * 256 * 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int* pre_tiles = (int*)(smem + 2 * STAGE);                       // [G+1] prefix of row tiles (FWD)
    int64_t* pre_rows = (int64_t*)(pre_tiles + MXL_MAX_GROUPS + 2);  // [G+1] prefix of rows / padded cols

    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5;
    const int wm = w >> 1, wn = w & 1;
    const int G = p.num_groups;

    // ---- per-workgroup group tables (device-side, no host sync) ----
    if (t == 0) {
        int tiles = 0;
        int64_t rows = 0;
        pre_tiles[0] = 0;
        pre_rows[0] = 0;
        for (int i = 0; i < G; ++i) {
            const int64_t len = p.group_lens ? p.group_lens[i] : p.total_m;
            if (MODE == MODE_FWD) {
                tiles += (int)((len + BM - 1) / BM);
                rows += len;
            } else {
                rows += (len + MXL_SEG_ALIGN - 1) / MXL_SEG_ALIGN * MXL_SEG_ALIGN;
            }
            pre_tiles[i + 1] = tiles;
            pre_rows[i + 1] = rows;
        }
    }
    __syncthreads();

    const int tiles_n = (int)((p.n + BN - 1) / BN);
    int tiles_m, total_tiles;
    if (MODE == MODE_FWD) {
        tiles_m = pre_tiles[G];
        total_tiles = tiles_m * tiles_n;
    } else {
        tiles_m = (int)((p.m + BM - 1) / BM);
        total_tiles = G * tiles_m * tiles_n;
    }

    // XCD-aware start: consecutive workgroup ids land on different XCDs, so give
    // each XCD a contiguous run of the tile order.
    const int nwg = gridDim.x;
    const int per_xcd = nwg >> 3;
    const int vwg = (nwg & 7) ? (int)blockIdx.x : ((int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3));

    const int64_t lda = (AFMT == kFmtE2M1) ? p.k / 2 : p.k;
    const int64_t ldb = (BFMT == kFmtE2M1) ? p.k / 2 : p.k;
    const int64_t ld_s = p.k / 32;  // scale row pitch (both operands)
    const bool s_aligned = ((((uintptr_t)p.sa | (uintptr_t)p.sb | (uintptr_t)ld_s) & 3) == 0);
    const int64_t a_rows_total = (MODE == MODE_FWD) ? p.total_m : p.m;
    const int64_t b_rows_total = (MODE == MODE_FWD) ? (int64_t)G * p.n : p.n;

    // per-thread constants of the global -> LDS mapping (see stage_to_lds)
    const int a_row = t / Op<AFMT>::cpr, a_pch = t % Op<AFMT>::cpr;
    const int a_lch = (AFMT == kFmtE2M1) ? (a_pch ^ (swz(a_row) & 3)) : (a_pch ^ swz(a_row));
    const uint32_t a_voff = (uint32_t)(a_row * (int)lda + 16 * a_lch);
    const int b_row = t / Op<BFMT>::cpr, b_pch = t % Op<BFMT>::cpr;
    const int b_lch = (BFMT == kFmtE2M1) ? (b_pch ^ (swz(b_row) & 3)) : (b_pch ^ swz(b_row));
    const uint32_t b_voff = (uint32_t)(b_row * (int)ldb + 16 * b_lch);
    const uint32_t s_voff = (uint32_t)(t * (int)ld_s);

    for (int tile = vwg; tile < total_tiles; tile += nwg) {
        // ---- decode tile -> (group, pid_m, pid_n) ----
        int grp = 0, pid_m, pid_n;
        int tl = tile;
        if (MODE == MODE_WGRAD) {
            grp = tl / (tiles_m * tiles_n);
            tl -= grp * tiles_m * tiles_n;
        }
        {
            const int width = GROUP_M * tiles_n;
            const int gid = tl / width;
            const int first = gid * GROUP_M;
            const int gsz = (tiles_m - first) < GROUP_M ? (tiles_m - first) : GROUP_M;
            pid_m = first + (tl % width) % gsz;
            pid_n = (tl % width) / gsz;
        }
        int64_t a_row0, b_row0, c_row0;
        int m_valid;
        int64_t k0, k1;  // contraction range in elements
        if (MODE == MODE_FWD) {
            // binary search: largest grp with pre_tiles[grp] <= pid_m
            int lo = 0, hi = G;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (pre_tiles[mid] <= pid_m) lo = mid; else hi = mid;
            }
            grp = lo;
            const int64_t g_row0 = pre_rows[grp], g_rows = pre_rows[grp + 1] - g_row0;
            const int64_t r = (int64_t)(pid_m - pre_tiles[grp]) * BM;
            a_row0 = g_row0 + r;
            m_valid = (g_rows - r) < BM ? (int)(g_rows - r) : BM;
            b_row0 = (int64_t)grp * p.n + (int64_t)pid_n * BN;
            c_row0 = a_row0;
            k0 = 0;
            k1 = p.k;
        } else {
            a_row0 = (int64_t)pid_m * BM;
            m_valid = (p.m - a_row0) < BM ? (int)(p.m - a_row0) : BM;
            b_row0 = (int64_t)pid_n * BN;
            c_row0 = (int64_t)grp * p.m + a_row0;
            k0 = pre_rows[grp];
            k1 = pre_rows[grp + 1];
        }
        const int64_t n0 = (int64_t)pid_n * BN;
        const int n_valid = (p.n - n0) < BN ? (int)(p.n - n0) : BN;
        const int kt_count = (int)((k1 - k0 + BK - 1) / BK);

        // Buffer descriptors anchored at the tile's first row: rows past the end
        // of the operand read as zero, rows of a neighbouring group are read but
        // never stored.
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a + a_row0 * lda, (a_rows_total - a_row0) * lda);
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + b_row0 * ldb, (b_rows_total - b_row0) * ldb);
        const __amdgpu_buffer_rsrc_t rsa = make_rsrc(p.sa + a_row0 * ld_s, (a_rows_total - a_row0) * ld_s);
        const __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.sb + b_row0 * ld_s, (b_rows_total - b_row0) * ld_s);

        v16f acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        uint32_t vsa = 0, vsb = 0;
        auto issue = [&](int kt, int stage) {
            const int64_t ke = k0 + (int64_t)kt * BK;
            const int left = (int)((k1 - ke) < BK ? (k1 - ke) : BK);
            uint8_t* s = smem + stage * STAGE;
            stage_to_lds<AFMT>(ra, s, a_voff, (AFMT == kFmtE2M1) ? ke / 2 : ke, lda, (AFMT == kFmtE2M1) ? left / 2 : left,
                               a_lch, w, l);
            stage_to_lds<BFMT>(rb, s + A_BYTES, b_voff, (BFMT == kFmtE2M1) ? ke / 2 : ke, ldb,
                               (BFMT == kFmtE2M1) ? left / 2 : left, b_lch, w, l);
            vsa = load_scale4(rsa, s_voff, ke / 32, k1 / 32, s_aligned);
            vsb = load_scale4(rsb, s_voff, ke / 32, k1 / 32, s_aligned);
        };
        auto put_scales = [&](int stage) {
            uint32_t* s = (uint32_t*)(smem + stage * STAGE + A_BYTES + B_BYTES);
            s[t] = vsa;
            s[256 + t] = vsb;
        };

        if (kt_count > 0) {
            issue(0, 0);
            put_scales(0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

        for (int kt = 0; kt < kt_count; ++kt) {
            const bool more = kt + 1 < kt_count;
            if (more) issue(kt + 1, (kt + 1) & 1);
            const uint8_t* s = smem + (kt & 1) * STAGE;
            const uint8_t* sA = s;
            const uint8_t* sB = s + A_BYTES;
            const uint32_t* sSA = (const uint32_t*)(s + A_BYTES + B_BYTES);
            const uint32_t* sSB = sSA + 256;
            int sca[4], scb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sca[i] = (int)(sSA[wm * 128 + i * 32 + lr] >> (8 * g));
                scb[i] = (int)(sSB[wn * 128 + i * 32 + lr] >> (8 * g));
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                v8i fa[4], fb[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    fa[i] = read_frag<AFMT>(sA, wm * 128 + i * 32 + lr, ks, g);
                    fb[i] = read_frag<BFMT>(sB, wn * 128 + i * 32 + lr, ks, g);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        // source 0 = N side (format cbsz), source 1 = M side (format blgp)
                        if (ks == 0)
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                fb[j], fa[i], acc[i][j], BFMT == kFmtE2M1 ? 4 : 0, AFMT == kFmtE2M1 ? 4 : 0, 0, scb[j], 0,
                                sca[i]);
                        else
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                fb[j], fa[i], acc[i][j], BFMT == kFmtE2M1 ? 4 : 0, AFMT == kFmtE2M1 ? 4 : 0, 2, scb[j], 2,
                                sca[i]);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the MFMAs above the wait: loads overlap with them
            if (more) put_scales((kt + 1) & 1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }

        // ---- epilogue: fp32 -> bf16, 4 consecutive columns per lane ----
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int mrow = wm * 128 + i * 32 + lr;
            if (mrow < m_valid) {
                uint16_t* crow = p.c + (c_row0 + mrow) * p.n + n0;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int ncol = wn * 128 + j * 32 + 8 * q + 4 * g;
                        if (ncol < n_valid) {
                            v4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1],
                                      (__bf16)acc[i][j][4 * q + 2], (__bf16)acc[i][j][4 * q + 3]};
                            *(v4bf*)(crow + ncol) = o;
                        }
                    }
            }
        }
    }
}

constexpr int gemm_lds_bytes(int afmt, int bfmt) {
    return 2 * (256 * (afmt == kFmtE2M1 ? 64 : 128) + 256 * (bfmt == kFmtE2M1 ? 64 : 128) + 2048) +
           (MXL_MAX_GROUPS + 2) * 4 + (MXL_MAX_GROUPS + 2) * 8;
}

static int num_cus() {
    static std::atomic<int> cached{0};
    int v = cached.load(std::memory_order_relaxed);
    if (v) return v;
    int dev = 0;
    hipDeviceProp_t pr;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&pr, dev) != hipSuccess) return 256;
    cached.store(pr.multiProcessorCount, std::memory_order_relaxed);
    return pr.multiProcessorCount;
}

template <int AFMT, int BFMT, int MODE>
static int launch_gemm(const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    constexpr int lds = gemm_lds_bytes(AFMT, BFMT);
    static std::atomic<bool> attr_set{false};
    auto kern = mx_gemm_kernel<AFMT, BFMT, MODE>;
    if (!attr_set.load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return MXL_ELAUNCH;
        attr_set.store(true, std::memory_order_release);
    }
    int64_t grid = num_cus();
    if (max_tiles < grid) grid = max_tiles;
    if (grid <= 0) return MXL_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(GTHREADS), lds, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

template <int MODE>
static int dispatch_gemm(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE>(a, max_tiles, st);
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E2M1, MODE>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E4M3, MODE>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E2M1, MODE>(a, max_tiles, st);
    return MXL_EINVAL;
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_grouped_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                   const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                   int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    if (!a_codes || !a_scales || !b_codes || !b_scales || !c_bf16) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % MXL_BLOCK != 0 || k % MXL_BLOCK != 0) return MXL_EINVAL;
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS) return MXL_EINVAL;
    if (num_groups > 1 && !group_lens) return MXL_EINVAL;
    if (total_m == 0) return MXL_OK;
    GemmArgs a;
    a.a = (const uint8_t*)a_codes;
    a.sa = (const uint8_t*)a_scales;
    a.b = (const uint8_t*)b_codes;
    a.sb = (const uint8_t*)b_scales;
    a.c = (uint16_t*)c_bf16;
    a.group_lens = group_lens;
    a.num_groups = num_groups;
    a.total_m = total_m;
    a.m = 0;
    a.n = n;
    a.k = k;
    const int64_t max_tiles = (total_m / BM + num_groups) * ((n + BN - 1) / BN);
    return dispatch_gemm<MODE_FWD>(a_fmt, b_fmt, a, max_tiles, (hipStream_t)stream);
}

extern "C" int mxl_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                           const void* b_scales, int b_fmt, void* c_bf16, int64_t m, int64_t n, int64_t k,
                           void* stream) {
    return mxl_grouped_gemm_nt(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, nullptr, 1, m, n, k,
                               stream);
}

extern "C" int mxl_grouped_gemm_wgrad(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                      const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                      int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    if (!a_codes || !a_scales || !b_codes || !b_scales || !c_bf16) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % MXL_BLOCK != 0 || k % MXL_BLOCK != 0) return MXL_EINVAL;
    if (num_groups < 0 || num_groups > MXL_MAX_GROUPS) return MXL_EINVAL;
    if ((num_groups > 0) != (group_lens != nullptr)) return MXL_EINVAL;
    const int G = num_groups > 0 ? num_groups : 1;
    GemmArgs a;
    a.a = (const uint8_t*)a_codes;
    a.sa = (const uint8_t*)a_scales;
    a.b = (const uint8_t*)b_codes;
    a.sb = (const uint8_t*)b_scales;
    a.c = (uint16_t*)c_bf16;
    a.group_lens = group_lens;
    a.num_groups = G;
    a.total_m = total_m;
    a.m = n;  // rows of the output per group
    a.n = k;  // columns of the output
    a.k = mxl_padded_width(total_m, G);
    if (a.k == 0) a.k = MXL_SEG_ALIGN;  // keeps pitches non-zero; no tile reads it
    const int64_t max_tiles = (int64_t)G * ((n + BM - 1) / BM) * ((k + BN - 1) / BN);
    return dispatch_gemm<MODE_WGRAD>(a_fmt, b_fmt, a, max_tiles, (hipStream_t)stream);
}

extern "C" int mxl_version(void) { return 1; }

extern "C" const char* mxl_error_string(int code) {
    switch (code) {
        case MXL_OK: return "ok";
        case MXL_EINVAL: return "invalid argument (shape, alignment, enum or null pointer)";
        case MXL_ELAUNCH: return "HIP launch error";
        case MXL_ENODEV: return "device is not gfx950";
        default: return "unknown error";
    }
}
