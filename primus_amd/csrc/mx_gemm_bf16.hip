// Grouped GEMM on unquantised bf16 operands for gfx950 (v_mfma_f32_32x32x16_bf16): what the reference's grouped
// linear runs when no low-precision recipe is active -- the first / last layers of an FP4 run fall back to it --
// (primus/backends/megatron/core/extensions/primus_turbo.py:2210-2216, primus/backends/megatron/core/fp4_utils.py:155-165),
// with tokens-per-expert consumed on the device like the quantised kernels do: no host read, capturable in a graph.
//
//   forward / dgrad :  c[rows of group g, n] = a[rows of group g, k] . b_g^T        b_g = [n, k]   (contraction contiguous)
//                                                                   or . b_g          b_g = [k, n]   (MXL_BF_B_KN)
//   wgrad           :  c[g][m_out, n_out] = sum over the tokens t of group g of p[t, m_out] * q[t, n_out]
//
// One workgroup (4 waves, 2 x 2) per 128 x 256 output tile, a wave owns 64 x 128 = 2 x 4 MFMA tiles of 32 x 32 with
// fp32 accumulators.  K advances in slots of 32 elements (64 bytes per row) through a 2-stage LDS buffer filled by
// LDS-direct loads (buffer_load ... lds) one slot ahead.  An operand whose contraction dim is contiguous in memory is
// staged [rows][32] and read with ds_read_b128; one whose contraction dim is the slow one (the [k, n] weight, both
// operands of wgrad) is staged as it lies, [32][columns], and read with the transposing LDS read ds_read_b64_tr_b16,
// which hands every lane four consecutive contraction elements of its own column.  Measured lane mapping of that
// read: inside each block of 16 lanes, lane 4 a + e receives element e of the 8-byte pieces addressed by lanes a,
// a + 4, a + 8, a + 12 (in this order).  16-byte pieces are XOR-swizzled on the global side so that both kinds of
// read are spread over the LDS banks.  The tile list is derived from group_lens by every workgroup; the grid is sized
// for the largest tile count the sizes allow and surplus workgroups leave at once.
#include "mx_device.h"

namespace mxl {

constexpr int BF_BM = 128, BF_BN = 256;
constexpr int BF_KS = 32;                  // contraction elements per slot (two MFMA K steps of 16)
constexpr int BF_THREADS = 256;
constexpr int BF_A_BYTES = BF_BM * 64, BF_B_BYTES = BF_BN * 64, BF_STAGE = BF_A_BYTES + BF_B_BYTES;   // 8 + 16 KiB
constexpr int BF_CPITCH = 264;             // bytes per staged output row: 128 bf16 + 8 (rows spread over the banks)
constexpr int BF_GROUP_M = 8;              // tile order: super-rows of this many row tiles

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));

struct Bf16Args {
    const uint8_t* a;      // forward: activations [total_m, k];   wgrad: p [total_m, m_out]
    const uint8_t* b;      // forward: weights [G, n, k] or [G, k, n];   wgrad: q [total_m, n_out]
    void* c;
    const int64_t* group_lens;
    int num_groups;
    int64_t total_m;
    int64_t m;             // wgrad: m_out
    int64_t n;             // forward: n;  wgrad: n_out
    int64_t k;             // forward: contraction length
};

__device__ __forceinline__ v4i bf_rsrc(const void* base, int64_t bytes) {
    const uint64_t p = (uint64_t)base;
    const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32) & 0xFFFF);
    r[2] = __builtin_amdgcn_readfirstlane((int)n);     // the range check covers per-lane + scalar offset: past it, zeros
    r[3] = 0x00020000;
    return r;
}
// LDS-direct 16-byte load: lane i's data lands at lds_off + 16 i.  (M0 holds nothing else in this kernel.)
__device__ __forceinline__ void bf_dma16(v4i rsrc, uint32_t lds_off, uint32_t voff, uint32_t soff) {
    asm volatile("" : "+s"(soff));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_off), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}

constexpr int bf16_lds_bytes() {
    return 2 * BF_STAGE + (MXL_MAX_GROUPS + 2) * 4 + (MXL_MAX_GROUPS + 2) * 8;
}
static_assert(BF_BM * BF_CPITCH <= 2 * BF_STAGE, "the output staging area reuses the operand stages");

// A_T / B_T: the operand's contraction dim is the slow one in memory (staged [32][cols], transposing reads).
// WGRAD: contraction over the tokens of a group (both operands A_T / B_T), one output matrix per group.
// ACCUM (wgrad): c is float32 and the result is added to it.
template <bool A_T, bool B_T, bool WGRAD, bool ACCUM>
__global__ __launch_bounds__(BF_THREADS, 2) void bf16_gemm_kernel(Bf16Args p) {
    static_assert(!WGRAD || (A_T && B_T), "wgrad contracts over tokens: both operands are token-major");
    static_assert(!ACCUM || WGRAD, "only the weight gradient accumulates");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int* pre_tiles = (int*)(smem + 2 * BF_STAGE);
    int64_t* pre_rows = (int64_t*)(pre_tiles + MXL_MAX_GROUPS + 2);
    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5;
    const int wm = w >> 1, wn = w & 1;
    const int G = p.num_groups;
    const uint32_t smem_base = (uint32_t)(uintptr_t)smem;

    // ---- group tables: prefix of rows and of 128-row tiles; lens clamped to what the buffers hold ----
    for (int i = t; i < G; i += BF_THREADS) pre_rows[i + 1] = p.group_lens ? p.group_lens[i] : p.total_m;
    __syncthreads();
    if (t == 0) {
        int tiles = 0;
        int64_t rows = 0;
        pre_tiles[0] = 0;
        pre_rows[0] = 0;
        for (int i = 0; i < G; ++i) {
            int64_t len = pre_rows[i + 1];
            len = len < 0 ? 0 : len;
            len = len > p.total_m - rows ? p.total_m - rows : len;
            tiles += (int)((len + BF_BM - 1) / BF_BM);
            rows += len;
            pre_tiles[i + 1] = tiles;
            pre_rows[i + 1] = rows;
        }
    }
    __syncthreads();

    const int tiles_n = (int)((p.n + BF_BN - 1) / BF_BN);
    const int tiles_m = WGRAD ? (int)((p.m + BF_BM - 1) / BF_BM) : pre_tiles[G];
    const int total_tiles = WGRAD ? G * tiles_m * tiles_n : tiles_m * tiles_n;
    // consecutive workgroup ids land on different XCDs: give every XCD a contiguous run of the tile order
    const int nwg = gridDim.x;
    int tile = (nwg & 7) ? (int)blockIdx.x : ((int)(blockIdx.x & 7) * (nwg >> 3) + (int)(blockIdx.x >> 3));
    if (tile >= total_tiles) return;

    int grp = 0;
    if (WGRAD) {
        grp = tile / (tiles_m * tiles_n);
        tile -= grp * tiles_m * tiles_n;
    }
    int pid_m, pid_n;
    {
        const int width = BF_GROUP_M * tiles_n;
        const int first = (tile / width) * BF_GROUP_M;
        const int gsz = (tiles_m - first) < BF_GROUP_M ? (tiles_m - first) : BF_GROUP_M;
        pid_m = first + (tile % width) % gsz;
        pid_n = (tile % width) / gsz;
    }
    const int64_t n0 = (int64_t)pid_n * BF_BN;
    const int n_valid = (p.n - n0) < BF_BN ? (int)(p.n - n0) : BF_BN;
    int m_valid, nslots;
    int64_t c_row0;                 // first output row (forward: token row; wgrad: row inside the group's matrix)
    v4i ra, rb;
    uint32_t a_step, b_step;        // bytes from one K slot to the next
    uint32_t va[2], vb[4];          // per-lane offsets of the load rounds
    if (!WGRAD) {
        int lo = 0, hi = G;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre_tiles[mid] <= pid_m) lo = mid; else hi = mid;
        }
        grp = lo;
        const int64_t g_row0 = pre_rows[grp], g_rows = pre_rows[grp + 1] - g_row0;
        const int64_t r = (int64_t)(pid_m - pre_tiles[grp]) * BF_BM;
        c_row0 = g_row0 + r;
        m_valid = (g_rows - r) < BF_BM ? (int)(g_rows - r) : BF_BM;
        nslots = (int)(p.k / BF_KS);
        // a: [total_m, k], contraction contiguous; rows past the operand's end are dropped by the range check
        const int64_t lda = p.k * 2;
        ra = bf_rsrc(p.a + c_row0 * lda, (p.total_m - c_row0) * lda);
        a_step = 64;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int row = (t >> 2) + 64 * e;
            va[e] = (uint32_t)(row * lda + 16 * ((t & 3) ^ ((row >> 2) & 3)));
        }
        if (!B_T) {
            const int64_t ldb = p.k * 2, b_row0 = (int64_t)grp * p.n + n0;
            rb = bf_rsrc(p.b + b_row0 * ldb, ((int64_t)G * p.n - b_row0) * ldb);
            b_step = 64;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = (t >> 2) + 64 * e;
                vb[e] = (uint32_t)(row * ldb + 16 * ((t & 3) ^ ((row >> 2) & 3)));
            }
        } else {
            // b_g: [k, n]: 32 contraction rows of 512 bytes per slot; the descriptor ends with the group's matrix
            const int64_t ldb = p.n * 2;
            rb = bf_rsrc(p.b + ((int64_t)grp * p.k * p.n + n0) * 2, (p.k * p.n - n0) * 2);
            b_step = (uint32_t)(BF_KS * ldb);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = (t >> 5) + 8 * e;
                vb[e] = (uint32_t)(row * ldb + 16 * ((t & 31) ^ ((row & 3) << 1)));
            }
        }
    } else {
        const int64_t m0 = (int64_t)pid_m * BF_BM;
        c_row0 = m0;
        m_valid = (p.m - m0) < BF_BM ? (int)(p.m - m0) : BF_BM;
        const int64_t t0 = pre_rows[grp], len = pre_rows[grp + 1] - t0;
        nslots = (int)((len + BF_KS - 1) / BF_KS);
        // p: [total_m, m_out], q: [total_m, n_out], token-major; the descriptors end with the group's last token, so
        // the rows of a partly filled last slot read as zero
        const int64_t lda = p.m * 2, ldb = p.n * 2;
        ra = bf_rsrc(p.a + t0 * lda + m0 * 2, len * lda - m0 * 2);
        rb = bf_rsrc(p.b + t0 * ldb + n0 * 2, len * ldb - n0 * 2);
        a_step = (uint32_t)(BF_KS * lda);
        b_step = (uint32_t)(BF_KS * ldb);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int row = (t >> 4) + 16 * e;
            va[e] = (uint32_t)(row * lda + 16 * ((t & 15) ^ ((row & 3) << 1)));
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = (t >> 5) + 8 * e;
            vb[e] = (uint32_t)(row * ldb + 16 * ((t & 31) ^ ((row & 3) << 1)));
        }
    }
    a_step = (uint32_t)__builtin_amdgcn_readfirstlane((int)a_step);
    b_step = (uint32_t)__builtin_amdgcn_readfirstlane((int)b_step);
    nslots = __builtin_amdgcn_readfirstlane(nslots);

    auto issue = [&](int slot, int stage) __attribute__((always_inline)) {
        const uint32_t base = smem_base + (uint32_t)(stage * BF_STAGE) + (uint32_t)(w * 1024);
        const uint32_t sa = (uint32_t)slot * a_step, sb = (uint32_t)slot * b_step;
#pragma unroll
        for (int e = 0; e < 2; ++e) bf_dma16(ra, base + e * 4096, va[e], sa);
#pragma unroll
        for (int e = 0; e < 4; ++e) bf_dma16(rb, base + BF_A_BYTES + e * 4096, vb[e], sb);
    };

    // ---- per-lane constants of the fragment reads ----
    // contiguous operand, 64-byte rows: lane (row lr, half g) reads piece 2 ks + g, XOR (row / 4) % 4
    const int ca_row = wm * 64 + lr, cb_row = wn * 128 + lr;
    // transposed operand: this lane ADDRESSES row j of a 4-row group, 8-byte piece `a4` of its 16-lane block's 16 columns
    const int tj = (l & 15) >> 2, ta4 = l & 3, tblk = (l >> 4) & 1;
    const int t_colbyte = 32 * tblk + 8 * ta4;     // byte offset of the piece inside a 32-column fragment

    v16f acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    auto read_contig = [&](const uint8_t* base, int row, int ks) __attribute__((always_inline)) {
        return *(const v8bf*)(base + row * 64 + 16 * ((2 * ks + g) ^ ((row >> 2) & 3)));
    };
    // pitch: bytes per staged contraction row (256 for the 128-wide operand, 512 for the 256-wide one); col0: first
    // column of the fragment inside the tile
    auto read_trans = [&](uint8_t* base, int pitch, int col0, int ks) __attribute__((always_inline)) {
        v8bf out;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = 16 * ks + 8 * g + 4 * h + tj;
            const int byte = 2 * col0 + t_colbyte;
            uint8_t* ptr = base + row * pitch + 16 * ((byte >> 4) ^ ((row & 3) << 1)) + (byte & 15);
            const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)ptr);
            const v4bf vb4 = __builtin_bit_cast(v4bf, v);
            out[4 * h] = vb4[0]; out[4 * h + 1] = vb4[1]; out[4 * h + 2] = vb4[2]; out[4 * h + 3] = vb4[3];
        }
        return out;
    };

    if (nslots > 0) issue(0, 0);
    for (int s = 0; s < nslots; ++s) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();     // slot s has landed everywhere, and every wave has left the other stage
        if (s + 1 < nslots) issue(s + 1, (s + 1) & 1);
        uint8_t* sa = smem + (s & 1) * BF_STAGE;
        uint8_t* sb = sa + BF_A_BYTES;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8bf fa[2], fb[4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = A_T ? read_trans(sa, 256, wm * 64 + 32 * i, ks) : read_contig(sa, ca_row + 32 * i, ks);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                fb[j] = B_T ? read_trans(sb, 512, wn * 128 + 32 * j, ks) : read_contig(sb, cb_row + 32 * j, ks);
            // the N-side fragment is MFMA source 0: a lane then holds 4 consecutive output columns per register quad
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
    }
    __syncthreads();         // every wave is done with the stages: they become the output staging area

    // lane (lr, g) of fragment (i, j) holds row 32 i + lr, columns 32 j + 8 q + 4 g .. + 3 in registers 4 q .. 4 q + 3
    if (ACCUM) {
        float* c = (float*)p.c + ((int64_t)grp * p.m + c_row0) * p.n + n0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = wm * 64 + 32 * i + lr;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int col = wn * 128 + 32 * j + 8 * q + 4 * g;
                    if (row < m_valid && col < n_valid) {      // n_out is a multiple of 8: a quad is in or out as a whole
                        v4f* dst = (v4f*)(c + (int64_t)row * p.n + col);
                        v4f o = *dst;
                        o[0] += acc[i][j][4 * q]; o[1] += acc[i][j][4 * q + 1]; o[2] += acc[i][j][4 * q + 2]; o[3] += acc[i][j][4 * q + 3];
                        *dst = o;
                    }
                }
        }
    } else {
        uint16_t* c = (uint16_t*)p.c + ((WGRAD ? (int64_t)grp * p.m : 0) + c_row0) * p.n + n0;
        // two passes, one per 128-column half: its waves stage 128 x 128 bf16, then all threads store whole rows
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h) __syncthreads();
            if (wn == h) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const v4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                            (__bf16)acc[i][j][4 * q + 3]};
                            *(v4bf*)(smem + (wm * 64 + 32 * i + lr) * BF_CPITCH + (32 * j + 8 * q + 4 * g) * 2) = o;
                        }
            }
            __syncthreads();
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = u * BF_THREADS + t, row = idx >> 4, piece = idx & 15;
                const int col = h * 128 + piece * 8;
                if (row < m_valid && col < n_valid) {
                    const uint2 lo = *(const uint2*)(smem + row * BF_CPITCH + piece * 16);      // rows are 8-byte aligned
                    const uint2 hi = *(const uint2*)(smem + row * BF_CPITCH + piece * 16 + 8);
                    *(uint4*)(c + (int64_t)row * p.n + col) = make_uint4(lo.x, lo.y, hi.x, hi.y);
                }
            }
        }
    }
}

template <bool A_T, bool B_T, bool WGRAD, bool ACCUM>
static int launch_bf16(const Bf16Args& a, int64_t max_tiles, hipStream_t st) {
    constexpr int lds = bf16_lds_bytes();
    if (!device_is_gfx950()) return MXL_ENODEV;
    static std::atomic<bool> attr_set[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MXL_ELAUNCH;
    auto kern = bf16_gemm_kernel<A_T, B_T, WGRAD, ACCUM>;
    if (!attr_set[dev & 63].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return MXL_ELAUNCH;
        attr_set[dev & 63].store(true, std::memory_order_release);
    }
    if (max_tiles <= 0) return MXL_OK;
    const int64_t grid = (max_tiles + 7) / 8 * 8;
    if (grid > 0x7FFFFFFF) return MXL_EINVAL;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(BF_THREADS), lds, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_grouped_gemm_bf16(const void* a_bf16, const void* b_bf16, void* c_bf16, const int64_t* group_lens,
                                     int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream) {
    if (flags & ~(uint32_t)MXL_BF_B_KN) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % 8 != 0 || k % BF_KS != 0) return MXL_EINVAL;
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS || (num_groups > 1 && !group_lens)) return MXL_EINVAL;
    if (total_m == 0) return MXL_OK;
    if (!a_bf16 || !b_bf16 || !c_bf16) return MXL_EINVAL;
    if ((((uintptr_t)a_bf16 | (uintptr_t)b_bf16 | (uintptr_t)c_bf16) & 15) != 0) return MXL_EINVAL;
    // offsets inside a tile's operand rows are 32-bit
    if (256 * k * 2 >= ((int64_t)1 << 31) || k * n * 2 >= ((int64_t)1 << 32)) return MXL_EINVAL;
    Bf16Args a{(const uint8_t*)a_bf16, (const uint8_t*)b_bf16, c_bf16, group_lens, num_groups, total_m, 0, n, k};
    const int64_t max_tiles = (total_m / BF_BM + num_groups) * ((n + BF_BN - 1) / BF_BN);
    if (flags & MXL_BF_B_KN) return launch_bf16<false, true, false, false>(a, max_tiles, (hipStream_t)stream);
    return launch_bf16<false, false, false, false>(a, max_tiles, (hipStream_t)stream);
}

extern "C" int mxl_grouped_gemm_bf16_wgrad(const void* p_bf16, const void* q_bf16, void* c, const int64_t* group_lens,
                                           int num_groups, int64_t total_m, int64_t m_out, int64_t n_out, uint32_t flags,
                                           void* stream) {
    if (flags & ~(uint32_t)MXL_BF_ACCUM_F32) return MXL_EINVAL;
    if (total_m < 0 || m_out <= 0 || n_out <= 0 || m_out % 8 != 0 || n_out % 8 != 0) return MXL_EINVAL;
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS || (num_groups > 1 && !group_lens)) return MXL_EINVAL;
    if (!c || ((uintptr_t)c & 15) != 0) return MXL_EINVAL;
    if (total_m > 0 && (!p_bf16 || !q_bf16 || (((uintptr_t)p_bf16 | (uintptr_t)q_bf16) & 15) != 0)) return MXL_EINVAL;
    // the K-slot advance inside a group's token range is a 32-bit byte offset
    if (total_m * m_out * 2 >= ((int64_t)1 << 32) || total_m * n_out * 2 >= ((int64_t)1 << 32)) return MXL_EINVAL;
    Bf16Args a{(const uint8_t*)p_bf16, (const uint8_t*)q_bf16, c, group_lens, num_groups, total_m, m_out, n_out, 0};
    const int64_t max_tiles = (int64_t)num_groups * ((m_out + BF_BM - 1) / BF_BM) * ((n_out + BF_BN - 1) / BF_BN);
    if (flags & MXL_BF_ACCUM_F32) return launch_bf16<true, true, true, true>(a, max_tiles, (hipStream_t)stream);
    return launch_bf16<true, true, true, false>(a, max_tiles, (hipStream_t)stream);
}
