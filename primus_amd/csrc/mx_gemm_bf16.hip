// Grouped GEMM on unquantised bf16 operands for gfx950 (v_mfma_f32_32x32x16_bf16): what the reference's grouped
// linear runs when no low-precision recipe is active -- the first / last layers of an FP4 run fall back to it --
// (primus/backends/megatron/core/extensions/primus_turbo.py:2210-2216, primus/backends/megatron/core/fp4_utils.py:155-165),
// with tokens-per-expert consumed on the device like the quantised kernels do: no host read, capturable in a graph.
//
//   forward / dgrad :  c[rows of group g, n] = a[rows of group g, k] . b_g^T        b_g = [n, k]   (contraction contiguous)
//                                                                   or . b_g          b_g = [k, n]   (MXL_BF_B_KN)
//   wgrad           :  c[g][m_out, n_out] = sum over the tokens t of group g of p[t, m_out] * q[t, n_out]
//
// One workgroup (4 waves, 2 x 2) per BM x 256 output tile, in two sizes chosen per launch: BM = 256 (a wave owns
// 128 x 128 = 4 x 4 MFMA tiles of 32 x 32, 256 fp32 accumulators, one workgroup per CU, a ring of four 32 KiB LDS
// stages filled three K slots ahead) for groups of many rows, and BM = 128 (64 x 128 per wave, two workgroups per CU,
// two stages) for groups of a few hundred rows, where a 256-row tile would mostly hold padding.  K advances in slots
// of 32 elements (64 bytes per row), filled by LDS-direct loads (buffer_load ... lds); loads complete in order, so a
// partial s_waitcnt leaves the younger slots in flight, and there is one barrier per slot.  An operand whose contraction dim is contiguous in memory is
// staged [rows][32] and read with ds_read_b128; one whose contraction dim is the slow one (the [k, n] weight, both
// operands of wgrad) is staged as it lies, [32][columns], and read with the transposing LDS read ds_read_b64_tr_b16,
// which hands every lane four consecutive contraction elements of its own column.  Measured lane mapping of that
// read: inside each block of 16 lanes, lane 4 a + e receives element e of the 8-byte pieces addressed by lanes a,
// a + 4, a + 8, a + 12 (in this order).  16-byte pieces are XOR-swizzled on the global side so that both kinds of
// read are spread over the LDS banks.  The tile list is derived from group_lens by every workgroup; the workgroups
// are persistent and walk it in rounds.
#include "mx_device.h"

#include <type_traits>

namespace mxl {

constexpr int BF_BN = 256;
constexpr int BF_KS = 32;                  // contraction elements per slot (two MFMA K steps of 16)
constexpr int BF_THREADS = 256;
constexpr int BF_B_BYTES = BF_BN * 64;     // 16 KiB of b per stage; a: BM * 64
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

// the same with the LDS address formed in the request's own scalar instruction (base + constant): two scalar
// instructions per request instead of five
template <int LDS_IMM>
__device__ __forceinline__ void bf_dma16_at(v4i rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, %4 offen lds"
                 :
                 : "s"(lds_base), "n"(LDS_IMM), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "scc");
}

constexpr int bf16_lds_bytes(int bm, int nst) {
    return nst * (bm * 64 + BF_B_BYTES) + (MXL_MAX_GROUPS + 2) * 4 + (MXL_MAX_GROUPS + 2) * 8;
}
// number of gaps g in [first, m) that are not wave ph's request gaps (g % 4 == ph): the index of the fragment read
// that the gap behind MFMA m holds
constexpr int bf_read_index(int m, int first, int ph) {
    int n = 0;
    for (int g = first; g < m; ++g) n += (g & 3) != ph;
    return n;
}
template <int N>
__device__ __forceinline__ void bf_wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// A_T / B_T: the operand's contraction dim is the slow one in memory (staged [32][cols], transposing reads).
// WGRAD: contraction over the tokens of a group (both operands A_T / B_T), one output matrix per group.
// ACCUM (wgrad): c is float32 and the result is added to it.
template <int BF_BM, int NST, bool A_T, bool B_T, bool WGRAD, bool ACCUM>
__global__ __launch_bounds__(BF_THREADS, BF_BM == 256 ? 1 : 2) void bf16_gemm_kernel(Bf16Args p) {
    static_assert(!WGRAD || (A_T && B_T), "wgrad contracts over tokens: both operands are token-major");
    static_assert(!ACCUM || WGRAD, "only the weight gradient accumulates");
    static_assert((BF_BM == 128 && NST == 2) || (BF_BM == 256 && NST == 4), "tile sizes built");
    constexpr int BF_A_BYTES = BF_BM * 64, BF_STAGE = BF_A_BYTES + BF_B_BYTES;
    constexpr int MI = BF_BM / 64;             // 32-row fragments per wave
    constexpr int AR = BF_BM / 64;             // load rounds of 4 KiB for a (b: 4)
    constexpr int LOADS = AR + 4;              // requests per wave and slot
    static_assert(BF_BM * BF_CPITCH <= NST * BF_STAGE, "the output staging area reuses the operand stages");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int* pre_tiles = (int*)(smem + NST * BF_STAGE);
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
    // Persistent workgroups (one per CU for the 256-row tile, two for the 128-row one) walk the tile order in rounds:
    // every workgroup starts its tile of a round at the same time and all tiles of a launch have the same contraction
    // length, so the 32 tiles an XCD works on stay within a few K slots of each other and share their operand panels
    // through that XCD's L2 (with one workgroup per tile, started whenever a CU fell free, the tiles of an XCD drifted
    // apart and the launch filled the L2s with 1.75 times the bytes).  Consecutive workgroup ids land on different XCDs:
    // XCD x takes the x-th run of gridDim / 8 tiles of every round.
    const int nwg = gridDim.x;
    const int vwg = (nwg & 7) ? (int)blockIdx.x : ((int)(blockIdx.x & 7) * (nwg >> 3) + (int)(blockIdx.x >> 3));
  for (int tile_id = vwg; tile_id < total_tiles; tile_id += nwg) {
    int tile = tile_id;
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
    uint32_t va[AR], vb[4];         // per-lane offsets of the load rounds
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
        for (int e = 0; e < AR; ++e) {
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
                vb[e] = (uint32_t)(row * ldb + 16 * ((t & 31) ^ ((row & 3) << 2)));
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
        // a round of 4 KiB holds 32 / AR contraction rows of BM columns
#pragma unroll
        for (int e = 0; e < AR; ++e) {
            const int row = t / (BF_BM / 8) + (32 / AR) * e;
            va[e] = (uint32_t)(row * lda + 16 * ((t % (BF_BM / 8)) ^ ((row & 3) << 2)));
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = (t >> 5) + 8 * e;
            vb[e] = (uint32_t)(row * ldb + 16 * ((t & 31) ^ ((row & 3) << 2)));
        }
    }
    a_step = (uint32_t)__builtin_amdgcn_readfirstlane((int)a_step);
    b_step = (uint32_t)__builtin_amdgcn_readfirstlane((int)b_step);
    nslots = __builtin_amdgcn_readfirstlane(nslots);

    auto issue = [&](int slot, int stage) __attribute__((always_inline)) {
        const uint32_t base = smem_base + (uint32_t)(stage * BF_STAGE) + (uint32_t)(w * 1024);
        const uint32_t sa = (uint32_t)slot * a_step, sb = (uint32_t)slot * b_step;
#pragma unroll
        for (int e = 0; e < AR; ++e) bf_dma16(ra, base + e * 4096, va[e], sa);
#pragma unroll
        for (int e = 0; e < 4; ++e) bf_dma16(rb, base + BF_A_BYTES + e * 4096, vb[e], sb);
    };

    // ---- per-lane constants of the fragment reads ----
    // contiguous operand, 64-byte rows: lane (row lr, half g) reads piece 2 ks + g, XOR (row / 4) % 4
    const int ca_row = wm * (BF_BM / 2) + lr, cb_row = wn * 128 + lr;
    // transposed operand: this lane ADDRESSES row j of a 4-row group, 8-byte piece `a4` of its 16-lane block's 16 columns
    const int tj = (l & 15) >> 2, ta4 = l & 3, tblk = (l >> 4) & 1;
    const int t_colbyte = 32 * tblk + 8 * ta4;     // byte offset of the piece inside a 32-column fragment

    v16f acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; ++i)
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
            uint8_t* ptr = base + row * pitch + 16 * ((byte >> 4) ^ ((row & 3) << 2)) + (byte & 15);
            const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)ptr);
            const v4bf vb4 = __builtin_bit_cast(v4bf, v);
            out[4 * h] = vb4[0]; out[4 * h + 1] = vb4[1]; out[4 * h + 2] = vb4[2]; out[4 * h + 3] = vb4[3];
        }
        return out;
    };

    // row fragments of this wave that hold rows of the tile (the others are neither read nor multiplied)
    int live = (m_valid - wm * (BF_BM / 2) + 31) >> 5;
    live = __builtin_amdgcn_readfirstlane(live < 0 ? 0 : (live > MI ? MI : live));

    // slot s has landed when at most the requests of the younger slots in flight are outstanding
    auto wait_slot = [&](int s) __attribute__((always_inline)) {
        const int younger = nslots - 1 - s;
        if (NST >= 4 && younger >= 2) bf_wait_vm<2 * LOADS>();
        else if (NST >= 3 && younger >= 1) bf_wait_vm<LOADS>();
        else bf_wait_vm<0>();
    };
    auto read_a = [&](uint8_t* sa, int i, int ks) __attribute__((always_inline)) {
        return A_T ? read_trans(sa, BF_BM * 2, wm * (BF_BM / 2) + 32 * i, ks) : read_contig(sa, ca_row + 32 * i, ks);
    };
    auto read_b = [&](uint8_t* sb, int j, int ks) __attribute__((always_inline)) {
        return B_T ? read_trans(sb, 512, wn * 128 + 32 * j, ks) : read_contig(sb, cb_row + 32 * j, ks);
    };
    if constexpr (NST >= 4) {
      if (live == MI && nslots > 0) {
        // One wave per SIMD: nothing but this wave's own instruction order keeps the MFMA pipe fed, so the order is
        // written out and pinned (sched_barrier): every fragment read and every load request sits between two MFMAs.
        // A slot is two halves of 16 MFMAs (4 x 4 fragments, 16 contraction elements).  While the MFMAs of half 0 run,
        // the fragments of half 1 are read; the first four MFMAs of half 1 are issued in front of the slot barrier (so
        // the pipe has work while the waves meet), the fragments of the next slot's half 0 are read behind it.
        // The 8 requests of slot s + 3 go out four per half, and the four waves -- which run in lockstep between the
        // barriers, one per SIMD -- take turns: wave PH issues behind MFMA 4 e + PH, so the address unit sees one
        // request per MFMA time instead of four at once and no wave waits at the unit's queue with its MFMA pipe
        // running empty (a bf16 MFMA is over in 32 clocks, a request occupies the unit for about 16).
        // Requests past the last slot fetch the last slot again (into a stage nobody reads any more): the request
        // count per slot is then the same in every iteration and the partial waits are constants.
        // The N-side fragment is MFMA source 0, so that a lane holds 4 consecutive output columns per register quad.
        static_assert(MI == 4 && AR == 4, "written out for the 256-row tile");
        const int last = nslots - 1;
#pragma unroll
        for (int s = 0; s < NST - 1; ++s) issue(s < last ? s : last, s);
        bf_wait_vm<2 * LOADS>();
        __syncthreads();
        auto run = [&](auto ph_tag) __attribute__((always_inline)) {
            constexpr int PH = decltype(ph_tag)::value;
            v8bf fa0[4], fb0[4], fa1[4], fb1[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) fb0[j] = read_b(smem + BF_A_BYTES, j, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) fa0[i] = read_a(smem, i, 0);
#define BF_PIN __builtin_amdgcn_sched_barrier(0)
            // The gap behind MFMA number M = 4 j + i of a half holds at most one other instruction of weight: wave PH's
            // load request (M - PH) / 4 of the half when M % 4 == PH, else the next fragment read (eight per half,
            // in the order the next half's MFMAs need them: b0, a0 .. a3, b1 .. b3), from gap FIRST on.
            auto rd = [&](auto r_tag, v8bf (&fa)[4], v8bf (&fb)[4], uint8_t* pa, uint8_t* pb, int ks) __attribute__((always_inline)) {
                constexpr int R = decltype(r_tag)::value;
                if constexpr (R == 0) fb[0] = read_b(pb, 0, ks);
                else if constexpr (R <= 4) fa[R - 1] = read_a(pa, R - 1, ks);
                else fb[R - 4] = read_b(pb, R - 4, ks);
            };
#define BF_STEP(FA, FB, M, R, VO, SO, OFF, RFA, RFB, PA, PB, KS, FIRST)                                                    \
    acc[(M) & 3][(M) >> 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FB[(M) >> 2], FA[(M) & 3], acc[(M) & 3][(M) >> 2], 0, 0, 0); \
    if constexpr (((M) & 3) == PH) bf_dma16_at<(OFF) + ((M) >> 2) * 4096>(R, in_base, VO[(M) >> 2], SO);                     \
    else if constexpr ((M) >= (FIRST) && bf_read_index(M, FIRST, PH) < 8)                                                  \
        rd(std::integral_constant<int, bf_read_index(M, FIRST, PH)>{}, RFA, RFB, PA, PB, KS);                              \
    BF_PIN
#define BF_HALF0(M) BF_STEP(fa0, fb0, M, ra, va, in_sa, 0, fa1, fb1, sa, sb, 1, 0)
#define BF_HALF1(M) BF_STEP(fa1, fb1, M, rb, vb, in_sb, BF_A_BYTES, fa0, fb0, na, nb, 0, 4)
            int stage = 0;                            // stage of slot s; slot s + 3 goes into the stage in front of it
            for (int s = 0; s < nslots; ++s) {
                uint8_t* sa = smem + stage * BF_STAGE;
                uint8_t* sb = sa + BF_A_BYTES;
                const int in_slot = s + NST - 1 < last ? s + NST - 1 : last;
                const uint32_t in_base = smem_base + (uint32_t)((stage == 0 ? NST - 1 : stage - 1) * BF_STAGE) + (uint32_t)(w * 1024);
                const uint32_t in_sa = (uint32_t)in_slot * a_step, in_sb = (uint32_t)in_slot * b_step;
                stage = stage == NST - 1 ? 0 : stage + 1;
                uint8_t* na = smem + stage * BF_STAGE;
                uint8_t* nb = na + BF_A_BYTES;
                // ---- half 0 multiplies, half 1 is read; requests: the a rows of slot s + 3 ----
                BF_HALF0(0); BF_HALF0(1); BF_HALF0(2); BF_HALF0(3); BF_HALF0(4); BF_HALF0(5); BF_HALF0(6); BF_HALF0(7);
                BF_HALF0(8); BF_HALF0(9); BF_HALF0(10); BF_HALF0(11); BF_HALF0(12); BF_HALF0(13); BF_HALF0(14); BF_HALF0(15);
                // ---- half 1 multiplies; behind the barrier the next slot's half 0 is read; requests: the b rows ----
                BF_HALF1(0); BF_HALF1(1); BF_HALF1(2); BF_HALF1(3);
                // slot s + 1 has landed when only slot s + 2, the a rows of slot s + 3 and its first b request are outstanding
                // (waves of a ragged tile that run the generic loop below meet the same barriers: one per slot)
                if (s + 1 < nslots) {
                    bf_wait_vm<LOADS + AR + 1>();
                    __syncthreads();   // slot s + 1 is in LDS for every wave; every wave holds its fragments of slot s
                }
                BF_PIN;
                BF_HALF1(4); BF_HALF1(5); BF_HALF1(6); BF_HALF1(7); BF_HALF1(8); BF_HALF1(9);
                BF_HALF1(10); BF_HALF1(11); BF_HALF1(12); BF_HALF1(13); BF_HALF1(14); BF_HALF1(15);
            }
#undef BF_HALF0
#undef BF_HALF1
#undef BF_STEP
#undef BF_PIN
        };
        if (w == 0) run(std::integral_constant<int, 0>{});
        else if (w == 1) run(std::integral_constant<int, 1>{});
        else if (w == 2) run(std::integral_constant<int, 2>{});
        else run(std::integral_constant<int, 3>{});
        bf_wait_vm<0>();     // the repeated requests of the last slots must not land in the output staging area
      }
    }
    if (NST < 4 || live != MI) {
#pragma unroll
        for (int s = 0; s < NST - 1; ++s)
            if (s < nslots) issue(s, s);
        int stage = 0, stage_in = NST - 1;        // stage of slot s; stage that slot s + NST - 1 goes into
        for (int s = 0; s < nslots; ++s) {
            wait_slot(s);
            __syncthreads();     // slot s is in LDS for every wave, and every wave has left the stage of slot s - 1
            if (s + NST - 1 < nslots) issue(s + NST - 1, stage_in);
            uint8_t* sa = smem + stage * BF_STAGE;
            uint8_t* sb = sa + BF_A_BYTES;
            if (live > 0) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    v8bf fb[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) fb[j] = read_b(sb, j, ks);
                    if (NST == 2 || live == MI) {
                        v8bf fa[MI];
#pragma unroll
                        for (int i = 0; i < MI; ++i) fa[i] = read_a(sa, i, ks);
#pragma unroll
                        for (int i = 0; i < MI; ++i)
#pragma unroll
                            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
                    } else {
#pragma unroll
                        for (int i = 0; i < MI; ++i) {
                            if (i < live) {
                                const v8bf fa = read_a(sa, i, ks);
#pragma unroll
                                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa, acc[i][j], 0, 0, 0);
                            }
                        }
                    }
                }
            }
            stage = stage == NST - 1 ? 0 : stage + 1;
            stage_in = stage_in == NST - 1 ? 0 : stage_in + 1;
        }
    }
    __syncthreads();         // every wave is done with the stages: they become the output staging area

    // lane (lr, g) of fragment (i, j) holds row 32 i + lr, columns 32 j + 8 q + 4 g .. + 3 in registers 4 q .. 4 q + 3
    if (ACCUM) {
        float* c = (float*)p.c + ((int64_t)grp * p.m + c_row0) * p.n + n0;
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int row = wm * (BF_BM / 2) + 32 * i + lr;
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
        // two passes, one per 128-column half: its waves stage BM x 128 bf16, then all threads store whole rows
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h) __syncthreads();
            if (wn == h) {
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const v4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                            (__bf16)acc[i][j][4 * q + 3]};
                            *(v4bf*)(smem + (wm * (BF_BM / 2) + 32 * i + lr) * BF_CPITCH + (32 * j + 8 * q + 4 * g) * 2) = o;
                        }
            }
            __syncthreads();
#pragma unroll
            for (int u = 0; u < BF_BM / 16; ++u) {
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
    __syncthreads();         // every wave has left the staging area: the next tile's requests may overwrite it
  }
}

static int bf16_num_cus(int dev) {
    static std::atomic<int> cached[64];
    int v = cached[dev & 63].load(std::memory_order_relaxed);
    if (v) return v;
    hipDeviceProp_t pr;
    if (hipGetDeviceProperties(&pr, dev) != hipSuccess || pr.multiProcessorCount <= 0) return 256;
    cached[dev & 63].store(pr.multiProcessorCount, std::memory_order_relaxed);
    return pr.multiProcessorCount;
}

template <int BM, int NST, bool A_T, bool B_T, bool WGRAD, bool ACCUM>
static int launch_bf16(const Bf16Args& a, int64_t max_tiles, hipStream_t st) {
    constexpr int lds = bf16_lds_bytes(BM, NST);
    if (!device_is_gfx950()) return MXL_ENODEV;
    static std::atomic<bool> attr_set[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MXL_ELAUNCH;
    auto kern = bf16_gemm_kernel<BM, NST, A_T, B_T, WGRAD, ACCUM>;
    if (!attr_set[dev & 63].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return MXL_ELAUNCH;
        attr_set[dev & 63].store(true, std::memory_order_release);
    }
    if (max_tiles <= 0) return MXL_OK;
    if (max_tiles > 0x7FFFFFFF) return MXL_EINVAL;
    // persistent: as many workgroups as the device holds at once (a multiple of 8, one share per XCD), fewer for few tiles
    int64_t grid = (int64_t)bf16_num_cus(dev) * (BM == 256 ? 1 : 2);
    grid = grid / 8 * 8;
    if (grid < 8) grid = 8;
    if ((max_tiles + 7) / 8 * 8 < grid) grid = (max_tiles + 7) / 8 * 8;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(BF_THREADS), lds, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

// Tile height of a launch: the caller's choice (MXL_BF_TILE_128 / MXL_BF_TILE_256), else from the average number of
// rows per group -- the counts live on the device, the average is all the host knows.  Measured: forward / dgrad
// tiles are cut from a group's rows, and 256-row tiles win from a few hundred rows per group on (512 rows: +7 %, 4096:
// +18-24 %; below, most of a group's last tile is padding).  The weight gradient reads both operands through the
// transposing LDS reads (twice the LDS instructions per MFMA): two workgroups per CU hide that better than one, and the
// 128-row tile wins at every shape tried (+2 % at 4096 rows per group, +50 % at 512), so it is the default there.
static bool bf16_tall_tiles(uint32_t flags, int64_t rows_per_group, int64_t threshold) {
    if (flags & MXL_BF_TILE_256) return true;
    if (flags & MXL_BF_TILE_128) return false;
    return rows_per_group >= threshold;
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_grouped_gemm_bf16(const void* a_bf16, const void* b_bf16, void* c_bf16, const int64_t* group_lens,
                                     int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream) {
    if (flags & ~(uint32_t)(MXL_BF_B_KN | MXL_BF_TILE_128 | MXL_BF_TILE_256)) return MXL_EINVAL;
    if ((flags & MXL_BF_TILE_128) && (flags & MXL_BF_TILE_256)) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % 8 != 0 || k % BF_KS != 0) return MXL_EINVAL;
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS || (num_groups > 1 && !group_lens)) return MXL_EINVAL;
    if (total_m == 0) return MXL_OK;
    if (!a_bf16 || !b_bf16 || !c_bf16) return MXL_EINVAL;
    if ((((uintptr_t)a_bf16 | (uintptr_t)b_bf16 | (uintptr_t)c_bf16) & 15) != 0) return MXL_EINVAL;
    // offsets inside a tile's operand rows are 32-bit
    if (256 * k * 2 >= ((int64_t)1 << 31) || k * n * 2 >= ((int64_t)1 << 32)) return MXL_EINVAL;
    Bf16Args a{(const uint8_t*)a_bf16, (const uint8_t*)b_bf16, c_bf16, group_lens, num_groups, total_m, 0, n, k};
    const bool tall = bf16_tall_tiles(flags, total_m / num_groups, 256);
    const int64_t max_tiles = (total_m / (tall ? 256 : 128) + num_groups) * ((n + BF_BN - 1) / BF_BN);
    hipStream_t st = (hipStream_t)stream;
    if (flags & MXL_BF_B_KN)
        return tall ? launch_bf16<256, 4, false, true, false, false>(a, max_tiles, st) : launch_bf16<128, 2, false, true, false, false>(a, max_tiles, st);
    return tall ? launch_bf16<256, 4, false, false, false, false>(a, max_tiles, st) : launch_bf16<128, 2, false, false, false, false>(a, max_tiles, st);
}

extern "C" int mxl_grouped_gemm_bf16_wgrad(const void* p_bf16, const void* q_bf16, void* c, const int64_t* group_lens,
                                           int num_groups, int64_t total_m, int64_t m_out, int64_t n_out, uint32_t flags,
                                           void* stream) {
    if (flags & ~(uint32_t)(MXL_BF_ACCUM_F32 | MXL_BF_TILE_128 | MXL_BF_TILE_256)) return MXL_EINVAL;
    if ((flags & MXL_BF_TILE_128) && (flags & MXL_BF_TILE_256)) return MXL_EINVAL;
    if (total_m < 0 || m_out <= 0 || n_out <= 0 || m_out % 8 != 0 || n_out % 8 != 0) return MXL_EINVAL;
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS || (num_groups > 1 && !group_lens)) return MXL_EINVAL;
    if (!c || ((uintptr_t)c & 15) != 0) return MXL_EINVAL;
    if (total_m > 0 && (!p_bf16 || !q_bf16 || (((uintptr_t)p_bf16 | (uintptr_t)q_bf16) & 15) != 0)) return MXL_EINVAL;
    // the K-slot advance inside a group's token range is a 32-bit byte offset
    if (total_m * m_out * 2 >= ((int64_t)1 << 32) || total_m * n_out * 2 >= ((int64_t)1 << 32)) return MXL_EINVAL;
    Bf16Args a{(const uint8_t*)p_bf16, (const uint8_t*)q_bf16, c, group_lens, num_groups, total_m, m_out, n_out, 0};
    // the tiles are cut from the [m_out, n_out] matrix of every group; the contraction runs over the group's tokens
    const bool tall = bf16_tall_tiles(flags, total_m / num_groups, INT64_MAX);
    const int bm = tall ? 256 : 128;
    const int64_t max_tiles = (int64_t)num_groups * ((m_out + bm - 1) / bm) * ((n_out + BF_BN - 1) / BF_BN);
    hipStream_t st = (hipStream_t)stream;
    if (flags & MXL_BF_ACCUM_F32)
        return tall ? launch_bf16<256, 4, true, true, true, true>(a, max_tiles, st) : launch_bf16<128, 2, true, true, true, true>(a, max_tiles, st);
    return tall ? launch_bf16<256, 4, true, true, true, false>(a, max_tiles, st) : launch_bf16<128, 2, true, true, true, false>(a, max_tiles, st);
}
