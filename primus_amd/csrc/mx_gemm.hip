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
// fp32 accumulators (256 accumulator registers per lane).  K advances in slots of 128
// elements -- one full 128-byte line per FP8 row, two MFMA K steps of 64 (two MX blocks
// each) -- through a 2-slot LDS ring (2 x 64 KiB) that is filled by asynchronous
// global->LDS loads (buffer_load ... lds).  The requests for the next slots are spread
// between the MFMAs of the current one, and the fragments of K step s+1 are read from LDS
// while the MFMAs of step s run: one barrier per K step, no register staging.  E8M0 scales
// travel in double-buffered "panels" (16 bytes per row = the scales of 8 K slots).
// 16-byte chunks are XOR-swizzled so the fragment reads are bank-conflict free.
//
// MFMA operand layout (measured on gfx950): lane l holds row l%32; its 32
// bytes are k = 16g + [0,16) and k = 32 + 16g + [0,16) with g = l/32; the
// scale of (row r, block kb) is taken from lane r + 32*kb, byte `opsel` of the
// scale register.  An FP4 operand instead holds k = 32g + [0,32) in its first
// four registers (low nibble first).  The kernel feeds the N-side operand as
// MFMA source 0 so a lane ends up with 4 consecutive output columns (one
// 8-byte bf16 store).
#include <type_traits>

#include "mx_device.h"
#include "mx_gemm_addr.h"

namespace mxl {

constexpr int BM = 256, BN = 256;
constexpr int BK = 64;     // one MFMA K step (two MX blocks)
constexpr int BKP = 128;   // K per LDS slot: two K steps, one full 128-byte line per FP8 row
constexpr int NSLOT = 2;
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
    const float* alpha_a;   // ALPHA kernels: the output is multiplied by *alpha_a * *alpha_b (per-tensor
    const float* alpha_b;   // scales of tensor-wise quantised operands) before it is rounded
};

template <int FMT> struct Op {
    static constexpr bool fp4 = (FMT == kFmtE2M1);
    static constexpr int kb = fp4 ? BKP / 2 : BKP;      // bytes per row per slot (128 or 64)
    static constexpr int cpr = kb / 16;                 // 16-byte chunks per row (= loads per thread per slot)
    static constexpr int rows_per_ld = GTHREADS / cpr;  // tile rows covered by one load round
    static constexpr int tile_bytes = 256 * kb;
    // XOR swizzle of the chunk index (both measured conflict-free for 16-byte reads by
    // 32 consecutive rows): 8 chunks per 128-byte row, 4 chunks per 64-byte row.
    static __device__ __forceinline__ int swz(int row) { return fp4 ? ((row >> 2) & 3) : ((row >> 1) & 7); }
};

// ---- asynchronous global -> LDS loads ------------------------------------
// Written as inline assembly on purpose: the compiler then keeps no record of
// LDS writes in flight and does not put a full vmcnt wait in front of every
// LDS read; completion is waited for explicitly (wait_vm) before the barrier
// that publishes a stage.  The hardware writes lane i's data to LDS address
// M0 + size*i, so the XOR swizzle is applied on the global side: the lane that
// owns physical chunk (row, pch) fetches logical chunk pch ^ swz(row).
__device__ __forceinline__ v4i make_rsrc(const void* base, int64_t bytes) {
    const uint64_t p = (uint64_t)base;
    const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32) & 0xFFFF);  // stride 0: raw buffer
    r[2] = __builtin_amdgcn_readfirstlane((int)n);                             // bytes; reads past it give 0
    r[3] = 0x00020000;
    return r;
}
// The statement writes M0 (the LDS address of an LDS-direct load).  M0 cannot be named in the clobber list: the
// compiler diagnoses clobbers of reserved registers.  Nothing else in these kernels lives in M0: LDS instructions do
// not take it on gfx950 and the kernels use no relative moves, messages or interpolation, and every use here
// reloads it first.
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t lds_off, uint32_t voff, uint32_t soff) {
    asm volatile("" : "+s"(soff));   // the scalar offset has to sit in a register, also when it is a known constant
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_off), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// The same load with the LDS address formed in M0 by one scalar add (base register + constant) and the scalar
// offset taken as it is: the ring kernel keeps a round's row offset in the per-lane offset instead of adding it to
// the scalar one, which leaves two scalar instructions per request.
template <int LDS_IMM>
__device__ __forceinline__ void dma16_at(v4i rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, %4 offen lds"
                 :
                 : "s"(lds_base), "n"(LDS_IMM), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "scc");
}

// Output stores are marked non-temporal: the kernel never reads its output back, and keeping it
// out of the way leaves L2 to the operand tiles that neighbouring workgroups share.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store16_streaming(uint8_t* dst, const uint4& v) {
    const u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (u32x4*)dst);
}

// LDS -> MFMA fragment of one 32-row tile for K step ks (0 or 1) of a slot.
template <int FMT>
__device__ __forceinline__ v8i read_frag(const uint8_t* lds, int row, int ks, int g) {
    v8i f;
    const int s = Op<FMT>::swz(row);
    if (FMT != kFmtE2M1) {
        const uint4 lo = *(const uint4*)(lds + row * 128 + 16 * ((4 * ks + g) ^ s));
        const uint4 hi = *(const uint4*)(lds + row * 128 + 16 * ((4 * ks + 2 + g) ^ s));
        f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
        f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
    } else {
        const uint4 v = *(const uint4*)(lds + row * 64 + 16 * ((2 * ks + g) ^ s));
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
        f[4] = 0; f[5] = 0; f[6] = 0; f[7] = 0;
    }
    return f;
}

// Which async load (0 .. 15, -1 = none) goes out in MFMA position q of the 32 positions between
// the moment a ring slot becomes free (barrier of the second K step of slot kp) and the barrier
// that needs its new contents (second K step of slot kp+1).  Requests are spread: four waves
// issuing one 1 KiB request each per MFMA keeps the texture addresser saturated and its queue
// full, which stalls the issuing waves, MFMAs included.
__host__ __device__ constexpr int load_at(int q) {
    return (q < 24 && q % 3 != 2) ? q - q / 3 : -1;           // two out of three positions, done by q = 22
}

struct Frags {
    v8i a[4], b[4];
    int sa[4], sb[4];
};

// compile-time loop: f(integral_constant<int, I>) for I .. N - 1
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// LAYOUT 0: operand codes row-major [rows, K].  LAYOUT 1: K-chunk-major [K / 128][rows][128 elements] (what the
// quantisers write with MXL_QF_KCHUNK): the rows of a tile's K slot are one contiguous block, so a load round
// fetches 4 KiB in a row instead of 16..64 row pieces; scales are row-major in both.
// ACCUM: the output is float32 and the result is ADDED to what it holds (the weight gradient going straight
// into the fp32 main_grad buffer that the reference's bridge otherwise adds it to in a separate pass,
// primus/backends/megatron/core/extensions/primus_turbo.py:166-240); every output tile belongs to one
// workgroup, so the read-modify-write needs no atomics.
// BSHUF (row-major E2M1 operands, forward / dgrad): b's codes are in the pre-shuffled byte order of mxl_shuffle_codes
// (what gemm_fp4_impl(..., preshuffled=True) is handed, primus_turbo_mxfp4_local.py:319-331).  The order moves whole
// 16-byte pieces, so the loads fetch each piece from its shuffled place and the LDS image -- hence everything behind
// the loads -- is that of the plain layout.
template <int AFMT, int BFMT, int MODE, int LAYOUT, bool ALPHA = false, bool ACCUM = false, bool BSHUF = false>
__global__ __launch_bounds__(GTHREADS) void mx_gemm_kernel(GemmArgs p) {
    static_assert(!BSHUF || (BFMT == kFmtE2M1 && LAYOUT == 0 && MODE == MODE_FWD && !ALPHA && !ACCUM), "pre-shuffled codes: row-major E2M1 weights, forward / dgrad");
    constexpr int A_BYTES = Op<AFMT>::tile_bytes, B_BYTES = Op<BFMT>::tile_bytes;
    constexpr int STAGE = A_BYTES + B_BYTES;            // one slot: K = 128 of both operands
    constexpr int LPA = Op<AFMT>::cpr, LPB = Op<BFMT>::cpr;
    constexpr int LPT = LPA + LPB;                      // async data loads per thread per slot
    // E8M0 scales travel in "panels": 16 bytes per row = the scales of 8 K stages
    // (K = 512), one 16-byte request per row per operand, double-buffered.
    constexpr int PANEL = 256 * 16;           // one operand
    constexpr int PANELS = 2 * 2 * PANEL;     // 2 buffers x 2 operands
    // operand format codes of the MFMA: 0 = E4M3, 1 = E5M2, 4 = E2M1
    constexpr int CB = BFMT == kFmtE2M1 ? 4 : BFMT == kFmtE5M2 ? 1 : 0, BL = AFMT == kFmtE2M1 ? 4 : AFMT == kFmtE5M2 ? 1 : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* panels = smem + NSLOT * STAGE;
    int* pre_tiles = (int*)(panels + PANELS);                        // [G+1] prefix of row tiles (FWD)
    int64_t* pre_rows = (int64_t*)(pre_tiles + MXL_MAX_GROUPS + 2);  // [G+1] prefix of rows / padded cols

    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5;
    const int wm = w >> 1, wn = w & 1;
    const int G = p.num_groups;
    const uint32_t smem_base = (uint32_t)(uintptr_t)smem;  // LDS byte address of the ring

    // ---- per-workgroup group tables (device-side, no host sync) ----
    // The lens are fetched by all threads at once and summed by one.  They are clamped to what the
    // operands hold (no negative length; the running sum never passes total_m, resp. the padded width),
    // so that lens which do not match the buffers cannot send a tile outside them.
    for (int i = t; i < G; i += GTHREADS) pre_rows[i + 1] = p.group_lens ? p.group_lens[i] : p.total_m;
    __syncthreads();
    if (t == 0) {
        int tiles = 0;
        int64_t rows = 0;
        const int64_t cap = (MODE == MODE_FWD) ? p.total_m : p.k;
        pre_tiles[0] = 0;
        pre_rows[0] = 0;
        for (int i = 0; i < G; ++i) {
            int64_t len = pre_rows[i + 1];
            len = len < 0 ? 0 : len;
            if (MODE == MODE_FWD) {
                len = len > cap - rows ? cap - rows : len;
                tiles += (int)((len + BM - 1) / BM);
                rows += len;
            } else {
                int64_t seg = (len + MXL_SEG_ALIGN - 1) / MXL_SEG_ALIGN * MXL_SEG_ALIGN;
                seg = seg > cap - rows ? cap - rows : seg;
                rows += seg;
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

    const int64_t lda = Op<AFMT>::fp4 ? p.k / 2 : p.k;
    const int64_t ldb = Op<BFMT>::fp4 ? p.k / 2 : p.k;
    const int64_t ld_s = p.k / 32;  // scale row pitch (both operands)
    const int64_t a_rows_total = (MODE == MODE_FWD) ? p.total_m : p.m;
    const int64_t b_rows_total = (MODE == MODE_FWD) ? (int64_t)G * p.n : p.n;

    // per-thread constants of the global -> LDS mapping (mx_gemm_addr.h holds the arithmetic and the rule it follows:
    // descriptors end with the operand, and the range check covers the per-lane and the scalar offset)
    const uint32_t a_voff = addr::slot2_code_lane(LAYOUT, t, Op<AFMT>::cpr, Op<AFMT>::swz(t / Op<AFMT>::cpr), lda, Op<AFMT>::kb);
    const uint32_t b_voff = BSHUF ? addr::slot2_code_lane_shuffled(t, Op<BFMT>::cpr, Op<BFMT>::swz(t / Op<BFMT>::cpr), ldb)
                                  : addr::slot2_code_lane(LAYOUT, t, Op<BFMT>::cpr, Op<BFMT>::swz(t / Op<BFMT>::cpr), ldb, Op<BFMT>::kb);
    // LAYOUT 1: bytes from one K chunk of an operand to the next (the host has checked that an operand stays below 4 GiB)
    const uint32_t a_cstride = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a_rows_total * Op<AFMT>::kb));
    const uint32_t b_cstride = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b_rows_total * Op<BFMT>::kb));

    const uint32_t s_voff = addr::slot2_scale_off(t, ld_s, 0u, 0);

    // Everything a tile needs, decoded from its index on the device.
    struct Tile {
        v4i ra, rb, rsa, rsb;      // buffer descriptors anchored at the tile's first rows
        uint32_t ka0, kb0, ks0;    // byte / block offsets of the contraction range
        int np;                    // K slots of 128
        int m_valid, n_valid;
        int64_t c_off;             // element offset of the tile's first output
    };
    auto decode = [&](int tile) __attribute__((always_inline)) {
        Tile d;
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
        int64_t a_row0, b_row0, c_row0, k0, k1;
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
            d.m_valid = (g_rows - r) < BM ? (int)(g_rows - r) : BM;
            b_row0 = (int64_t)grp * p.n + (int64_t)pid_n * BN;
            c_row0 = a_row0;
            k0 = 0;
            k1 = p.k;
        } else {
            a_row0 = (int64_t)pid_m * BM;
            d.m_valid = (p.m - a_row0) < BM ? (int)(p.m - a_row0) : BM;
            b_row0 = (int64_t)pid_n * BN;
            c_row0 = (int64_t)grp * p.m + a_row0;
            k0 = pre_rows[grp];
            k1 = pre_rows[grp + 1];
        }
        const int64_t n0 = (int64_t)pid_n * BN;
        d.n_valid = (p.n - n0) < BN ? (int)(p.n - n0) : BN;
        d.c_off = c_row0 * p.n + n0;
        d.np = __builtin_amdgcn_readfirstlane((int)((k1 - k0) / BKP));
        // Descriptors start at the tile's first row and end with the operand: whatever lies past the operand's last
        // byte is dropped by the range check and reads as zero; rows of a neighbouring group are read but never stored.
        {
            const addr::Desc da = addr::slot2_code_desc(LAYOUT, a_rows_total, a_row0, lda, Op<AFMT>::kb);
            const addr::Desc db = addr::slot2_code_desc(LAYOUT, b_rows_total, b_row0, ldb, Op<BFMT>::kb);
            const addr::Desc dsa = addr::slot2_scale_desc(a_rows_total, a_row0, ld_s);
            const addr::Desc dsb = addr::slot2_scale_desc(b_rows_total, b_row0, ld_s);
            d.ra = make_rsrc(p.a + da.base, da.records);
            d.rb = make_rsrc(p.b + db.base, db.records);
            d.rsa = make_rsrc(p.sa + dsa.base, dsa.records);
            d.rsb = make_rsrc(p.sb + dsb.base, dsb.records);
        }
        // first byte of the contraction range inside a row (LAYOUT 0) or its first K chunk (LAYOUT 1)
        d.ka0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(LAYOUT ? k0 / BKP : (Op<AFMT>::fp4 ? k0 / 2 : k0)));
        d.kb0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(LAYOUT ? k0 / BKP : (Op<BFMT>::fp4 ? k0 / 2 : k0)));
        d.ks0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(k0 / 32));
        return d;
    };
    // One async load of K slot `kp` (K = 128) of tile d into ring slot `slot`: round r covers
    // tile rows [r * rows_per_ld, (r+1) * rows_per_ld) of the M-side operand for r < LPA, of
    // the N-side operand for LPA <= r < LPT; a round past the end is a no-op.
    auto issue_1 = [&](const Tile& d, int kp, int slot, int r) __attribute__((always_inline)) {
        if (r < LPA) {
            const uint32_t off = addr::slot2_code_k(LAYOUT, d.ka0, kp, Op<AFMT>::kb, a_cstride) +
                                 addr::slot2_code_round(LAYOUT, r, Op<AFMT>::rows_per_ld, lda, Op<AFMT>::kb);
            dma16(d.ra, smem_base + slot * STAGE + (r * 4 + w) * 1024, a_voff, off);
        } else if (r < LPT) {
            const int i = r - LPA;
            const uint32_t off = (BSHUF ? addr::slot2_code_k_shuffled(kp) : addr::slot2_code_k(LAYOUT, d.kb0, kp, Op<BFMT>::kb, b_cstride)) +
                                 addr::slot2_code_round(LAYOUT, i, Op<BFMT>::rows_per_ld, ldb, Op<BFMT>::kb);
            dma16(d.rb, smem_base + slot * STAGE + A_BYTES + (i * 4 + w) * 1024, b_voff, off);
        }
    };
    // scale panel pn (K slots 4pn .. 4pn+3) into panel buffer pn & 1
    auto issue_s = [&](const Tile& d, int pn) __attribute__((always_inline)) {
        if (ALPHA) return;   // per-tensor factors: the block scales are the unit byte by contract and are not read
        const uint32_t base = smem_base + NSLOT * STAGE + (pn & 1) * 2 * PANEL;
        const uint32_t koff = addr::slot2_scale_off(0, ld_s, d.ks0, pn);
        dma16(d.rsa, base + w * 1024, s_voff, koff);
        dma16(d.rsb, base + PANEL + w * 1024, s_voff, koff);
    };
    // first requests of a tile: scale panel 0 and all of K slot 0
    auto issue_head = [&](const Tile& d) __attribute__((always_inline)) {
        issue_s(d, 0);
#pragma unroll
        for (int r = 0; r < LPT; ++r) issue_1(d, 0, 0, r);
    };

    // NA: how many of this wave's four 32-row fragments hold rows of the tile (see `live` below); the MFMAs and
    // fragment reads of the others are left out
#define MXL_MFMA(F, I, J) \
    do { if ((I) < NA) acc[I][J] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(F.b[J], F.a[I], acc[I][J], CB, BL, 0, F.sb[J], 0, F.sa[I]); } while (0)
#define MXL_PIN __builtin_amdgcn_sched_barrier(0)
    // read one fragment (+ its scale byte) of the K step described by (sn, pan, ks_n)
#define MXL_RD_A(F, I) \
    do { if ((I) < NA) { F.a[I] = read_frag<AFMT>(sn, wm * 128 + (I) * 32 + lr, ks_n, g); \
                         F.sa[I] = ALPHA ? 127 : pan[16 * (wm * 128 + (I) * 32 + lr)]; } } while (0)
#define MXL_RD_B(F, J) \
    do { if (NA > 0) { F.b[J] = read_frag<BFMT>(sn + A_BYTES, wn * 128 + (J) * 32 + lr, ks_n, g); \
                       F.sb[J] = ALPHA ? 127 : pan[PANEL + 16 * (wn * 128 + (J) * 32 + lr)]; } } while (0)

    int tile = vwg;
    if (tile >= total_tiles) return;
    Tile d = decode(tile);
    issue_head(d);
    while (tile < total_tiles) {
        v16f acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        Frags f0, f1;
        // K slot 0 and scale panel 0 of this tile were requested before the previous tile's
        // epilogue.  K slots past the end are requested as well (their data is never used):
        // it keeps every step of the pipeline identical and free of branches.
        wait_vm<0>();
        __syncthreads();
        // K slot 1: the part of its request window that lies before the first K step
#pragma unroll
        for (int q = 0; q < 12; ++q)
            if (load_at(q) >= 0) issue_1(d, 1, 1, load_at(q));
        {
            const uint8_t* sn = smem;
            const uint8_t* pan = panels + g;
            constexpr int ks_n = 0;
            constexpr int NA = 4;
            MXL_RD_B(f0, 0); MXL_RD_B(f0, 1); MXL_RD_B(f0, 2); MXL_RD_B(f0, 3);
            MXL_RD_A(f0, 0); MXL_RD_A(f0, 1); MXL_RD_A(f0, 2); MXL_RD_A(f0, 3);
        }
        // One K step (16 MFMAs) of K slot kp.  KS = 0: first half of the slot.  KS = 1: second
        // half; after its barrier K slot kp+1 has landed in the other ring slot and this ring
        // slot is dead, so the requests for K slot kp+2 start to go out.
        // The body is written in its final instruction order and pinned with scheduling
        // barriers; each LDS fragment read sits next to an MFMA that hides it.
        auto kstep = [&](auto ks_tag, auto sub_tag, auto na_tag, int kp, Frags& cur, Frags& nxt) __attribute__((always_inline)) {
            constexpr int KS = decltype(ks_tag)::value;
            constexpr int SUB = decltype(sub_tag)::value;      // kp & 3, known at compile time
            constexpr int NA = decltype(na_tag)::value;
            constexpr int slot = SUB & 1;
            constexpr int ks_n = 1 - KS;                       // K step (within its slot) of the fragments read here
            const int st_n = 2 * kp + KS + 1;                  // its global K-step index
            const uint8_t* sn = smem + (KS == 0 ? slot : (slot ^ 1)) * STAGE;
            const uint8_t* pan = panels + ((st_n >> 3) & 1) * 2 * PANEL + 2 * (st_n & 7) + g;
            // position m of this K step in the 32-position window of the slot being refilled:
            //   KS = 1, m >= 4 : q = m - 4   (K slot kp+2 -> this ring slot, free after the barrier below)
            //   KS = 0         : q = 12 + m  (K slot kp+1 -> the other ring slot)
            //   KS = 1, m <  4 : q = 28 + m  (K slot kp+1 -> the other ring slot)
#define MXL_LD(M) \
    do { \
        constexpr int q_ = (KS == 1) ? ((M) >= 4 ? (M) - 4 : 28 + (M)) : 12 + (M); \
        constexpr int r_ = load_at(q_); \
        if (r_ >= 0) { \
            if (KS == 1 && (M) >= 4) issue_1(d, kp + 2, slot, r_); \
            else issue_1(d, kp + 1, slot ^ 1, r_); \
        } \
    } while (0)
            MXL_MFMA(cur, 0, 0); MXL_LD(0); MXL_PIN;
            MXL_MFMA(cur, 1, 0); MXL_LD(1); MXL_PIN;
            MXL_MFMA(cur, 2, 0); MXL_LD(2); MXL_PIN;
            MXL_MFMA(cur, 3, 0); MXL_LD(3); MXL_PIN;
            if (KS == 1) wait_vm<0>();  // K slot kp+1 has landed (its last request went out several MFMAs ago)
            __syncthreads();
            MXL_PIN;
            if (KS == 1 && SUB == 0) issue_s(d, (kp >> 2) + 1);  // next scale panel; its buffer is dead since K slot kp-1
            MXL_RD_B(nxt, 0); MXL_MFMA(cur, 0, 1); MXL_LD(4); MXL_PIN;
            MXL_RD_A(nxt, 0); MXL_MFMA(cur, 1, 1); MXL_LD(5); MXL_PIN;
            MXL_RD_A(nxt, 1); MXL_MFMA(cur, 2, 1); MXL_LD(6); MXL_PIN;
            MXL_RD_A(nxt, 2); MXL_MFMA(cur, 3, 1); MXL_LD(7); MXL_PIN;
            MXL_RD_A(nxt, 3); MXL_MFMA(cur, 0, 2); MXL_LD(8); MXL_PIN;
            MXL_RD_B(nxt, 1); MXL_MFMA(cur, 1, 2); MXL_LD(9); MXL_PIN;
            MXL_RD_B(nxt, 2); MXL_MFMA(cur, 2, 2); MXL_LD(10); MXL_PIN;
            MXL_RD_B(nxt, 3); MXL_MFMA(cur, 3, 2); MXL_LD(11); MXL_PIN;
            MXL_MFMA(cur, 0, 3); MXL_LD(12); MXL_PIN;
            MXL_MFMA(cur, 1, 3); MXL_LD(13); MXL_PIN;
            MXL_MFMA(cur, 2, 3); MXL_LD(14); MXL_PIN;
            MXL_MFMA(cur, 3, 3); MXL_LD(15); MXL_PIN;
#undef MXL_LD
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        using I4 = std::integral_constant<int, 4>;
        const int np = d.np;
        auto kloop = [&](auto na) __attribute__((always_inline)) {
            for (int kp = 0; kp < np; kp += 4) {
                kstep(I0{}, I0{}, na, kp, f0, f1);
                kstep(I1{}, I0{}, na, kp, f1, f0);
                if (kp + 1 < np) {
                    kstep(I0{}, I1{}, na, kp + 1, f0, f1);
                    kstep(I1{}, I1{}, na, kp + 1, f1, f0);
                }
                if (kp + 2 < np) {
                    kstep(I0{}, I2{}, na, kp + 2, f0, f1);
                    kstep(I1{}, I2{}, na, kp + 2, f1, f0);
                }
                if (kp + 3 < np) {
                    kstep(I0{}, I3{}, na, kp + 3, f0, f1);
                    kstep(I1{}, I3{}, na, kp + 3, f1, f0);
                }
            }
        };
        // Rows of this wave's 128 that lie inside the tile.  In the forward / dgrad GEMM a group's last row tile is
        // ragged (an expert with 500 tokens: its second tile has 244 rows, a third would have a handful), and the
        // fragments past its end would multiply another group's rows into accumulators that are never stored: a wave
        // runs the loop variant for 4, 2 or 0 live fragments.  Loads and barriers are the same in all of them.
        const int live = (MODE == MODE_FWD && !ACCUM) ? d.m_valid - wm * 128 : 128;
        if (live > 64) kloop(I4{});
        else if (live > 0) kloop(I2{});
        else kloop(I0{});
        // Drain the look-ahead requests (they target the ring) and make sure every wave is done
        // reading it; then the next tile's first requests go out and overlap with the epilogue.
        wait_vm<0>();
        __syncthreads();
        // The tile's facts are uniform: moved to scalar registers they stay out of the vector registers' spills.  The
        // lane number is taken afresh from the hardware, and every offset of the epilogue is rebuilt from it: computed in
        // front of the tile loop those offsets would have to live through the main loop, where every register is taken,
        // and would come back from scratch memory one dependent load after the other.
        const int m_valid = __builtin_amdgcn_readfirstlane(d.m_valid), n_valid = __builtin_amdgcn_readfirstlane(d.n_valid);
        const int64_t c_off = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(d.c_off >> 32)) << 32) |
                                        (uint32_t)__builtin_amdgcn_readfirstlane((int)d.c_off));
        // (the count starts from a zero the optimiser cannot see through: a plain lane count is loop-invariant to it, and
        // would again be computed in front of the tile loop and spilled)
        auto lane_now = [] {
            uint32_t z = 0;
            asm volatile("" : "+v"(z));
            return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
        };
        uint16_t* ctile = p.c + c_off;
        // ACCUM: the old float32 values of the first 32-row block are requested before the next tile's operand
        // requests go out (memory returns in order per wave: behind them they would wait for 64 KiB of loads)
        float* ctile32 = (float*)p.c + c_off;
        const bool full_tile = (m_valid == BM) && (n_valid == BN);
        v4f old[ACCUM ? 2 : 1][ACCUM ? 16 : 1];
        auto fetch_old = [&](int i, v4f* dst, int el) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int row = wm * 128 + i * 32 + 4 * u + (el >> 4), col = wn * 128 + (el & 15) * 4 + jj * 64;
                    dst[jj * 8 + u] = v4f{0.f, 0.f, 0.f, 0.f};
                    if (full_tile || (row < m_valid && col < n_valid))
                        dst[jj * 8 + u] = *(const v4f*)(ctile32 + (int64_t)row * p.n + col);
                }
        };
        if (ACCUM) fetch_old(0, old[0], lane_now());
        tile += nwg;
        // (past the last tile the requests are still sent, for the last tile again: nobody reads them)
        d = decode(tile < total_tiles ? tile : total_tiles - 1);
        issue_head(d);
        MXL_PIN;  // keep the accumulator read-out below: it would otherwise be hoisted and spill

        // ---- epilogue: fp32 -> bf16 through a wave-private LDS patch (in ring slot 1, which the
        // requests above do not touch), so that the global stores are 16 bytes per lane and each
        // store instruction covers 4 rows x 256 contiguous bytes ----
        {
            // bytes per staged row: 256 + 16 spreads the rows over the banks; with two FP4 operands ring slot 1
            // is only 32 KiB, which the four 32-row patches fill exactly without the padding -- a padded patch
            // would reach into the scale panels behind the ring, which the next tile's first requests are
            // already writing
            constexpr int SP = (4 * 32 * 272 <= STAGE) ? 272 : 256;
            static_assert(4 * 32 * SP <= STAGE, "the epilogue patches must stay inside ring slot 1");
            const int el = lane_now();     // taken behind the requests above: no register is held across them
            const int elr = el & 31, eg = el >> 5;
            uint8_t* stg = smem + STAGE + w * (32 * SP);
            uint8_t* wr = stg + elr * SP + 8 * eg;                   // this lane's row while writing
            const uint8_t* rd = stg + (el >> 4) * SP + (el & 15) * 16;  // this lane's 16 bytes while reading
            const int rr = el >> 4, cc = wn * 128 + (el & 15) * 8;
            const uint32_t lane_off = (uint32_t)((rr * (int)p.n + (el & 15) * 8) * 2);
            const bool full = (m_valid == BM) && (n_valid == BN);
            float alpha = 1.f;
            if (ALPHA) alpha = *p.alpha_a * *p.alpha_b;
            if (ACCUM) {
                // float32 read-modify-write, 64 columns (256 bytes per row) of a 32-row block at a time through
                // the same patch: a memory instruction covers 4 rows x 256 contiguous bytes.  The old values of
                // a 32-row block (16 x 16 bytes per lane) are requested one block ahead, so their latency is
                // covered by the staging and the stores of the block before.
                uint8_t* wr32 = stg + elr * SP + 16 * eg;
                const int colq = wn * 128 + (el & 15) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (i + 1 < 4) fetch_old(i + 1, old[(i + 1) & 1], el);
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int jl = 0; jl < 2; ++jl)
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const int j = 2 * jj + jl;
                                v4f o = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                                if (ALPHA) o *= alpha;
                                *(v4f*)(wr32 + (jl * 32 + 8 * q) * 4) = o;
                            }
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const v4f v = *(const v4f*)(rd + 4 * u * SP);
                            const int row = wm * 128 + i * 32 + 4 * u + rr, col = colq + jj * 64;
                            if (full || (row < m_valid && col < n_valid))
                                *(v4f*)(ctile32 + (int64_t)row * p.n + col) = old[i & 1][jj * 8 + u] + v;
                        }
                    }
                    MXL_PIN;
                }
            } else {
                // Four patches of 32 rows x 128 columns go through the staging area one after the other.  The LDS runs a
                // wave's accesses in order, so patch n + 1 may be written once the reads of patch n have been ISSUED: the
                // stores of patch n, which wait for those reads, come behind the conversions and writes of patch n + 1.
                // lane (lr, g) holds row lr of a 32-row block: columns j*32 + 8q + 4g .. +3;
                // 16 lanes per row, 4 rows per store instruction; the row base is uniform
                auto write_out = [&](auto full_tag) __attribute__((always_inline)) {
                    constexpr bool FULL = decltype(full_tag)::value;
                    uint4 v[8];
                    static_for<0, 5>([&](auto it_tag) {
                        constexpr int it = decltype(it_tag)::value;
                        if constexpr (it < 4) {
                            constexpr int i = it;
#pragma unroll
                            for (int j = 0; j < 4; ++j)
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    if (ALPHA) {
#pragma unroll
                                        for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] *= alpha;
                                    }
                                    v4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                              (__bf16)acc[i][j][4 * q + 3]};
                                    *(v4bf*)(wr + (j * 32 + 8 * q) * 2) = o;
                                }
                        }
                        if constexpr (it > 0) {
                            constexpr int i = it - 1;
                            uint8_t* rowbase = (uint8_t*)(ctile + (int64_t)(wm * 128 + i * 32) * p.n + wn * 128);
#pragma unroll
                            for (int u = 0; u < 8; ++u)
                                if (FULL || (wm * 128 + i * 32 + 4 * u + rr < m_valid && cc < n_valid))
                                    store16_streaming(rowbase + (int64_t)(4 * u) * p.n * 2 + lane_off, v[u]);
                        }
                        if constexpr (it < 4) {
#pragma unroll
                            for (int u = 0; u < 8; ++u) v[u] = *(const uint4*)(rd + 4 * u * SP);
                        }
                        MXL_PIN;  // one 32-row block at a time: 64 accumulators live, not 256
                    });
                };
                if (full) write_out(std::true_type{});
                else write_out(std::false_type{});
            }
        }
    }
#undef MXL_MFMA
#undef MXL_PIN
#undef MXL_RD_A
#undef MXL_RD_B
}

// ---------------------------------------------------------------------------------------------------
// 4-slot ring kernel (FP8-family operands in the K-step-major layout, at most RING_MAX_GROUPS groups).
//
// Same tiling, MFMA schedule and epilogue idea as mx_gemm_kernel; what differs is how operands travel:
//   * a ring slot holds ONE MFMA K step (K = 64: 64-byte row pieces, 16 KiB per operand), four slots;
//   * the 8 load rounds of K step s+4 go out during step s, one per two MFMAs (six after the step's
//     barrier, the last two at the start of the next step), into the slot step s has just released:
//     a request has between two and three K steps to land, and the request stream never pauses or bunches;
//   * the wait in front of a step's barrier is partial: vmcnt(16) lets the requests of the two youngest
//     steps stay in flight (loads return in order, so anything older has landed whatever else is pending);
//   * the stream runs across tile boundaries: the last four steps of a tile request the first four steps of
//     the workgroup's next tile.  Only the 6 requests that would overwrite the slot the epilogue stages its
//     output in are held back until the epilogue has left it.
// Measured on cache-shared operands with this discipline the MFMA pipe never waits for operands; with the
// 2-slot ring of mx_gemm_kernel (one K = 128 slot in flight, everything waited for) it idles 12 % and more.
// ---------------------------------------------------------------------------------------------------
constexpr int RING_SLOTS = 4;
constexpr int RING_STAGE = 2 * 256 * BK;          // both operands, K = 64, FP8: 32 KiB
constexpr int RING_MAX_GROUPS = 256;          // what the group tables may take of the 160 KiB of LDS next to ring and panels
constexpr int RING_PANEL = 256 * 16;              // scale panel of one operand: 16 bytes per row = 8 K steps
constexpr int RING_PANEL_BUFS = 3;
constexpr int RING_TBL = RING_MAX_GROUPS + 2;

constexpr int ring_lds_bytes() {
    return RING_SLOTS * RING_STAGE + RING_PANEL_BUFS * 2 * RING_PANEL + RING_TBL * 4 + RING_TBL * 8 + RING_TBL * 4 + RING_TBL * 4;
}


// BT (forward / dgrad of FP8-format operands; E2M1 x E2M1 further down): b_codes hold the codes of the TRANSPOSED matrices -- [G, k, n] instead of
// [G, n, k], K-step-major along n: [n_ld / 64][G * k][64] -- i.e. the row-wise copy of a weight serves its dgrad GEMM
// and no transposed copy of the codes is ever written.  Valid where transposing the codes is all a transposed copy
// amounts to: 2-D 32 x 32 block scales (the quantiser's transposed SCALES are still passed as b_scales, they are
// 1/32 of the bytes) or one scale per tensor.  A K step of b is then 64 rows (contraction) x 256 columns: four pieces
// of 64 rows x 64 bytes, one per 64-column plane, each a contiguous 4 KiB; the fragments come out of LDS through the
// transposing read ds_read_b64_tr_b8, which hands a lane 8 consecutive contraction bytes of its own column.  Measured
// lane mapping of that read: inside a block of 16 lanes, lane 8 a + e receives byte e of the 8-byte pieces
// addressed by lanes a, a + 2, ..., a + 14 (in this order).
// With both operands E2M1 (128-element steps, 64-byte rows) a plane of the row-wise codes holds 128 output columns, a K
// step is 128 contraction rows of the tile's two planes (four rounds of 64 rows x 64 bytes), and the fragments come
// through ds_read_b64_tr_b4, a 16 x 16 nibble transpose inside each block of 16 lanes.
template <int AFMT, int BFMT, int MODE, bool ALPHA, bool ACCUM = false, bool BT = false>
__global__ __launch_bounds__(GTHREADS) void mx_gemm_ring_kernel(GemmArgs p) {
    static_assert(!BT || (MODE == MODE_FWD && ((AFMT != kFmtE2M1 && BFMT != kFmtE2M1) || (AFMT == kFmtE2M1 && BFMT == kFmtE2M1))),
                  "transposed weight codes: forward / dgrad, both operands FP8 formats or both E2M1");
    // ACCUM (wgrad): p.c is a float32 buffer the result is ADDED to (one workgroup per output tile: no race, and the
    // sum does not depend on any order)
    static_assert(!ACCUM || MODE == MODE_WGRAD, "the accumulating epilogue belongs to the weight-gradient GEMM");
    // F44: both operands FP4, stored like FP8 operands byte for byte -- 64-byte rows per K step, which then hold 128
    // elements: a step is two MFMA K steps (the low and the high half of every fragment register group), scale panels
    // cover 4 steps instead of 8, and a contraction range may be an odd number of steps.
    constexpr bool F44 = AFMT == kFmtE2M1 && BFMT == kFmtE2M1;
    static_assert(AFMT != kFmtE2M1 || (F44 && !ALPHA), "an FP4 row operand needs an FP4 weight operand (MX recipe)");
    static_assert(BFMT != kFmtE2M1 || F44 || (MODE == MODE_FWD && !ALPHA), "an E2M1 weight operand against FP8 rows: forward / dgrad of the MX recipe");
    constexpr bool B4 = BFMT == kFmtE2M1 && !F44;     // FP4 weights against FP8 rows: 32 bytes per row and K step
    constexpr int KS = F44 ? 2 * BK : BK;             // elements of the contraction per step
    constexpr int PSTEPS = 512 / KS;                  // steps per scale panel
    constexpr int B_ROW = B4 ? BK / 2 : BK;           // bytes of a row of b in a K step
    constexpr int ROUNDS = B4 ? 6 : 8;                // load rounds of 4 KiB per K step: 4 of a, 2 or 4 of b
    constexpr int A_BYTES = 256 * BK;                 // 16 KiB
    constexpr int STAGE = RING_STAGE;
    constexpr int PANEL = RING_PANEL;
    constexpr int CB = BFMT == kFmtE2M1 ? 4 : BFMT == kFmtE5M2 ? 1 : 0, BL = F44 ? 4 : AFMT == kFmtE5M2 ? 1 : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* panels = smem + RING_SLOTS * STAGE;
    int* pre_tiles = (int*)(panels + RING_PANEL_BUFS * 2 * PANEL);
    int64_t* pre_rows = (int64_t*)(pre_tiles + RING_TBL);
    int* pre_pan = (int*)(pre_rows + RING_TBL);                      // [G+1] prefix of scale panels (WGRAD)
    int* by_len = pre_pan + RING_TBL;                                // [G] groups by descending contraction length (WGRAD)

    const int t = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l = t & 63, lr = l & 31, g = l >> 5;
    const int wm = w >> 1, wn = w & 1;
    const int G = p.num_groups;
    const uint32_t smem_base = (uint32_t)(uintptr_t)smem;

    // ---- per-workgroup group tables (as in mx_gemm_kernel, plus the scale-panel prefix) ----
    for (int i = t; i < G; i += GTHREADS) pre_rows[i + 1] = p.group_lens ? p.group_lens[i] : p.total_m;
    __syncthreads();
    if (t == 0) {
        int tiles = 0, pans = 0;
        int64_t rows = 0;
        const int64_t cap = (MODE == MODE_FWD) ? p.total_m : p.k;
        pre_tiles[0] = 0;
        pre_rows[0] = 0;
        pre_pan[0] = 0;
        for (int i = 0; i < G; ++i) {
            int64_t len = pre_rows[i + 1];
            len = len < 0 ? 0 : len;
            if (MODE == MODE_FWD) {
                len = len > cap - rows ? cap - rows : len;
                tiles += (int)((len + BM - 1) / BM);
                rows += len;
            } else {
                int64_t seg = (len + MXL_SEG_ALIGN - 1) / MXL_SEG_ALIGN * MXL_SEG_ALIGN;
                seg = seg > cap - rows ? cap - rows : seg;
                rows += seg;
                pans += (int)((seg + 511) / 512);
            }
            pre_tiles[i + 1] = tiles;
            pre_rows[i + 1] = rows;
            pre_pan[i + 1] = pans;
        }
    }
    __syncthreads();

    // wgrad: the tiles of a group all run that group's contraction length, and lengths differ widely between
    // groups.  The tile order goes through the groups from the longest to the shortest (ties by index; groups
    // without tokens come last), and the workgroups walk it in a serpentine (below): every workgroup then gets
    // nearly the same number of K steps instead of whatever mix of groups its stride happens to hit.
    if (MODE == MODE_WGRAD) {
        for (int i = t; i < G; i += GTHREADS) {
            const int64_t len = pre_rows[i + 1] - pre_rows[i];
            int rank = 0;
            for (int j = 0; j < G; ++j) {
                const int64_t lj = pre_rows[j + 1] - pre_rows[j];
                rank += (lj > len || (lj == len && j < i)) ? 1 : 0;
            }
            by_len[rank] = i;
        }
        __syncthreads();
    }

    const int tiles_n = (int)((p.n + BN - 1) / BN);
    int tiles_m, total_tiles;
    if (MODE == MODE_FWD) {
        tiles_m = pre_tiles[G];
        total_tiles = tiles_m * tiles_n;
    } else {
        tiles_m = (int)((p.m + BM - 1) / BM);
        total_tiles = G * tiles_m * tiles_n;
    }
    const int nwg = gridDim.x;
    const int per_xcd = nwg >> 3;
    const int vwg = (nwg & 7) ? (int)blockIdx.x : ((int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3));

    const int64_t a_rows_total = (MODE == MODE_FWD) ? p.total_m : p.m;
    const int64_t b_rows_total = (MODE == MODE_FWD) ? (int64_t)G * p.n : p.n;
    // K-step-major codes: [k / 64][rows][64]; scales: [ceil(k / 512)][rows][16] (16 bytes = 8 K steps of a row)
    const uint32_t a_cstride = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a_rows_total * BK));
    // BT: the rows of b's code array are the contraction index (G * k of them); a K step moves on by 64 rows inside
    // a plane, and the four load rounds of a step are one plane apart
    const int64_t bt_rows = (int64_t)G * p.k;
    // (E2M1 x E2M1: a step is 128 contraction rows of a 128-column plane, and a tile's two planes take two rounds each)
    const uint32_t b_cstride = BT ? (uint32_t)(KS * BK) : (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b_rows_total * B_ROW));
    const uint32_t a_pstride = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a_rows_total * 16));
    const uint32_t b_pstride = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b_rows_total * 16));
    // a load round covers 64 consecutive rows = 4 KiB: thread -> (row t / 4, 16-byte piece t % 4); the XOR swizzle of
    // the piece index is applied on the global side so that the LDS image (64-byte rows) reads without bank conflicts
    // panels in a scale array: a contraction that is split into groups restarts its panels at every group
    const int64_t n_panels = (p.k + 511) / 512 + ((MODE == MODE_WGRAD && p.group_lens) ? G + 1 : 0);
    // FP4 rows are 32 bytes: a round covers 128 rows, thread -> (row t / 2, piece t % 2), pieces swapped in every
    // second group of 8 rows so that the 16-byte fragment reads of 16 consecutive rows cover all banks
    const uint32_t s_voff = addr::ring_panel_lane(t);     // scale panel: row t of the tile, 16 bytes
    // per-lane offsets of the load rounds: round e of an operand starts e * 64 rows = e * 4 KiB further on
    const uint32_t wave_base = smem_base + (uint32_t)(w * 1024);    // ring slot 0, this wave's 1 KiB of a round
    uint32_t va[4], vb[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        va[e] = addr::ring_code_lane(t, e, false);
        vb[e] = !BT ? addr::ring_code_lane(t, e, B4) : F44 ? addr::ring_bt4_lane(t, e, bt_rows) : addr::ring_bt_lane(t, e, bt_rows);
    }

    struct Tile {
        v4i ra, rb, rsa, rsb;
        uint32_t ca0, cb0;         // byte offset of the first K step of each operand
        uint32_t pa0, pb0;         // byte offset of the scale panel of the first K step
        uint32_t cal, cbl;         // byte offset of the LAST K step of the contraction range (requests never pass it)
        int nst, nst_real;         // K steps to run (>= 4, even) and how many of them multiply (the first nst_real)
        int m_valid, n_valid;
        int c_row0, c_col0;        // first output row and column of the tile
    };
    auto decode = [&](int tile) __attribute__((always_inline)) {
        Tile d;
        int grp = 0, pid_m, pid_n;
        int tl = tile;
        if (MODE == MODE_WGRAD) {
            const int pos = tl / (tiles_m * tiles_n);
            tl -= pos * tiles_m * tiles_n;
            grp = __builtin_amdgcn_readfirstlane(by_len[pos]);
        }
        {
            const int width = GROUP_M * tiles_n;
            const int gid = tl / width;
            const int first = gid * GROUP_M;
            const int gsz = (tiles_m - first) < GROUP_M ? (tiles_m - first) : GROUP_M;
            pid_m = first + (tl % width) % gsz;
            pid_n = (tl % width) / gsz;
        }
        int64_t a_row0, b_row0, c_row0, k0, k1;
        if (MODE == MODE_FWD) {
            int lo = 0, hi = G;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (pre_tiles[mid] <= pid_m) lo = mid; else hi = mid;
            }
            grp = lo;
            const int64_t g_row0 = pre_rows[grp], g_rows = pre_rows[grp + 1] - g_row0;
            const int64_t r = (int64_t)(pid_m - pre_tiles[grp]) * BM;
            a_row0 = g_row0 + r;
            d.m_valid = __builtin_amdgcn_readfirstlane((g_rows - r) < BM ? (int)(g_rows - r) : BM);
            b_row0 = (int64_t)grp * p.n + (int64_t)pid_n * BN;
            c_row0 = a_row0;
            k0 = 0;
            k1 = p.k;
        } else {
            a_row0 = (int64_t)pid_m * BM;
            d.m_valid = __builtin_amdgcn_readfirstlane((p.m - a_row0) < BM ? (int)(p.m - a_row0) : BM);
            b_row0 = (int64_t)pid_n * BN;
            c_row0 = (int64_t)grp * p.m + a_row0;
            k0 = pre_rows[grp];
            k1 = pre_rows[grp + 1];
        }
        const int64_t n0 = (int64_t)pid_n * BN;
        // the epilogue's tile facts are uniform: kept in scalar registers they survive the main loop without
        // taking part in the vector register spills
        d.n_valid = __builtin_amdgcn_readfirstlane((p.n - n0) < BN ? (int)(p.n - n0) : BN);
        d.c_row0 = __builtin_amdgcn_readfirstlane((int)c_row0);
        d.c_col0 = __builtin_amdgcn_readfirstlane((int)n0);
        // the range is a multiple of 128 elements: an even number of steps, except with FP4 rows (one step each)
        const int nreal = __builtin_amdgcn_readfirstlane((int)((k1 - k0) / KS));
        d.nst_real = nreal;
        d.nst = nreal < 4 ? 4 : nreal + (nreal & 1);
        // Descriptors start at the tile's first row inside K step 0 / panel 0 and end with the operand: the range
        // check covers the per-lane offset (row, load round) and the scalar offset (K step / panel) together, so a
        // row past the operand's last one is dropped in the last plane and reads a later plane's rows in the others.
        {
            const addr::Desc da = addr::ring_code_desc(a_rows_total, p.k / KS, a_row0, BK);
            const addr::Desc db = BT ? addr::ring_bt_desc(bt_rows, (p.n + 127) / 128 * (F44 ? 1 : 2), (int64_t)grp * p.k, (int64_t)pid_n * (F44 ? BN / 128 : BN / 64))
                                     : addr::ring_code_desc(b_rows_total, p.k / KS, b_row0, B_ROW);
            const addr::Desc dsa = addr::ring_panel_desc(a_rows_total, n_panels, a_row0), dsb = addr::ring_panel_desc(b_rows_total, n_panels, b_row0);
            d.ra = make_rsrc(p.a + da.base, da.records);
            d.rb = make_rsrc(p.b + db.base, db.records);
            d.rsa = make_rsrc(p.sa + dsa.base, dsa.records);
            d.rsb = make_rsrc(p.sb + dsb.base, dsb.records);
        }
        const uint32_t st0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(k0 / KS));
        d.ca0 = st0 * a_cstride;
        d.cb0 = st0 * b_cstride;
        d.cal = d.ca0 + (uint32_t)(nreal - 1) * a_cstride;
        d.cbl = d.cb0 + (uint32_t)(nreal - 1) * b_cstride;
        // scale panels restart at every group of a ragged contraction (wgrad): panel 0 of a tile is its group's first
        const uint32_t pan0 = (MODE == MODE_WGRAD) ? (uint32_t)__builtin_amdgcn_readfirstlane(pre_pan[grp]) : 0u;
        d.pa0 = pan0 * a_pstride;
        d.pb0 = pan0 * b_pstride;
        return d;
    };

    // ---- the request stream ----
    // Requests are issued in K-step groups of 8 rounds (A rows 0-63, 64-127, 128-191, 192-255, then B likewise).
    // lra / lrb: descriptors of the tile the stream is in; lca / lcb: byte offset of the K chunk the next group
    // starts in; ga / gb: byte offset (chunk + half) of the group in flight.
    v4i lra, lrb, crb;
    uint32_t lca, lcb, lla, llb, ga = 0, gb = 0, cgb = 0;
    auto stream_enter = [&](const Tile& d) __attribute__((always_inline)) {
        lra = d.ra; lrb = d.rb; lca = d.ca0; lcb = d.cb0; lla = d.cal; llb = d.cbl;
    };
    // start the group of the stream's next K step: fixes ga / gb and moves the stream on.  A step past the tile's
    // contraction range (a range of two steps is padded to four) requests the range's last step again: every
    // request stays inside the operand, its data is never multiplied.
    auto group_begin = [&]() __attribute__((always_inline)) {
        ga = lca < lla ? lca : lla;
        gb = lcb < llb ? lcb : llb;
        lca += a_cstride;
        lcb += b_cstride;
        // rounds 6 and 7 of this group go out at the start of the next step, possibly after the stream has
        // moved on to the next tile: they keep their own copy of the descriptor and offset
        crb = lrb;
        cgb = gb;
    };
    // round e (0 .. 7) of the group in flight into ring slot `slot` (0 .. 3, run time)
    // (slot_base already holds the wave's 1 KiB share, w * 1024; the round's 4 KiB come in as a constant)
    auto issue_e = [&](auto e_tag, uint32_t slot_base) __attribute__((always_inline)) {
        constexpr int e = decltype(e_tag)::value;
        if constexpr (e < 4) dma16_at<e * 4096>(lra, slot_base, va[e], ga);
        else if constexpr (e >= 6) dma16_at<A_BYTES + (e - 4) * 4096>(crb, slot_base, vb[e - 4], cgb);
        else dma16_at<A_BYTES + (e - 4) * 4096>(lrb, slot_base, vb[e - 4], gb);
    };
    // scale panel pn of tile d (its K steps 8 pn .. 8 pn + 7) into panel buffer `buf`: 4 KiB per operand
    auto issue_s = [&](const Tile& d, int pn, int buf) __attribute__((always_inline)) {
        if (ALPHA) return;   // per-tensor factors: the block scales are the unit byte by contract and are not read
        const uint32_t base = smem_base + (uint32_t)(RING_SLOTS * STAGE + buf * 2 * PANEL);
        dma16(d.rsa, base + w * 1024, s_voff, d.pa0 + (uint32_t)pn * a_pstride);
        dma16(d.rsb, base + PANEL + w * 1024, s_voff, d.pb0 + (uint32_t)pn * b_pstride);
    };
    auto next3 = [](int b) { return b == 2 ? 0 : b + 1; };

#define MXL_MFMA(F, I, J) \
    do { if (MF && (I) < LIVE) { \
             acc[I][J] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(F.b[J], F.a[I], acc[I][J], CB, BL, 0, F.sb[J], 0, F.sa[I]); \
             if (F44) acc[I][J] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4( \
                 __builtin_shufflevector(F.b[J], F.b[J], 4, 5, 6, 7, 4, 5, 6, 7), __builtin_shufflevector(F.a[I], F.a[I], 4, 5, 6, 7, 4, 5, 6, 7), \
                 acc[I][J], CB, BL, 1, F.sb[J], 1, F.sa[I]); } } while (0)
#define MXL_PIN __builtin_amdgcn_sched_barrier(0)
    // fragment (+ scale byte) reads of the K step in ring slot at `sn`, panel bytes at `pan`
#define MXL_RD_A(F, I) \
    do { if ((I) < LIVE) { const uint8_t* r_ = sn + a_frag + (I) * (32 * BK); \
         const uint4 lo_ = *(const uint4*)(r_ + a_lo), hi_ = *(const uint4*)(r_ + a_hi); \
         F.a[I][0] = lo_.x; F.a[I][1] = lo_.y; F.a[I][2] = lo_.z; F.a[I][3] = lo_.w; \
         F.a[I][4] = hi_.x; F.a[I][5] = hi_.y; F.a[I][6] = hi_.z; F.a[I][7] = hi_.w; } } while (0)
#define MXL_RD_B(F, J) \
    do { const uint8_t* r_ = sn + A_BYTES + b_frag + (J) * (32 * B_ROW); \
         if (BT && F44) { \
             _Pragma("unroll") for (int q_ = 0; q_ < 2; ++q_) _Pragma("unroll") for (int h_ = 0; h_ < 2; ++h_) { \
                 const v2i v_ = __builtin_amdgcn_ds_read_tr4_b64_v2i32( \
                     (__attribute__((address_space(3))) v2i*)((uint8_t*)sn + A_BYTES + (2 * wn + q_) * 4096 + (bt4_off[h_] ^ (16 * (J))))); \
                 F.b[J][4 * q_ + 2 * h_] = v_[0]; F.b[J][4 * q_ + 2 * h_ + 1] = v_[1]; } \
         } else if (BT) { \
             uint8_t* t_ = (uint8_t*)sn + A_BYTES + (2 * wn + ((J) >> 1)) * 4096; \
             _Pragma("unroll") for (int q_ = 0; q_ < 2; ++q_) _Pragma("unroll") for (int h_ = 0; h_ < 2; ++h_) { \
                 const v2i v_ = __builtin_amdgcn_ds_read_tr8_b64_v2i32( \
                     (__attribute__((address_space(3))) v2i*)(t_ + 2048 * q_ + bt_off[h_][(J) & 1])); \
                 F.b[J][4 * q_ + 2 * h_] = v_[0]; F.b[J][4 * q_ + 2 * h_ + 1] = v_[1]; } \
         } else if (B4) { \
             const uint4 lo_ = *(const uint4*)(r_ + b4_lo); \
             F.b[J][0] = lo_.x; F.b[J][1] = lo_.y; F.b[J][2] = lo_.z; F.b[J][3] = lo_.w; \
             F.b[J][4] = 0; F.b[J][5] = 0; F.b[J][6] = 0; F.b[J][7] = 0; \
         } else { \
             const uint4 lo_ = *(const uint4*)(r_ + a_lo), hi_ = *(const uint4*)(r_ + a_hi); \
             F.b[J][0] = lo_.x; F.b[J][1] = lo_.y; F.b[J][2] = lo_.z; F.b[J][3] = lo_.w; \
             F.b[J][4] = hi_.x; F.b[J][5] = hi_.y; F.b[J][6] = hi_.z; F.b[J][7] = hi_.w; \
         } } while (0)
    // the scale byte of step `psh / 8` of the panel, for fragment I of A / J of B (one shift each; they are spread
    // over the second half of a step's MFMAs so that the panel reads have long landed)
#define MXL_SC_A(F, I) do { F.sa[I] = ALPHA ? 127 : (int)(uint32_t)(psa[I] >> psh); } while (0)
#define MXL_SC_B(F, J) do { F.sb[J] = ALPHA ? 127 : (int)(uint32_t)(psb[J] >> psh); } while (0)
    // per-lane constants of the fragment reads: 64-byte rows, piece index XOR (row / 4) % 4
    const int sw = (lr >> 2) & 3;
    const int a_frag = (wm * 128 + lr) * BK, b_frag = (wn * 128 + lr) * B_ROW;
    const int b4_lo = 16 * (g ^ ((lr >> 3) & 1));      // FP4: lane (row, g) holds elements 32 g .. 32 g + 31 of the K step
    // BT: this lane ADDRESSES contraction row 16 g + 8 h + tj (+ 32 for the second half of the step) and the 8-byte
    // piece of its 16-lane block's 16 columns: bt_off[h][J & 1] inside a plane's 64 rows x 64 bytes (same swizzle
    // as the loads: 16-byte piece XOR (row / 4) % 4)
    // BT, E2M1 x E2M1 (ds_read_b64_tr_b4: in a block of 16 lanes, lane i receives nibble i of the 8-byte pieces
    // addressed by lanes 0 .. 15, in this order): this lane ADDRESSES contraction row 32 g + 16 h + l % 16 of a round's
    // 64 rows and the 8-byte half (l / 16) % 2 of a fragment's 16 bytes; fragment J is 16-byte piece J of the 64-byte
    // row, XOR (row / 4) % 4 as the loads placed it -- the XOR with 16 J is applied at the read.
    int bt4_off[2] = {0, 0};
    if (BT && F44) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = 32 * g + 16 * h + (l & 15);
            bt4_off[h] = row * 64 + 16 * ((row >> 2) & 3) + 8 * ((l >> 4) & 1);
        }
    }
    int bt_off[2][2];
    if (BT && !F44) {
        const int tj = (l & 15) >> 1, ta = l & 1, tblk = (l >> 4) & 1;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int row = 16 * g + 8 * h + tj, cb = 32 * jj + 16 * tblk + 8 * ta;
                bt_off[h][jj] = row * 64 + 16 * ((cb >> 4) ^ ((row >> 2) & 3)) + (cb & 15);
            }
    }
    const int a_lo = 16 * (g ^ sw), a_hi = 16 * ((2 + g) ^ sw);
    // Scale bytes: a panel row holds [g][K step] = 2 x 8 bytes, so the 8 bytes at (row, g) are the lane's scale
    // bytes of the panel's 8 K steps.  They are read once per panel (8 reads of 8 bytes per wave, 512 consecutive
    // bytes each) and the byte of a step is shifted down in registers: the MFMA takes byte 0 of its scale operand.
    const int a_sc = (wm * 128 + lr) * 16 + 8 * g, b_sc = (wn * 128 + lr) * 16 + 8 * g;
    uint64_t psa[4], psb[4];
#define MXL_RD_PANEL(PAN) \
    do { if (!ALPHA) _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) { \
             psa[i_] = *(const uint64_t*)((PAN) + a_sc + i_ * (32 * 16)); \
             psb[i_] = *(const uint64_t*)((PAN) + PANEL + b_sc + i_ * (32 * 16)); } } while (0)

    // The workgroup's tiles: one per round of nwg tiles, at position vwg of the round -- in wgrad at position
    // nwg - 1 - vwg in odd rounds (the serpentine; an XCD's workgroups still hold a contiguous run of the order).
    // A tile whose contraction range is empty (wgrad of a group without tokens) never enters the pipeline: its
    // output is zero-filled on the spot and the sequence moves on.
    auto tile_at = [&](int round) __attribute__((always_inline)) {
        return round * nwg + ((MODE == MODE_WGRAD && (round & 1)) ? nwg - 1 - vwg : vwg);
    };
    int round = 0;
    auto next_tile = [&]() __attribute__((always_inline)) {
        int tl = tile_at(round);
        if (MODE == MODE_WGRAD) {
            while (tl < total_tiles) {
                const int pos = tl / (tiles_m * tiles_n);
                const int grp = __builtin_amdgcn_readfirstlane(by_len[pos]);
                if (__builtin_amdgcn_readfirstlane((int)(pre_rows[grp + 1] > pre_rows[grp]))) break;   // uniform by construction
                const int rem = tl - pos * tiles_m * tiles_n;
                const int width = GROUP_M * tiles_n;
                const int first = (rem / width) * GROUP_M;
                const int gsz = (tiles_m - first) < GROUP_M ? (tiles_m - first) : GROUP_M;
                const int64_t row0 = (int64_t)(first + (rem % width) % gsz) * BM, col0 = (int64_t)((rem % width) / gsz) * BN;
                if (!ACCUM) {    // (nothing to add for a group without tokens)
                    uint16_t* ct = p.c + ((int64_t)grp * p.m + row0) * p.n + col0;
                    const int mv = (p.m - row0) < BM ? (int)(p.m - row0) : BM, nv = (p.n - col0) < BN ? (int)(p.n - col0) : BN;
                    for (int r = t >> 5; r < mv; r += GTHREADS / 32) {
                        const int c = (t & 31) * 8;
                        if (c < nv) store16_streaming((uint8_t*)(ct + (int64_t)r * p.n + c), make_uint4(0u, 0u, 0u, 0u));
                    }
                }
                tl = tile_at(++round);
            }
        }
        ++round;
        return __builtin_amdgcn_readfirstlane(tl);
    };
    int tile = next_tile();
    if (tile >= total_tiles) return;
    int tile_n = next_tile();
    Tile d = decode(tile);
    // past the last tile the stream requests the last tile's first steps again (nobody reads them)
    Tile dn = decode(tile_n < total_tiles ? tile_n : tile);
    int gs = 0;          // K steps run so far by this workgroup (ring slot of a step = its number & 3)
    int pb_rd = 0;       // panel buffer of the scales being read
    int pb_is = 0;       // panel buffer of the most recent panel request
    // prologue: panel 0 and K steps 0, 1, 2 of the first tile, and the first six rounds of step 3
    stream_enter(d);
    issue_s(d, 0, 0);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        group_begin();
        static_for<0, ROUNDS>([&](auto e) { issue_e(e, wave_base + (uint32_t)(s * STAGE)); });
    }
    group_begin();
    static_for<0, 6>([&](auto e) { issue_e(e, wave_base + (uint32_t)(3 * STAGE)); });
    wait_vm<2 * ROUNDS + 6>();       // everything up to K step 0 has landed
    __syncthreads();

    while (true) {
        v16f acc[4][4];
        Frags f0, f1;
        const int nst = d.nst, nst_real = d.nst_real;
        // LIVE: how many of the wave's four 32-row fragments hold rows of the tile (4, 2 or 0).  A tile at the ragged end of
        // a group has fewer than 256 rows; fragments beyond them are neither read nor multiplied (loads, barriers and the
        // request stream are the same for every wave).
        auto run_tile = [&](auto live_tag) __attribute__((always_inline)) {
            constexpr int LIVE = decltype(live_tag)::value;
            {   // fragments of K step 0
                const uint8_t* sn = smem + (gs & 3) * STAGE;
                MXL_RD_PANEL(panels + pb_rd * 2 * PANEL);
                const int psh = 0;
                MXL_RD_B(f0, 0); MXL_RD_B(f0, 1); MXL_RD_B(f0, 2); MXL_RD_B(f0, 3);
                MXL_RD_A(f0, 0); MXL_RD_A(f0, 1); MXL_RD_A(f0, 2); MXL_RD_A(f0, 3);
                MXL_PIN;
                // the accumulators are cleared while those reads are on their way
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
                MXL_PIN;
                MXL_SC_B(f0, 0); MXL_SC_B(f0, 1); MXL_SC_B(f0, 2); MXL_SC_B(f0, 3);
                MXL_SC_A(f0, 0); MXL_SC_A(f0, 1); MXL_SC_A(f0, 2); MXL_SC_A(f0, 3);
            }
            // One K step s (local number, parity PAR) of 16 MFMAs.  MF: multiply (false for the padding steps of a
            // tile whose contraction range is shorter than four steps).  LAST: the tile's last step; the six rounds
            // that would go into the slot the epilogue is about to use are issued after the epilogue instead.
            using E0 = std::integral_constant<int, 0>; using E1 = std::integral_constant<int, 1>;
            using E2 = std::integral_constant<int, 2>; using E3 = std::integral_constant<int, 3>;
            using E4 = std::integral_constant<int, 4>; using E5 = std::integral_constant<int, 5>;
            using E6 = std::integral_constant<int, 6>; using E7 = std::integral_constant<int, 7>;
            auto kstep = [&](auto par_tag, auto mf_tag, auto last_tag, int s, Frags& cur, Frags& nxt) __attribute__((always_inline)) {
                constexpr int PAR = decltype(par_tag)::value;
                constexpr bool MF = decltype(mf_tag)::value;
                constexpr bool LAST = decltype(last_tag)::value;
                const uint32_t slot_prev = wave_base + (uint32_t)(((gs + 3) & 3) * STAGE);   // group of step gs + 3
                const uint32_t slot_new = wave_base + (uint32_t)((gs & 3) * STAGE);          // group of step gs + 4
                MXL_MFMA(cur, 0, 0); if (ROUNDS == 8) issue_e(E6{}, slot_prev); MXL_PIN;
                MXL_MFMA(cur, 1, 0); MXL_PIN;
                MXL_MFMA(cur, 2, 0); if (ROUNDS == 8) issue_e(E7{}, slot_prev); MXL_PIN;
                MXL_MFMA(cur, 3, 0); MXL_PIN;
                wait_vm<2 * ROUNDS>();       // the group of step gs + 1 has landed (two younger groups may be in flight)
                __syncthreads();
                MXL_PIN;
                // bookkeeping between the barrier and the first read: panel of the next step, stream hand-over
                const int s1 = s + 1;
                if ((s1 & (PSTEPS - 1)) == 0 && s1 < nst) {
                    pb_rd = next3(pb_rd);
                    MXL_RD_PANEL(panels + pb_rd * 2 * PANEL);
                }
                if (!LAST) group_begin();
                const uint8_t* sn = smem + ((gs + 1) & 3) * STAGE;
                const int psh = (64 / PSTEPS) * (s1 & (PSTEPS - 1));   // FP4 rows: a step owns two bytes, the MFMAs pick with op_sel
                MXL_PIN;
                MXL_RD_B(nxt, 0); MXL_MFMA(cur, 0, 1);  if (!LAST) issue_e(E0{}, slot_new); MXL_PIN;
                MXL_RD_A(nxt, 0); MXL_MFMA(cur, 1, 1);  MXL_PIN;
                MXL_RD_A(nxt, 1); MXL_MFMA(cur, 2, 1);  if (!LAST) issue_e(E1{}, slot_new); MXL_PIN;
                MXL_RD_A(nxt, 2); MXL_MFMA(cur, 3, 1);  MXL_PIN;
                MXL_RD_A(nxt, 3); MXL_MFMA(cur, 0, 2);  if (!LAST) issue_e(E2{}, slot_new); MXL_PIN;
                MXL_RD_B(nxt, 1); MXL_MFMA(cur, 1, 2);  MXL_SC_B(nxt, 0); MXL_PIN;
                MXL_RD_B(nxt, 2); MXL_MFMA(cur, 2, 2);  if (!LAST) issue_e(E3{}, slot_new); MXL_SC_A(nxt, 0); MXL_PIN;
                MXL_RD_B(nxt, 3); MXL_MFMA(cur, 3, 2);  MXL_SC_A(nxt, 1); MXL_PIN;
                MXL_MFMA(cur, 0, 3); if (!LAST) issue_e(E4{}, slot_new); MXL_SC_A(nxt, 2); MXL_PIN;
                MXL_MFMA(cur, 1, 3); MXL_SC_A(nxt, 3); MXL_SC_B(nxt, 1); MXL_PIN;
                MXL_MFMA(cur, 2, 3); if (!LAST) issue_e(E5{}, slot_new); MXL_SC_B(nxt, 2); MXL_PIN;
                MXL_MFMA(cur, 3, 3); MXL_SC_B(nxt, 3); MXL_PIN;
                ++gs;
            };
            using P0 = std::integral_constant<int, 0>;
            using P1 = std::integral_constant<int, 1>;
            using Yes = std::integral_constant<bool, true>;
            using No = std::integral_constant<bool, false>;
            if (nst_real >= 3) {
                for (int s = 0; s < nst - 2; s += 2) {
                    if (s == nst - 4) {
                        // the request stream moves on to the workgroup's next tile: its scale panel 0 first
                        pb_is = next3(pb_is);
                        issue_s(dn, 0, pb_is);
                        stream_enter(dn);
                    } else if ((s & (PSTEPS - 1)) == PSTEPS - 4 && s + 4 < nst) {
                        // this tile's next scale panel (K steps s + 4 ...): first read three barriers from here
                        pb_is = next3(pb_is);
                        issue_s(d, (s + 4) / PSTEPS, pb_is);
                    }
                    kstep(P0{}, Yes{}, No{}, s, f0, f1);
                    kstep(P1{}, Yes{}, No{}, s + 1, f1, f0);
                }
                kstep(P0{}, Yes{}, No{}, nst - 2, f0, f1);
                if (!F44 || nst_real == nst) kstep(P1{}, Yes{}, Yes{}, nst - 1, f1, f0);
                else kstep(P1{}, No{}, Yes{}, nst - 1, f1, f0);          // an odd range: the padding step does not multiply
            } else {
                // a contraction range of one or two steps: four steps run, the others without multiplying
                pb_is = next3(pb_is);
                issue_s(dn, 0, pb_is);
                stream_enter(dn);
                kstep(P0{}, Yes{}, No{}, 0, f0, f1);
                if (!F44 || nst_real == 2) kstep(P1{}, Yes{}, No{}, 1, f1, f0);
                else kstep(P1{}, No{}, No{}, 1, f1, f0);
                kstep(P0{}, No{}, No{}, 2, f0, f1);
                kstep(P1{}, No{}, Yes{}, 3, f1, f0);
            }
        };
        {
            const int live = (MODE == MODE_FWD) ? d.m_valid - wm * 128 : 128;
            if (MODE != MODE_FWD || live > 64) run_tile(std::integral_constant<int, 4>{});
            else if (live > 0) run_tile(std::integral_constant<int, 2>{});
            else run_tile(std::integral_constant<int, 0>{});
        }
        // K step 0 of the next tile (and its scale panel) has landed; every wave is done reading the ring
        wait_vm<2 * ROUNDS>();
        __syncthreads();
        MXL_PIN;

        // ---- epilogue: fp32 -> bf16 through a wave-private LDS patch of 32 rows x 128 bytes in the ring slot of
        // the step that has just finished, so that the global stores are 16 bytes per lane, 8 rows x 128
        // contiguous bytes per instruction.  The patch is not padded (the four patches fill half a slot);
        // 16-byte pieces are XOR-swizzled by (row / 2) % 8 and the 8-byte halves swapped in rows 16-31:
        // conflict-free for the 8-byte writes (a lane owns a row) and the 16-byte reads (8 lanes per row).
        // The lane's offsets into the patch and into the output tile are rebuilt here from the lane number, taken afresh
        // from the hardware: computed once in front of the tile loop they would have to live through the main loop, where
        // every register is taken, and would come back from scratch memory one dependent load after the other, each of
        // them waiting for all operand requests in flight (measured: 5 of the epilogue's 6.5 us).
        {
            uint32_t z = 0;    // a zero the optimiser cannot see through: the count must not be hoisted out of the tile loop
            asm volatile("" : "+v"(z));
            const int lo = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
            const int elr = lo & 31, eg = lo >> 5;
            const int m_valid = d.m_valid, n_valid = d.n_valid;
            uint16_t* ctile = p.c + ((int64_t)d.c_row0 * p.n + d.c_col0);
            uint8_t* stg = smem + ((gs + 3) & 3) * STAGE + w * (32 * 128);
            uint8_t* wr = stg + elr * 128 + 8 * (eg ^ (elr >> 4));
            const int wsw = (elr >> 1) & 7;
            const int rrow = lo >> 3, rch = lo & 7;
            // rows 8u + rrow: (row / 2) % 8 = (4 (u & 1) + rrow / 2) % 8
            const uint8_t* rd0 = stg + rrow * 128 + 16 * (rch ^ (rrow >> 1));
            const uint8_t* rd1 = stg + rrow * 128 + 16 * (rch ^ (4 + (rrow >> 1)));
            const uint32_t lane_off = (uint32_t)((rrow * (int)p.n + rch * 8) * 2);   // bytes from the row base
            const bool full = (m_valid == BM) && (n_valid == BN);
            float alpha = 1.f;
            if (ALPHA) alpha = *p.alpha_a * *p.alpha_b;
            // Eight patches (32 rows x 64 columns each) go through the staging area one after the other.  The LDS runs
            // a wave's accesses in order, so patch n + 1 may be written as soon as the reads of patch n have been ISSUED:
            // the stores of patch n, which wait for those reads, come behind the conversions and writes of patch n + 1
            // and find their data there.  The loop exists twice, for whole tiles (nothing predicated) and for tiles at
            // an edge.
            auto write_out = [&](auto full_tag) __attribute__((always_inline)) {
                constexpr bool FULL = decltype(full_tag)::value;
                uint4 v[4];
                static_for<0, 9>([&](auto it_tag) {
                    constexpr int it = decltype(it_tag)::value;
                    if constexpr (it < 8) {
                        constexpr int i = it >> 1, jh = it & 1;
#pragma unroll
                        for (int jl = 0; jl < 2; ++jl)
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const int j = 2 * jh + jl;
                                if (ALPHA) {
#pragma unroll
                                    for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] *= alpha;
                                }
                                v4bf o = {(__bf16)acc[i][j][4 * q], (__bf16)acc[i][j][4 * q + 1], (__bf16)acc[i][j][4 * q + 2],
                                          (__bf16)acc[i][j][4 * q + 3]};
                                *(v4bf*)(wr + 16 * ((4 * jl + q) ^ wsw)) = o;
                            }
                    }
                    if constexpr (it > 0) {
                        constexpr int i = (it - 1) >> 1, jh = (it - 1) & 1;
                        // uniform base of the patch's rows; the lane adds a 32-bit offset
                        uint8_t* rowbase = (uint8_t*)(ctile + (int64_t)(wm * 128 + i * 32) * p.n + wn * 128 + jh * 64);
                        const int cc = wn * 128 + jh * 64 + rch * 8;
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            if (FULL || (wm * 128 + i * 32 + 8 * u + rrow < m_valid && cc < n_valid))
                                store16_streaming(rowbase + (int64_t)(8 * u) * p.n * 2 + lane_off,
                                                  u >= 2 ? make_uint4(v[u].z, v[u].w, v[u].x, v[u].y) : v[u]);
                    }
                    if constexpr (it < 8) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] = *(const uint4*)(((u & 1) ? rd1 : rd0) + u * (8 * 128));
                    }
                    MXL_PIN;
                });
            };
            // ACCUM: the same staging with float32 patches of 32 rows x 32 columns (sixteen per wave; 16-byte pieces
            // XOR-swizzled by (row / 2) % 8), read back one word per lane -- two whole output rows of the patch per
            // instruction -- and added to the buffer with float atomics that return nothing: the L2 does the
            // read-modify-write, the wave waits for no old value.  Every output element belongs to one workgroup and gets
            // exactly one add per launch.
            auto add_out = [&](auto full_tag) __attribute__((always_inline)) {
                constexpr bool FULL = decltype(full_tag)::value;
                float* ctile32 = (float*)p.c + ((int64_t)d.c_row0 * p.n + d.c_col0);
                uint8_t* wr32 = stg + elr * 128;
                const int wsw32 = (elr >> 1) & 7;
                const int rw = lo & 31, rr2 = lo >> 5;                         // word of the row, row parity while reading
                const uint8_t* rd32 = stg + rr2 * 128 + 4 * (rw & 3);
                const uint32_t lane_off32 = (uint32_t)(rr2 * (int)p.n + rw);  // elements from a patch's first one
                float val[16];
                static_for<0, 17>([&](auto it_tag) {
                    constexpr int it = decltype(it_tag)::value;
                    if constexpr (it < 16) {
                        constexpr int i = it >> 2, j = it & 3;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            v4f o = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                            if (ALPHA) o *= alpha;
                            *(v4f*)(wr32 + 16 * ((2 * q + eg) ^ wsw32)) = o;
                        }
                    }
                    if constexpr (it > 0) {
                        constexpr int i = (it - 1) >> 2, j = (it - 1) & 3;
                        float* base = ctile32 + (int64_t)(wm * 128 + i * 32) * p.n + wn * 128 + j * 32;   // uniform
                        const bool col_ok = FULL || wn * 128 + j * 32 + rw < n_valid;
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (FULL || (col_ok && wm * 128 + i * 32 + 2 * v + rr2 < m_valid))
                                unsafeAtomicAdd(base + (int64_t)(2 * v) * p.n + lane_off32, val[v]);
                    }
                    if constexpr (it < 16) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)    // row 2 v + rr2: its swizzle is v % 8
                            val[v] = *(const float*)(rd32 + v * 256 + 16 * ((rw >> 2) ^ (v & 7)));
                    }
                    MXL_PIN;
                });
            };
            if constexpr (ACCUM) {
                if (full) add_out(std::true_type{});
                else add_out(std::false_type{});
            } else {
                if (full) write_out(std::true_type{});
                else write_out(std::false_type{});
            }
        }
        if (tile_n >= total_tiles) break;
        __syncthreads();      // every wave has left the patch: its slot takes K step 3 of the next tile
        // (the stream entered the next tile four steps ago; the group of its step 3 begins here)
        group_begin();
        {
            const uint32_t slot_new = wave_base + (uint32_t)(((gs + 3) & 3) * STAGE);
            static_for<0, 6>([&](auto e) { issue_e(e, slot_new); });
        }
        d = dn;
        tile = tile_n;
        tile_n = next_tile();
        dn = decode(tile_n < total_tiles ? tile_n : tile);
        pb_rd = next3(pb_rd);
        MXL_PIN;
    }
    wait_vm<0>();   // nothing may still be writing this workgroup's LDS when it ends
#undef MXL_MFMA
#undef MXL_PIN
#undef MXL_RD_A
#undef MXL_RD_B
#undef MXL_RD_PANEL
#undef MXL_SC_A
#undef MXL_SC_B
}

constexpr int gemm_lds_bytes(int afmt, int bfmt) {
    return NSLOT * (256 * (afmt == kFmtE2M1 ? BKP / 2 : BKP) + 256 * (bfmt == kFmtE2M1 ? BKP / 2 : BKP)) + 4 * 256 * 16 +
           (MXL_MAX_GROUPS + 2) * 4 + (MXL_MAX_GROUPS + 2) * 8;
}

// Per-device caches are indexed by the device ordinal (64 slots; a process with more devices shares slots,
// which only costs a repeated query).
static int current_device_slot() {
    int dev = 0;
    return hipGetDevice(&dev) == hipSuccess ? (dev & 63) : 0;
}

static int num_cus(int slot) {
    static std::atomic<int> cached[64];
    int v = cached[slot].load(std::memory_order_relaxed);
    if (v) return v;
    int dev = 0;
    hipDeviceProp_t pr;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&pr, dev) != hipSuccess) return 256;
    cached[slot].store(pr.multiProcessorCount, std::memory_order_relaxed);
    return pr.multiProcessorCount;
}

template <int AFMT, int BFMT, int MODE, int LAYOUT, bool ALPHA = false, bool ACCUM = false, bool BSHUF = false>
static int launch_gemm(const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    constexpr int lds = gemm_lds_bytes(AFMT, BFMT);
    if (!device_is_gfx950()) return MXL_ENODEV;
    static std::atomic<bool> attr_set[64];   // the attribute belongs to the (kernel, device) pair
    const int slot = current_device_slot();
    auto kern = mx_gemm_kernel<AFMT, BFMT, MODE, LAYOUT, ALPHA, ACCUM, BSHUF>;
    if (!attr_set[slot].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return MXL_ELAUNCH;
        attr_set[slot].store(true, std::memory_order_release);
    }
    int64_t grid = num_cus(slot);
    if (max_tiles < grid) grid = max_tiles;
    if (grid <= 0) return MXL_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(GTHREADS), lds, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

template <int AFMT, int BFMT, int MODE, bool ALPHA, bool ACCUM = false, bool BT = false>
static int launch_gemm_ring(const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    constexpr int lds = ring_lds_bytes();
    if (!device_is_gfx950()) return MXL_ENODEV;
    static std::atomic<bool> attr_set[64];
    const int slot = current_device_slot();
    auto kern = mx_gemm_ring_kernel<AFMT, BFMT, MODE, ALPHA, ACCUM, BT>;
    if (!attr_set[slot].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return MXL_ELAUNCH;
        attr_set[slot].store(true, std::memory_order_release);
    }
    int64_t grid = num_cus(slot);
    if (max_tiles < grid) grid = max_tiles;
    if (grid <= 0) return MXL_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(GTHREADS), lds, st, a);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

// The 4-slot ring kernel serves operands in the K-step-major layout with at most RING_MAX_GROUPS groups: FP8 x FP8,
// and FP8 rows against an FP4 weight operand in the forward / dgrad GEMM.
template <int MODE>
static bool ring_serves(int afmt, int bfmt, const GemmArgs& a) {
    if (a.num_groups > RING_MAX_GROUPS) return false;
    if (a.alpha_a != nullptr)    // per-tensor factors: E4M3 or E5M2 rows against E4M3, and E5M2 against E5M2
        return (bfmt == MXL_FMT_E4M3 && (afmt == MXL_FMT_E4M3 || afmt == MXL_FMT_E5M2)) || (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E5M2);
    // MX: E4M3 x E4M3, in the forward / dgrad GEMM E4M3 activations against E2M1 weights, and E2M1 x E2M1
    if (afmt == MXL_FMT_E2M1) return bfmt == MXL_FMT_E2M1;
    return afmt == MXL_FMT_E4M3 && (bfmt == MXL_FMT_E4M3 || (bfmt == MXL_FMT_E2M1 && MODE == MODE_FWD));
}
template <int MODE>
static int dispatch_gemm_ring(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    if (a.alpha_a != nullptr) {
        if (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E5M2) return launch_gemm_ring<MXL_FMT_E5M2, MXL_FMT_E5M2, MODE, true>(a, max_tiles, st);
        if (afmt == MXL_FMT_E5M2) return launch_gemm_ring<MXL_FMT_E5M2, MXL_FMT_E4M3, MODE, true>(a, max_tiles, st);
        return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE, true>(a, max_tiles, st);
    }
    if (afmt == MXL_FMT_E2M1) return launch_gemm_ring<MXL_FMT_E2M1, MXL_FMT_E2M1, MODE, false>(a, max_tiles, st);
    if constexpr (MODE == MODE_FWD) {
        if (bfmt == MXL_FMT_E2M1) return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E2M1, MODE_FWD, false>(a, max_tiles, st);
    }
    return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE, false>(a, max_tiles, st);
}

template <int MODE, int LAYOUT>
static int dispatch_gemm_l(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE, LAYOUT>(a, max_tiles, st);
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E2M1, MODE, LAYOUT>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E4M3, MODE, LAYOUT>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E2M1, MODE, LAYOUT>(a, max_tiles, st);
    return MXL_EINVAL;
}

// tensor-wise scaled operands: E4M3 x E4M3 (forward, or every GEMM of the E4M3 format), E5M2 x E4M3 (gradient
// times weight / activation of the HYBRID format) and E5M2 x E5M2 (the FP8 backward of the MXFP4 linear, which
// re-quantises all three tensors to the gradient format); output times *alpha_a * *alpha_b
template <int MODE, int LAYOUT>
static int dispatch_gemm_alpha_l(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3)
        return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE, LAYOUT, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E4M3)
        return launch_gemm<MXL_FMT_E5M2, MXL_FMT_E4M3, MODE, LAYOUT, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E5M2)
        return launch_gemm<MXL_FMT_E5M2, MXL_FMT_E5M2, MODE, LAYOUT, true>(a, max_tiles, st);
    return MXL_EINVAL;
}

// wgrad accumulated into a float32 buffer: K-chunk-major operands only
static int dispatch_wgrad_accum(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    constexpr int W = MODE_WGRAD;
    if (a.alpha_a != nullptr) {
        if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E4M3, W, 1, true, true>(a, max_tiles, st);
        if (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E5M2, MXL_FMT_E4M3, W, 1, true, true>(a, max_tiles, st);
        return MXL_EINVAL;
    }
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E4M3, W, 1, false, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E4M3, MXL_FMT_E2M1, W, 1, false, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E4M3) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E4M3, W, 1, false, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E2M1) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E2M1, W, 1, false, true>(a, max_tiles, st);
    return MXL_EINVAL;
}

// the weight-gradient GEMM that adds into a float32 buffer, on K-step-major operands
static int dispatch_wgrad_accum_ring(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    constexpr int W = MODE_WGRAD;
    if (a.alpha_a != nullptr) {
        if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, W, true, true>(a, max_tiles, st);
        if (afmt == MXL_FMT_E5M2 && bfmt == MXL_FMT_E4M3) return launch_gemm_ring<MXL_FMT_E5M2, MXL_FMT_E4M3, W, true, true>(a, max_tiles, st);
        return MXL_EINVAL;
    }
    if (afmt == MXL_FMT_E4M3 && bfmt == MXL_FMT_E4M3) return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, W, false, true>(a, max_tiles, st);
    if (afmt == MXL_FMT_E2M1 && bfmt == MXL_FMT_E2M1) return launch_gemm_ring<MXL_FMT_E2M1, MXL_FMT_E2M1, W, false, true>(a, max_tiles, st);
    return MXL_EINVAL;
}

// forward / dgrad on the row-wise codes of the transposed weight (MXL_GF_B_TRANSPOSED): E4M3 weights with E4M3 or E5M2
// rows, or E2M1 weights with E2M1 rows (128-element steps)
static int dispatch_gemm_ring_bt(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, hipStream_t st) {
    if (a.num_groups > RING_MAX_GROUPS) return MXL_EINVAL;
    if (bfmt == MXL_FMT_E2M1) {
        if (afmt != MXL_FMT_E2M1 || a.alpha_a != nullptr) return MXL_EINVAL;
        return launch_gemm_ring<MXL_FMT_E2M1, MXL_FMT_E2M1, MODE_FWD, false, false, true>(a, max_tiles, st);
    }
    if (bfmt != MXL_FMT_E4M3) return MXL_EINVAL;
    if (a.alpha_a != nullptr) {
        if (afmt == MXL_FMT_E5M2) return launch_gemm_ring<MXL_FMT_E5M2, MXL_FMT_E4M3, MODE_FWD, true, false, true>(a, max_tiles, st);
        if (afmt == MXL_FMT_E4M3) return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE_FWD, true, false, true>(a, max_tiles, st);
        return MXL_EINVAL;
    }
    if (afmt != MXL_FMT_E4M3) return MXL_EINVAL;
    return launch_gemm_ring<MXL_FMT_E4M3, MXL_FMT_E4M3, MODE_FWD, false, false, true>(a, max_tiles, st);
}

// a_rows / b_rows: rows of the whole operands (for the 4 GiB bound of the chunk-major layout)
// layout: 0 row-major codes, 1 K-chunk-major codes, 2 K-step-major codes and scales
template <int MODE>
static int dispatch_gemm(int afmt, int bfmt, const GemmArgs& a, int64_t max_tiles, int layout, int64_t a_rows, int64_t b_rows,
                         hipStream_t st, bool accum = false) {
    const bool kchunk = layout == 1;
    if (layout == 2) {
        if ((accum && MODE != MODE_WGRAD) || !ring_serves<MODE>(afmt, bfmt, a)) return MXL_EINVAL;
        // offsets inside an operand are 32-bit
        if (a_rows * a.k >= ((int64_t)1 << 32) || b_rows * a.k >= ((int64_t)1 << 32)) return MXL_EINVAL;
        // the kernel keeps a tile's first output row in 32 bits
        if ((MODE == MODE_WGRAD ? (int64_t)a.num_groups * a.m : a.total_m) >= ((int64_t)1 << 31)) return MXL_EINVAL;
        if (accum) return dispatch_wgrad_accum_ring(afmt, bfmt, a, max_tiles, st);
        return dispatch_gemm_ring<MODE>(afmt, bfmt, a, max_tiles, st);
    }
    if (accum) {
        if (MODE != MODE_WGRAD || !kchunk) return MXL_EINVAL;
        if (a_rows * a.k >= ((int64_t)1 << 32) || b_rows * a.k >= ((int64_t)1 << 32)) return MXL_EINVAL;
        return dispatch_wgrad_accum(afmt, bfmt, a, max_tiles, st);
    }
    const bool alpha = a.alpha_a != nullptr;
    if (!kchunk) return alpha ? dispatch_gemm_alpha_l<MODE, 0>(afmt, bfmt, a, max_tiles, st)
                              : dispatch_gemm_l<MODE, 0>(afmt, bfmt, a, max_tiles, st);
    // chunk offsets inside an operand are 32-bit
    if (a_rows * a.k >= ((int64_t)1 << 32) || b_rows * a.k >= ((int64_t)1 << 32)) return MXL_EINVAL;
    return alpha ? dispatch_gemm_alpha_l<MODE, 1>(afmt, bfmt, a, max_tiles, st)
                 : dispatch_gemm_l<MODE, 1>(afmt, bfmt, a, max_tiles, st);
}

}  // namespace mxl

using namespace mxl;

// Offsets inside a tile's operand rows (up to 256 rows of the contraction length) are 32-bit.
constexpr int64_t MAX_CONTRACTION = (int64_t)1 << 23;

__global__ __launch_bounds__(256) void zero_fill_kernel(uint32_t* dst, int64_t words) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < words) dst[i] = 0u;
}

static int grouped_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes, const void* b_scales,
                           int b_fmt, void* c_bf16, const int64_t* group_lens, int num_groups, int64_t total_m, int64_t n,
                           int64_t k, const float* alpha_a, const float* alpha_b, uint32_t flags, void* stream) {
    if (flags & ~(uint32_t)(MXL_GF_KCHUNK | MXL_GF_KSTEP | MXL_GF_B_TRANSPOSED | MXL_GF_B_SHUFFLED)) return MXL_EINVAL;
    if ((flags & MXL_GF_KCHUNK) && (flags & MXL_GF_KSTEP)) return MXL_EINVAL;
    // pre-shuffled weight codes: row-major E2M1 x E2M1, block scales, whole 16-row blocks per group
    if ((flags & MXL_GF_B_SHUFFLED) && (flags != MXL_GF_B_SHUFFLED || a_fmt != MXL_FMT_E2M1 || b_fmt != MXL_FMT_E2M1 || alpha_a || n % 16 != 0))
        return MXL_EINVAL;
    if ((flags & MXL_GF_B_TRANSPOSED) && !(flags & MXL_GF_KSTEP)) return MXL_EINVAL;
    if ((alpha_a == nullptr) != (alpha_b == nullptr)) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % MXL_BLOCK != 0 || k % 128 != 0) return MXL_EINVAL;
    if (k > MAX_CONTRACTION) return MXL_EINVAL;   // tile-relative byte offsets are 32-bit
    if (num_groups < 1 || num_groups > MXL_MAX_GROUPS) return MXL_EINVAL;
    if (num_groups > 1 && !group_lens) return MXL_EINVAL;
    if (total_m == 0) return MXL_OK;   // no rows: nothing to read or write (the row operands may be null)
    if (!a_codes || !b_codes || !c_bf16) return MXL_EINVAL;
    if (alpha_a == nullptr && (!a_scales || !b_scales)) return MXL_EINVAL;   // block scales are read unless per-tensor factors are given
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
    a.alpha_a = alpha_a;
    a.alpha_b = alpha_b;
    const int64_t max_tiles = (total_m / BM + num_groups) * ((n + BN - 1) / BN);
    if (flags & MXL_GF_B_SHUFFLED) return launch_gemm<MXL_FMT_E2M1, MXL_FMT_E2M1, MODE_FWD, 0, false, false, true>(a, max_tiles, (hipStream_t)stream);
    if (flags & MXL_GF_B_TRANSPOSED) {
        // offsets inside an operand are 32-bit; the kernel keeps a tile's first output row in 32 bits
        const int64_t n_ld = (n + 127) / 128 * 128;
        if (total_m * k >= ((int64_t)1 << 32) || (int64_t)num_groups * k * n_ld >= ((int64_t)1 << 32) || total_m >= ((int64_t)1 << 31))
            return MXL_EINVAL;
        return dispatch_gemm_ring_bt(a_fmt, b_fmt, a, max_tiles, (hipStream_t)stream);
    }
    return dispatch_gemm<MODE_FWD>(a_fmt, b_fmt, a, max_tiles, (flags & MXL_GF_KSTEP) ? 2 : (flags & MXL_GF_KCHUNK) ? 1 : 0, total_m,
                                   (int64_t)num_groups * n, (hipStream_t)stream);
}

extern "C" int mxl_grouped_gemm_nt_ex(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                      const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                      int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags, void* stream) {
    return grouped_gemm_nt(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups, total_m, n, k,
                           nullptr, nullptr, flags, stream);
}

extern "C" int mxl_grouped_gemm_nt_scaled(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                          const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                          int num_groups, int64_t total_m, int64_t n, int64_t k, const float* alpha_a,
                                          const float* alpha_b, uint32_t flags, void* stream) {
    if (!alpha_a || !alpha_b) return MXL_EINVAL;
    return grouped_gemm_nt(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups, total_m, n, k,
                           alpha_a, alpha_b, flags, stream);
}

extern "C" int mxl_grouped_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                   const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                   int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    return mxl_grouped_gemm_nt_ex(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups, total_m,
                                  n, k, 0, stream);
}

extern "C" int mxl_gemm_nt(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                           const void* b_scales, int b_fmt, void* c_bf16, int64_t m, int64_t n, int64_t k,
                           void* stream) {
    return mxl_grouped_gemm_nt_ex(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, nullptr, 1, m, n, k, 0, stream);
}

static int grouped_gemm_wgrad(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                              const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens, int num_groups,
                              int64_t total_m, int64_t n, int64_t k, const float* alpha_a, const float* alpha_b,
                              uint32_t flags, void* stream) {
    if (flags & ~(uint32_t)(MXL_GF_KCHUNK | MXL_GF_KSTEP | MXL_GF_ACCUM_F32)) return MXL_EINVAL;
    if ((flags & MXL_GF_KCHUNK) && (flags & MXL_GF_KSTEP)) return MXL_EINVAL;
    const bool accum = (flags & MXL_GF_ACCUM_F32) != 0;
    if (accum && !(flags & (MXL_GF_KCHUNK | MXL_GF_KSTEP))) return MXL_EINVAL;
    if ((alpha_a == nullptr) != (alpha_b == nullptr)) return MXL_EINVAL;
    if (total_m < 0 || n <= 0 || k <= 0 || n % MXL_BLOCK != 0 || k % MXL_BLOCK != 0) return MXL_EINVAL;
    if (num_groups < 0 || num_groups > MXL_MAX_GROUPS) return MXL_EINVAL;
    if ((num_groups > 0) != (group_lens != nullptr)) return MXL_EINVAL;
    const int G = num_groups > 0 ? num_groups : 1;
    if (!c_bf16) return MXL_EINVAL;
    // a padded width of 0 (no tokens, one group) leaves nothing to read: the operands may be null and the
    // kernel only writes the zero gradient
    if (mxl_padded_width(total_m, G) > MAX_CONTRACTION) return MXL_EINVAL;
    const bool nothing_to_read = mxl_padded_width(total_m, G) == 0;
    if (nothing_to_read && accum) return MXL_OK;   // nothing to add
    if (nothing_to_read) {
        // The GEMM kernel requests the first K slot of every tile unconditionally, so it is never launched on
        // operands that do not exist; a fill kernel (not a memset, which callers could not capture in a graph)
        // writes the zero gradient.
        const int64_t words = (int64_t)G * n * k / 2;   // n and k are multiples of 32
        const int64_t grid = (words + 255) / 256;
        if (grid > 0x7FFFFFFF) return MXL_EINVAL;
        if (!device_is_gfx950()) return MXL_ENODEV;
        hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (uint32_t*)c_bf16,
                           words);
        return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
    }
    if (!a_codes || !b_codes) return MXL_EINVAL;
    if (alpha_a == nullptr && (!a_scales || !b_scales)) return MXL_EINVAL;   // block scales are read unless per-tensor factors are given
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
    a.alpha_a = alpha_a;
    a.alpha_b = alpha_b;
    const int64_t max_tiles = (int64_t)G * ((n + BM - 1) / BM) * ((k + BN - 1) / BN);
    return dispatch_gemm<MODE_WGRAD>(a_fmt, b_fmt, a, max_tiles, (flags & MXL_GF_KSTEP) ? 2 : (flags & MXL_GF_KCHUNK) ? 1 : 0, n, k,
                                     (hipStream_t)stream, accum);
}

extern "C" int mxl_grouped_gemm_wgrad_ex(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                         const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                         int num_groups, int64_t total_m, int64_t n, int64_t k, uint32_t flags,
                                         void* stream) {
    return grouped_gemm_wgrad(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups, total_m, n,
                              k, nullptr, nullptr, flags, stream);
}

extern "C" int mxl_grouped_gemm_wgrad_scaled(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                             const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                             int num_groups, int64_t total_m, int64_t n, int64_t k, const float* alpha_a,
                                             const float* alpha_b, uint32_t flags, void* stream) {
    if (!alpha_a || !alpha_b) return MXL_EINVAL;
    return grouped_gemm_wgrad(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups, total_m, n,
                              k, alpha_a, alpha_b, flags, stream);
}

extern "C" int mxl_grouped_gemm_wgrad(const void* a_codes, const void* a_scales, int a_fmt, const void* b_codes,
                                      const void* b_scales, int b_fmt, void* c_bf16, const int64_t* group_lens,
                                      int num_groups, int64_t total_m, int64_t n, int64_t k, void* stream) {
    return mxl_grouped_gemm_wgrad_ex(a_codes, a_scales, a_fmt, b_codes, b_scales, b_fmt, c_bf16, group_lens, num_groups,
                                     total_m, n, k, 0, stream);
}

extern "C" int mxl_version(void) { return 1; }

extern "C" const char* mxl_error_string(int code) {
    switch (code) {
        case MXL_OK: return "ok";
        case MXL_EINVAL: return "invalid argument (shape, alignment, enum or null pointer)";
        case MXL_ELAUNCH: return "HIP launch error";
        case MXL_ENODEV: return "device is not gfx950";
        case MXL_ESCRATCH: return "the problem needs more scratch memory than this allocation-free entry point owns";
        case MXL_ESTREAM: return "the allocation-free entry point is bound to another stream on this device (or unbound while capturing)";
        default: return "unknown error";
    }
}
