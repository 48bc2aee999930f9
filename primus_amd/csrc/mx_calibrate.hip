// A register-only MFMA loop: what the matrix cores of this board sustain when nothing else runs.  The published
// peak of the scaled FP8/FP4 MFMAs assumes the 2.4 GHz boost clock; under a GEMM's load the board sits at its power
// limit and clocks lower, so a measured ceiling is the honest yardstick beside the published one.  Every wave
// holds the 128 x 128 accumulator tile of the GEMM kernels (16 accumulators of 32 x 32) and four fragments per
// operand with pseudo-random codes and scale bytes, and issues the GEMM's 16 MFMAs per K step back to back:
// no LDS, no global memory, no barriers.
#include "mx_device.h"

namespace mxl {

__device__ float calibrate_sink[64];   // external linkage: the store below must count as observable

__device__ __forceinline__ uint32_t calib_hash(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

// CA / CB: the MFMA's format codes of the two operands (0 = E4M3, 4 = E2M1)
template <int CA, int CB>
__global__ __launch_bounds__(256) void mfma_only_kernel(int iters) {
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x;
    v8i a[4], b[4];
    int sa[4], sb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            // magnitudes below 2 and no NaN codes, so that the sums stay finite for any number of iterations
            a[i][e] = (int)(calib_hash(tid * 131u + i * 17u + e) & 0xBFBFBFBFu);
            b[i][e] = (int)(calib_hash(tid * 257u + i * 29u + e + 99u) & 0xBFBFBFBFu);
        }
        sa[i] = 100 + (int)(calib_hash(tid + i) & 15u);
        sb[i] = 100 + (int)(calib_hash(tid * 3u + i) & 15u);
    }
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j], a[i], acc[i][j], CB, CA, 0, sb[j], 0, sa[i]);
        a[0][0] ^= it;           // the operands change a little from step to step
        b[1][3] ^= it << 3;
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    if (s == 12345.678f) calibrate_sink[threadIdx.x & 63] = s;   // keeps the loop alive; practically never taken
}

// The same for the bf16 MFMA of the unquantised grouped GEMM (32 x 32 x 16): 32 MFMAs per iteration on the 128 x 128
// accumulator tile, i.e. one K slot of 32 elements.
typedef __bf16 cal_v8bf __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void mfma_only_bf16_kernel(int iters) {
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // two bf16 per word, exponents 0x3C .. 0x3F (magnitudes below 2, no NaN or Inf patterns)
            a[i][e] = (int)((calib_hash(tid * 131u + i * 17u + e) & 0x81FF81FFu) | 0x3E003E00u);
            b[i][e] = (int)((calib_hash(tid * 257u + i * 29u + e + 99u) & 0x81FF81FFu) | 0x3E003E00u);
        }
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(cal_v8bf, b[j]), __builtin_bit_cast(cal_v8bf, a[i]),
                                                                        acc[i][j], 0, 0, 0);
            a[0][0] ^= (it & 0xFF);   // the operands change a little from step to step (mantissa bits only)
            b[1][3] ^= (it & 0x1F) << 3;
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    if (s == 12345.678f) calibrate_sink[threadIdx.x & 63] = s;
}

// The traffic of the dual quantiser without its arithmetic: every workgroup reads a 128 x 128 bf16 tile (16 bytes per
// lane, rows adjacent) and writes one byte per element at the tile's place in a row-major array and one byte per
// element at its place in the transposed array (16-byte stores; the bytes are XORs of the input, nothing is
// transposed or converted), streaming loads and stores, tiles walked in the quantiser's order (8 x 8 supertiles, one
// XCD each).  What this moves per second is what the quantiser's access pattern allows on the board.
typedef uint32_t cu32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t cu32x2 __attribute__((ext_vector_type(2)));
template <bool ROW, bool COL>
__global__ __launch_bounds__(256) void tile_copy_kernel(const uint16_t* in, uint8_t* o_row, uint8_t* o_col, int64_t cols,
                                                        int64_t w_ld, int tiles_r, int tiles_c, int super_c, int n_super) {
    constexpr int TR = 128, TC = 128;
    const int L = blockIdx.x, xcd = L & 7, k = L >> 3;
    const int sup = (k / 64) * 8 + xcd;
    if (sup >= n_super) return;
    const int within = k % 64;
    const int pt = (sup / super_c) * 8 + within / 8, ct = (sup % super_c) * 8 + within % 8;
    if (pt >= tiles_r || ct >= tiles_c) return;
    const int t = threadIdx.x;
    constexpr int LPR = TC * 2 / 16, RPI = 256 / LPR, NIT = TR / RPI;   // 16 lanes a row, 16 rows a pass, 8 passes
    cu32x4 d[NIT];
    const int64_t r0 = (int64_t)pt * TR, c0 = (int64_t)ct * TC;
#pragma unroll
    for (int i = 0; i < NIT; ++i) {
        const int r = i * RPI + t / LPR, c = (t % LPR) * 8;
        d[i] = __builtin_nontemporal_load((const cu32x4*)(in + (r0 + r) * cols + c0 + c));
    }
    cu32x4 acc = d[0];
#pragma unroll
    for (int i = 1; i < NIT; ++i) acc ^= d[i];
    if (ROW) {
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int r = i * RPI + t / LPR, c = (t % LPR) * 8;
            const cu32x2 v = {d[i].x ^ d[i].y, d[i].z ^ d[i].w};
            __builtin_nontemporal_store(v, (cu32x2*)(o_row + (r0 + r) * cols + c0 + c));
        }
    }
    if (COL) {
        constexpr int LPR2 = TR / 16, RPI2 = 256 / LPR2;                // 8 lanes a transposed row, 32 rows a pass
#pragma unroll
        for (int i = 0; i < TC / RPI2; ++i) {
            const int c = i * RPI2 + t / LPR2, ch = t % LPR2;
            __builtin_nontemporal_store(acc ^ d[i % NIT], (cu32x4*)(o_col + (c0 + c) * w_ld + r0 + ch * 16));
        }
    }
    if (!ROW && !COL && acc.x == 0x12345u && acc.y == 0x54321u) calibrate_sink[t & 63] = 1.f;   // keeps the loads alive
}


// The rule the GEMM kernels' operand requests rely on, made observable: one LDS-direct 16-byte buffer load per case
// through a raw descriptor over `buf` with num_records = cases[i].records, per-lane offset .voff and scalar offset
// .soff; out[4 i .. 4 i + 3] = the four dwords that arrived in LDS (zeros where the range check dropped them).
struct RangeCase { uint32_t voff, soff, records; };
__global__ __launch_bounds__(64) void range_check_kernel(const uint8_t* buf, const RangeCase* cases, int n, uint32_t* out) {
    __shared__ __attribute__((aligned(16))) uint32_t lds[64 * 4];
    const uint64_t p = (uint64_t)buf;
    for (int i = 0; i < n; ++i) {
        const RangeCase cs = cases[i];
        v4i r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32) & 0xFFFF);
        r[2] = __builtin_amdgcn_readfirstlane((int)cs.records);
        r[3] = 0x00020000;
        const uint32_t voff = cs.voff, soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)cs.soff);
        for (int j = threadIdx.x; j < 256; j += 64) lds[j] = 0xDEADBEEFu;
        __syncthreads();
        const uint32_t lbase = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds\n\ts_waitcnt vmcnt(0)"
                     :
                     : "s"(lbase), "v"(voff), "s"(r), "s"(soff)
                     : "memory");
        __syncthreads();
        if (threadIdx.x < 4) out[4 * i + threadIdx.x] = lds[threadIdx.x];
        __syncthreads();
    }
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_calibrate_tile_copy(const void* in_bf16, int64_t rows, int64_t cols, void* out_row, void* out_colT,
                                       void* stream) {
    if (rows <= 0 || cols <= 0 || rows % 128 || cols % 128 || rows > (int64_t(1) << 30) || cols > (int64_t(1) << 30) || !in_bf16)
        return MXL_EINVAL;
    if ((((uintptr_t)in_bf16 | (uintptr_t)out_row | (uintptr_t)out_colT) & 15) != 0) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const int tiles_r = (int)(rows / 128), tiles_c = (int)(cols / 128);
    const int super_r = (tiles_r + 7) / 8, super_c = (tiles_c + 7) / 8, n_super = super_r * super_c;
    const int64_t wgs = (int64_t)(n_super + 7) / 8 * 8 * 64;
    if (wgs > 0x7FFFFFFF) return MXL_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)wgs), block(256);
    const uint16_t* in = (const uint16_t*)in_bf16;
    uint8_t *o1 = (uint8_t*)out_row, *o2 = (uint8_t*)out_colT;
    if (o1 && o2) hipLaunchKernelGGL((tile_copy_kernel<true, true>), grid, block, 0, st, in, o1, o2, cols, rows, tiles_r, tiles_c, super_c, n_super);
    else if (o1) hipLaunchKernelGGL((tile_copy_kernel<true, false>), grid, block, 0, st, in, o1, o2, cols, rows, tiles_r, tiles_c, super_c, n_super);
    else if (o2) hipLaunchKernelGGL((tile_copy_kernel<false, true>), grid, block, 0, st, in, o1, o2, cols, rows, tiles_r, tiles_c, super_c, n_super);
    else hipLaunchKernelGGL((tile_copy_kernel<false, false>), grid, block, 0, st, in, o1, o2, cols, rows, tiles_r, tiles_c, super_c, n_super);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int64_t mxl_calibrate_mfma_flops(int64_t iters) {
    // 256 workgroups x 4 waves x iters x 16 MFMAs of 32 x 32 x 64
    return iters < 0 ? -1 : 256 * 4 * iters * 16 * (2LL * 32 * 32 * 64);
}

extern "C" int mxl_calibrate_mfma(int a_fmt, int b_fmt, int64_t iters, void* stream) {
    if (iters < 1 || iters > (1 << 24)) return MXL_EINVAL;
    const bool a4 = a_fmt == MXL_FMT_E2M1, b4 = b_fmt == MXL_FMT_E2M1;
    if ((a_fmt != MXL_FMT_E4M3 && !a4) || (b_fmt != MXL_FMT_E4M3 && !b4)) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(256), block(256);
    if (a4 && b4) hipLaunchKernelGGL((mfma_only_kernel<4, 4>), grid, block, 0, st, (int)iters);
    else if (a4) hipLaunchKernelGGL((mfma_only_kernel<4, 0>), grid, block, 0, st, (int)iters);
    else if (b4) hipLaunchKernelGGL((mfma_only_kernel<0, 4>), grid, block, 0, st, (int)iters);
    else hipLaunchKernelGGL((mfma_only_kernel<0, 0>), grid, block, 0, st, (int)iters);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int64_t mxl_calibrate_mfma_bf16_flops(int64_t iters) {
    // 256 workgroups x 4 waves x iters x 32 MFMAs of 32 x 32 x 16
    return iters < 0 ? -1 : 256 * 4 * iters * 32 * (2LL * 32 * 32 * 16);
}

extern "C" int mxl_calibrate_mfma_bf16(int64_t iters, void* stream) {
    if (iters < 1 || iters > (1 << 24)) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipLaunchKernelGGL(mfma_only_bf16_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, (int)iters);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int mxl_calibrate_range_check(const void* buf, int64_t buf_bytes, const void* cases, int num_cases, void* out,
                                         int64_t max_offset_host, void* stream) {
    // max_offset_host: the largest voff + soff among the cases, stated by the caller: every case must stay inside
    // `buf` whatever the hardware decides, so that the probe can never touch memory it does not own
    if (!buf || !cases || !out || num_cases < 0 || max_offset_host < 0 || max_offset_host + 16 > buf_bytes) return MXL_EINVAL;
    if (((uintptr_t)buf & 15) != 0) return MXL_EINVAL;
    if (num_cases == 0) return MXL_OK;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipLaunchKernelGGL(range_check_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (const uint8_t*)buf,
                       (const RangeCase*)cases, num_cases, (uint32_t*)out);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}
