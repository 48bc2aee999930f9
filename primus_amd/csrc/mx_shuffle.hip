// The "pre-shuffled" MXFP4 layouts: byte permutations of packed FP4 codes and of E8M0 scale arrays, the layouts
// behind the shuffle_* flags of the reference's dual quantisation op and gemm_fp4_impl(preshuffled = True)
// (primus/backends/megatron/core/extensions/primus_turbo_mxfp4_local.py:147-161, :184-198, :319-331).
//
//   codes  [rows, row_bytes]: blocks of 16 rows x 32 bytes become 512 consecutive bytes, stored as
//          [half of 16 bytes][row in block][16 bytes]; the block order is row-major over (rows / 16, row_bytes / 32)
//   scales [rows, cols] -> [ceil(rows / 256) * 256, ceil(cols / 8) * 8] (zero bytes in the padding): 32 rows x 8
//          columns form a 256-byte group stored as [col % 4][row % 16][(col / 4) % 2][(row / 16) % 2]; the group
//          order is row-major over (rows / 32, cols / 8)
//
// The GEMM kernels of this library read their own layouts; these kernels convert at the boundary.  Index work only:
// one 16-byte piece (codes) or one byte (scales) per thread, the destination written linearly.
#include "mx_device.h"

namespace mxl {

typedef uint32_t su32x4 __attribute__((ext_vector_type(4)));

template <int INVERSE>
__global__ __launch_bounds__(256) void shuffle_codes_kernel(const su32x4* src, su32x4* dst, int64_t pieces, int64_t blocks_per_row,
                                                            int64_t row_pieces) {
    for (int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x; d < pieces; d += (int64_t)gridDim.x * 256) {
        if (INVERSE) {
            // d indexes the row-major array: piece (r, c)
            const int64_t r = d / row_pieces, c = d % row_pieces;
            const int64_t s = ((r / 16) * blocks_per_row + c / 2) * 32 + (c & 1) * 16 + r % 16;
            dst[d] = src[s];
        } else {
            // d indexes the shuffled array
            const int64_t block = d / 32, within = d % 32;
            const int64_t r = (block / blocks_per_row) * 16 + within % 16;
            const int64_t c = (block % blocks_per_row) * 2 + within / 16;
            dst[d] = src[r * row_pieces + c];
        }
    }
}

__device__ __forceinline__ int64_t scale_slot(int64_t m, int64_t n, int64_t groups_per_row) {
    return ((m / 32) * groups_per_row + n / 8) * 256 + (n % 4) * 64 + (m % 16) * 4 + ((n / 4) % 2) * 2 + (m / 16) % 2;
}

template <int INVERSE>
__global__ __launch_bounds__(256) void shuffle_scales_kernel(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t cols,
                                                             int64_t padded_rows, int64_t padded_cols) {
    const int64_t gpr = padded_cols / 8;
    if (INVERSE) {
        const int64_t total = rows * cols;
        for (int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x; d < total; d += (int64_t)gridDim.x * 256)
            dst[d] = src[scale_slot(d / cols, d % cols, gpr)];
    } else {
        const int64_t total = padded_rows * padded_cols;
        for (int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x; d < total; d += (int64_t)gridDim.x * 256) {
            const int64_t group = d / 256, w = d % 256;
            const int64_t m = (group / gpr) * 32 + (w % 2) * 16 + (w % 64) / 4;
            const int64_t n = (group % gpr) * 8 + ((w % 4) / 2) * 4 + w / 64;
            dst[d] = (m < rows && n < cols) ? src[m * cols + n] : (uint8_t)0;
        }
    }
}

static unsigned grid_for(int64_t items) {
    int64_t blocks = (items + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

}  // namespace mxl

using namespace mxl;

extern "C" int mxl_shuffle_codes(const void* src, int64_t rows, int64_t row_bytes, void* dst, int inverse, void* stream) {
    if (rows < 0 || row_bytes < 0 || rows % 16 || row_bytes % 32 || rows > (int64_t(1) << 40) || row_bytes > (int64_t(1) << 40))
        return MXL_EINVAL;
    if (rows == 0 || row_bytes == 0) return MXL_OK;
    if (!src || !dst || src == dst || (((uintptr_t)src | (uintptr_t)dst) & 15)) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const int64_t pieces = rows * (row_bytes / 16);
    hipStream_t st = (hipStream_t)stream;
    if (inverse)
        hipLaunchKernelGGL((shuffle_codes_kernel<1>), dim3(grid_for(pieces)), dim3(256), 0, st, (const su32x4*)src, (su32x4*)dst,
                           pieces, row_bytes / 32, row_bytes / 16);
    else
        hipLaunchKernelGGL((shuffle_codes_kernel<0>), dim3(grid_for(pieces)), dim3(256), 0, st, (const su32x4*)src, (su32x4*)dst,
                           pieces, row_bytes / 32, row_bytes / 16);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int mxl_shuffle_scales(const void* src, int64_t rows, int64_t cols, void* dst, int inverse, void* stream) {
    if (rows < 0 || cols < 0 || rows > (int64_t(1) << 40) || cols > (int64_t(1) << 32)) return MXL_EINVAL;
    if (rows == 0 || cols == 0) return MXL_OK;
    if (!src || !dst || src == dst) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const int64_t pr = (rows + 255) / 256 * 256, pc = (cols + 7) / 8 * 8;
    hipStream_t st = (hipStream_t)stream;
    if (inverse)
        hipLaunchKernelGGL((shuffle_scales_kernel<1>), dim3(grid_for(rows * cols)), dim3(256), 0, st, (const uint8_t*)src,
                           (uint8_t*)dst, rows, cols, pr, pc);
    else
        hipLaunchKernelGGL((shuffle_scales_kernel<0>), dim3(grid_for(pr * pc)), dim3(256), 0, st, (const uint8_t*)src,
                           (uint8_t*)dst, rows, cols, pr, pc);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}
