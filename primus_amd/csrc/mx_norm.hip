// RMSNorm in front of the column-parallel linear (the reference's LayerNormColumnParallelLinear runs
// rmsnorm(x, layer_norm_weight, eps) and hands the result to gemm_fp8 / gemm_fp4:
// primus/backends/megatron/core/extensions/primus_turbo.py:1689-1700):
//
//   rstd[m] = 1 / sqrt(mean_j x[m, j]^2 + eps)          y[m, j] = (x[m, j] * rstd[m]) * w[j]
//
// bf16 in and out, fp32 arithmetic, one rounding per output.  All kernels stream: a workgroup per row
// (forward) or per strided set of rows (backward), 16 bytes per lane and access; a row is read twice, the
// second time from cache.  The sum of squares has a fixed order (per lane over its 8-element chunks in
// order, xor-butterfly over the 64 lanes from distance 32 down to 1, then the four waves in order), so a
// CPU restatement reproduces rstd and y bit for bit.
//
// Backward: with g = dy * w and xh = x * rstd,  dx = (g - xh * mean_j(g * xh)) * rstd  and
// dw[j] = sum_m dy[m, j] * xh[m, j].  The column sums are accumulated per workgroup in registers over the
// rows it owns, written to a caller-provided fp32 workspace [blocks, k] and added up by a second kernel.
#include "mx_device.h"

namespace mxl {

constexpr int NTHREADS = 256;
constexpr int NORM_MAX_K = 16384;          // 8 chunks of 8 columns per lane
constexpr int NORM_CHUNK_K = NTHREADS * 8;  // columns one round of 16-byte loads of the workgroup covers

typedef uint32_t nu32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 norm_load16(const void* s) {
    const nu32x4 t = *(const nu32x4*)s;
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void norm_store16(void* d, const uint4& v) {
    const nu32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (nu32x4*)d);
}

// sum over the workgroup in a fixed order; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* part) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) v += __shfl_xor(v, s);
    __syncthreads();   // part may still be read from the previous use
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    return ((part[0] + part[1]) + part[2]) + part[3];
}

__device__ __forceinline__ float row_rstd(const uint16_t* xr, int64_t k, float eps, float* part) {
    float ss = 0.f;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < k; c += NTHREADS * 8) {
        const uint4 v = norm_load16(xr + c);
        const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float a = bf16_lo(wv[i]), b = bf16_hi(wv[i]);
            ss += a * a;   // squares of bf16 values are exact in fp32
            ss += b * b;
        }
    }
    const float total = block_sum(ss, part);
    return 1.0f / sqrtf(total / (float)k + eps);
}

// y may be null: then only rstd is produced (the fused normalisation + quantisation reads x itself)
__global__ __launch_bounds__(NTHREADS) void rmsnorm_fwd_kernel(const uint16_t* x, const uint16_t* w, float eps, int64_t k,
                                                               uint16_t* y, float* rstd) {
    __shared__ float part[NTHREADS / 64];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * k;
    const float r = row_rstd(xr, k, eps, part);
    if (threadIdx.x == 0) rstd[row] = r;
    if (y == nullptr) return;
    uint16_t* yr = y + row * k;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < k; c += NTHREADS * 8)
        norm_store16(yr + c, norm8(norm_load16(xr + c), norm_load16(w + c), r));
}

// CH: 8-column chunks per lane (k <= CH * 2048).  The weight chunks are loaded once per workgroup and a
// row's x and dy stay in registers between the reduction and the output pass.
template <int CH>
__global__ __launch_bounds__(NTHREADS) void rmsnorm_bwd_kernel(const uint16_t* dy, const uint16_t* x, const uint16_t* w,
                                                               const float* rstd, int64_t rows, int64_t k, uint16_t* dx,
                                                               float* partial) {
    __shared__ float part[NTHREADS / 64];
    float acc[CH][8];
    uint4 wv[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int64_t c = ((int64_t)j * NTHREADS + threadIdx.x) * 8;
        wv[j] = c < k ? norm_load16(w + c) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
    }
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const uint16_t *xr = x + row * k, *dr = dy + row * k;
        uint16_t* dxr = dx + row * k;
        uint4 xv[CH], dv[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int64_t c = ((int64_t)j * NTHREADS + threadIdx.x) * 8;
            xv[j] = dv[j] = make_uint4(0, 0, 0, 0);
            if (c < k) {
                xv[j] = norm_load16(xr + c);
                dv[j] = norm_load16(dr + c);
            }
        }
        const float r = rstd[row];
        // sum_j g * xh, and the column sums (chunks past k hold zeros)
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const uint32_t xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, dw[4] = {dv[j].x, dv[j].y, dv[j].z, dv[j].w},
                           ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float xh0 = bf16_lo(xw[i]) * r, xh1 = bf16_hi(xw[i]) * r;
                const float d0 = bf16_lo(dw[i]), d1 = bf16_hi(dw[i]);
                acc[j][2 * i] += d0 * xh0;
                acc[j][2 * i + 1] += d1 * xh1;
                dot += d0 * bf16_lo(ww[i]) * xh0;
                dot += d1 * bf16_hi(ww[i]) * xh1;
            }
        }
        const float cmean = block_sum(dot, part) / (float)k;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int64_t c = ((int64_t)j * NTHREADS + threadIdx.x) * 8;
            if (c < k) {
                const uint32_t xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, dw[4] = {dv[j].x, dv[j].y, dv[j].z, dv[j].w},
                               ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float xh0 = bf16_lo(xw[i]) * r, xh1 = bf16_hi(xw[i]) * r;
                    const float g0 = bf16_lo(dw[i]) * bf16_lo(ww[i]), g1 = bf16_hi(dw[i]) * bf16_hi(ww[i]);
                    o[i] = pack_bf16((g0 - xh0 * cmean) * r, (g1 - xh1 * cmean) * r);
                }
                norm_store16(dxr + c, make_uint4(o[0], o[1], o[2], o[3]));
            }
        }
    }
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int64_t c = ((int64_t)j * NTHREADS + threadIdx.x) * 8;
        if (c < k) {
            float* pr = partial + (int64_t)blockIdx.x * k + c;
            *(float4*)pr = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
            *(float4*)(pr + 4) = make_float4(acc[j][4], acc[j][5], acc[j][6], acc[j][7]);
        }
    }
}

// dw[j] = sum over the blocks' partial rows.  A workgroup owns 32 columns: thread (bg, cg) adds rows
// bg, bg + 32, ... of column group cg (4 columns) in order, then the 32 partial sums are added in order.
__global__ __launch_bounds__(NTHREADS) void rmsnorm_dw_kernel(const float* partial, int blocks, int64_t k, uint16_t* dw) {
    __shared__ float4 part[32][8];
    const int cg = threadIdx.x & 7, bg = threadIdx.x >> 3;
    const int64_t c = (int64_t)blockIdx.x * 32 + 4 * cg;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < k) {
        for (int b = bg; b < blocks; b += 32) {
            const float4 v = *(const float4*)(partial + (int64_t)b * k + c);
            s.x += v.x;
            s.y += v.y;
            s.z += v.z;
            s.w += v.w;
        }
    }
    part[bg][cg] = s;
    __syncthreads();
    if (bg == 0 && c < k) {
        float4 t = part[0][cg];
        for (int i = 1; i < 32; ++i) {
            const float4 v = part[i][cg];
            t.x += v.x;
            t.y += v.y;
            t.z += v.z;
            t.w += v.w;
        }
        *(uint2*)(dw + c) = make_uint2(pack_bf16(t.x, t.y), pack_bf16(t.z, t.w));
    }
}

}  // namespace mxl

using namespace mxl;

static bool norm_shape_ok(int64_t rows, int64_t k) {
    return rows >= 0 && rows <= 0x7FFFFFFF && k > 0 && k % 8 == 0 && k <= NORM_MAX_K;
}

// chunks per lane the backward kernel is compiled for, and the workgroups it runs (= rows of the workspace):
// the narrow variants keep few registers, so more workgroups fit a CU
static int norm_bwd_chunks(int64_t k) { return k <= NORM_CHUNK_K ? 1 : k <= 2 * NORM_CHUNK_K ? 2 : k <= 4 * NORM_CHUNK_K ? 4 : 8; }
static int norm_bwd_blocks(int64_t rows, int64_t k) {
    const int ch = norm_bwd_chunks(k);
    const int64_t cap = 2048 / ch;   // about what is resident on 256 CUs at the variant's register count
    return (int)(rows < cap ? rows : cap);
}

extern "C" int mxl_rmsnorm_fwd(const void* x_bf16, const void* w_bf16, float eps, int64_t rows, int64_t k, void* y_bf16,
                               void* rstd_f32, void* stream) {
    if (!norm_shape_ok(rows, k) || !(eps >= 0.f)) return MXL_EINVAL;
    if (rows == 0) return MXL_OK;
    if (!x_bf16 || !rstd_f32 || (y_bf16 && !w_bf16)) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipLaunchKernelGGL(rmsnorm_fwd_kernel, dim3((unsigned)rows), dim3(NTHREADS), 0, (hipStream_t)stream,
                       (const uint16_t*)x_bf16, (const uint16_t*)w_bf16, eps, k, (uint16_t*)y_bf16, (float*)rstd_f32);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int64_t mxl_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t k) {
    if (!norm_shape_ok(rows, k)) return -1;
    return (int64_t)norm_bwd_blocks(rows, k) * k * 4;
}

// shared by the two backward entry points; `workspace` is the caller's buffer or this device's static scratch
static int rmsnorm_bwd(const void* dy_bf16, const void* x_bf16, const void* w_bf16, const void* rstd_f32,
                       int64_t rows, int64_t k, void* dx_bf16, void* dw_bf16, void* workspace,
                       int64_t workspace_bytes, void* stream) {
    if (!norm_shape_ok(rows, k) || !dw_bf16) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipStream_t st = (hipStream_t)stream;
    const int blocks = norm_bwd_blocks(rows, k);
    if (rows > 0) {
        if (!dy_bf16 || !x_bf16 || !w_bf16 || !rstd_f32 || !dx_bf16 || !workspace) return MXL_EINVAL;
        if (workspace_bytes < (int64_t)blocks * k * 4 || ((uintptr_t)workspace & 15) != 0) return MXL_EINVAL;
#define MXL_NORM_BWD(CH)                                                                                              \
    hipLaunchKernelGGL(rmsnorm_bwd_kernel<CH>, dim3((unsigned)blocks), dim3(NTHREADS), 0, st, (const uint16_t*)dy_bf16,   \
                       (const uint16_t*)x_bf16, (const uint16_t*)w_bf16, (const float*)rstd_f32, rows, k,                  \
                       (uint16_t*)dx_bf16, (float*)workspace)
        switch (norm_bwd_chunks(k)) {
            case 1: MXL_NORM_BWD(1); break;
            case 2: MXL_NORM_BWD(2); break;
            case 4: MXL_NORM_BWD(4); break;
            default: MXL_NORM_BWD(8); break;
        }
#undef MXL_NORM_BWD
        if (hipGetLastError() != hipSuccess) return MXL_ELAUNCH;
    }
    // no rows: the weight gradient is zero (the loop over zero blocks writes it)
    const int64_t grid = (k + 31) / 32;
    hipLaunchKernelGGL(rmsnorm_dw_kernel, dim3((unsigned)grid), dim3(NTHREADS), 0, st, (const float*)workspace, blocks, k,
                       (uint16_t*)dw_bf16);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int mxl_rmsnorm_bwd(const void* dy_bf16, const void* x_bf16, const void* w_bf16, const void* rstd_f32,
                               int64_t rows, int64_t k, void* dx_bf16, void* dw_bf16, void* workspace,
                               int64_t workspace_bytes, void* stream) {
    return rmsnorm_bwd(dy_bf16, x_bf16, w_bf16, rstd_f32, rows, k, dx_bf16, dw_bf16, workspace, workspace_bytes, stream);
}

// ---- the same without a workspace argument and without any allocation ----
// The partial column sums go through a file-scope device array.  Each GPU holds its own copy of it at its own
// address (from the moment the library's code is loaded there until the process ends); the address is asked
// for once per device, with that device current, and kept.  Host code must never hand the array's NAME to a
// kernel: on the host that name is a stand-in, not a device address.
constexpr int64_t NORM_SCRATCH_BYTES = (int64_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[NORM_SCRATCH_BYTES];

// Per device: the array's address and the stream the entry point is bound to.  All calls on a GPU share the one
// array, so two calls in flight at once would mix their partial sums: the entry point serves ONE stream per device
// (calls on a stream are ordered) and refuses any other with MXL_ESTREAM until the caller rebinds it.
constexpr int NORM_MAXDEV = 1024;
static std::atomic<void*> norm_scratch_ptrs[NORM_MAXDEV];
static std::atomic<uintptr_t> norm_scratch_owner[NORM_MAXDEV];      // 0 = unbound, else the stream handle | 1
static uintptr_t stream_key(void* stream) { return (uintptr_t)stream | 1u; }

// the current device's copy of the array; asked for once per device (never while a stream is capturing: the
// query is not a stream operation, but it may initialise the module on the device)
static int norm_scratch_resolve(int dev, void** out) {
    void* ptr = norm_scratch_ptrs[dev].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MXL_ELAUNCH;
        norm_scratch_ptrs[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return MXL_OK;
}

extern "C" int64_t mxl_rmsnorm_bwd_noalloc_max_bytes(void) { return NORM_SCRATCH_BYTES; }

extern "C" int mxl_rmsnorm_bwd_noalloc_bind(void* stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NORM_MAXDEV) return MXL_ENODEV;
    if (!device_is_gfx950()) return MXL_ENODEV;
    void* ptr = nullptr;
    const int rc = norm_scratch_resolve(dev, &ptr);
    if (rc != MXL_OK) return rc;
    norm_scratch_owner[dev].store(stream_key(stream), std::memory_order_release);
    return MXL_OK;
}

extern "C" int mxl_rmsnorm_bwd_noalloc(const void* dy_bf16, const void* x_bf16, const void* w_bf16, const void* rstd_f32,
                                       int64_t rows, int64_t k, void* dx_bf16, void* dw_bf16, void* stream) {
    if (!norm_shape_ok(rows, k) || !dw_bf16) return MXL_EINVAL;
    // same partial-sum geometry as mxl_rmsnorm_bwd (hence the same bits); a problem whose partial sums do not
    // fit the static array is refused
    if ((int64_t)norm_bwd_blocks(rows, k) * k * 4 > NORM_SCRATCH_BYTES) return MXL_ESCRATCH;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NORM_MAXDEV) return MXL_ENODEV;
    uintptr_t owner = norm_scratch_owner[dev].load(std::memory_order_acquire);
    if (owner == 0) {
        // first use on this device without a bind: this call binds its stream, unless that stream is being
        // captured (set-up does not belong into a capture: the caller binds beforehand)
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing((hipStream_t)stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return MXL_ESTREAM;
        const int rc = mxl_rmsnorm_bwd_noalloc_bind(stream);
        if (rc != MXL_OK) return rc;
        owner = stream_key(stream);
    }
    if (owner != stream_key(stream)) return MXL_ESTREAM;
    void* ptr = norm_scratch_ptrs[dev].load(std::memory_order_acquire);
    if (!ptr) return MXL_ELAUNCH;
    return rmsnorm_bwd(dy_bf16, x_bf16, w_bf16, rstd_f32, rows, k, dx_bf16, dw_bf16, ptr, NORM_SCRATCH_BYTES, stream);
}
