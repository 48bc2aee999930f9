// Gated activation of the expert MLP fused with the router probability and the row mask
// (swiglu_with_probs / geglu_with_probs as called by the reference's fused_bias_act_with_probs,
// primus/backends/megatron/core/extensions/primus_turbo.py:1954-1980; unfused arithmetic at
// primus/backends/megatron/core/transformer/experts.py:100-118):
//
//   y[m, j] = act(x[m, j]) * x[m, F + j] * p[m]            rows with mask 0 give 0
//
// for bf16 x[rows, 2F], computed in fp32 and rounded once to bf16.  Backward returns dx[rows, 2F]
// and dp[rows] (fp32).  Both kernels stream: one workgroup per row, 16 bytes per lane and access.
#include "mx_device.h"

namespace mxl {

constexpr int ATHREADS = 256;

typedef uint32_t au32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 act_load16(const void* s) {
    const au32x4 t = __builtin_nontemporal_load((const au32x4*)s);
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void act_store16(void* d, const uint4& v) {
    const au32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (au32x4*)d);
}
// act(g) together with its derivative, fp32
template <int ACT> __device__ __forceinline__ void act_both(float g, float& a, float& da) {
    if (ACT == MXL_ACT_SILU) {
        const float s = 1.f / (1.f + expf(-g));
        a = g * s;
        da = s * (1.f + g * (1.f - s));
    } else {
        const float c = 0.5f * erfcf(-g * 0.70710678118654752f);
        a = g * c;
        da = c + g * 0.39894228040143268f * expf(-0.5f * g * g);
    }
}

template <int ACT>
__global__ __launch_bounds__(ATHREADS) void glu_probs_fwd_kernel(const uint16_t* x, const void* probs, int probs_bf16,
                                                                 const uint8_t* row_mask, int64_t f, uint16_t* y) {
    const int64_t row = blockIdx.x;
    const bool live = row_mask == nullptr || row_mask[row] != 0;
    const float p = live ? load_prob(probs, probs_bf16, row) : 0.f;
    const uint16_t* xg = x + row * 2 * f;
    uint16_t* yr = y + row * f;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < f; c += ATHREADS * 8) {
        uint4 o = make_uint4(0, 0, 0, 0);
        if (live) {
            o = glu8<ACT>(act_load16(xg + c), act_load16(xg + f + c), p);
        }
        act_store16(yr + c, o);
    }
}

template <int ACT>
__global__ __launch_bounds__(ATHREADS) void glu_probs_bwd_kernel(const uint16_t* dy, const uint16_t* x, const void* probs,
                                                                 int probs_bf16, const uint8_t* row_mask, int64_t f,
                                                                 uint16_t* dx, float* dprobs) {
    __shared__ float part[ATHREADS / 64];
    const int64_t row = blockIdx.x;
    const bool live = row_mask == nullptr || row_mask[row] != 0;
    const float p = live ? load_prob(probs, probs_bf16, row) : 0.f;
    const uint16_t* xg = x + row * 2 * f;
    const uint16_t* dyr = dy + row * f;
    uint16_t* dxr = dx + row * 2 * f;
    float acc = 0.f;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < f; c += ATHREADS * 8) {
        uint4 o1 = make_uint4(0, 0, 0, 0), o2 = o1;
        if (live) {
            const uint4 g = act_load16(xg + c), u = act_load16(xg + f + c), d = act_load16(dyr + c);
            const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w}, dw[4] = {d.x, d.y, d.z, d.w};
            uint32_t w1[4], w2[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float a0, da0, a1, da1;
                act_both<ACT>(bf16_lo(gw[k]), a0, da0);
                act_both<ACT>(bf16_hi(gw[k]), a1, da1);
                const float u0 = bf16_lo(uw[k]), u1 = bf16_hi(uw[k]);
                const float d0 = bf16_lo(dw[k]), d1 = bf16_hi(dw[k]);
                acc += d0 * (a0 * u0) + d1 * (a1 * u1);
                w1[k] = pack_bf16(d0 * p * u0 * da0, d1 * p * u1 * da1);
                w2[k] = pack_bf16(d0 * p * a0, d1 * p * a1);
            }
            o1 = make_uint4(w1[0], w1[1], w1[2], w1[3]);
            o2 = make_uint4(w2[0], w2[1], w2[2], w2[3]);
        }
        act_store16(dxr + c, o1);
        act_store16(dxr + f + c, o2);
    }
    // row sum of dy * act(g) * u over the workgroup
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) acc += __shfl_xor(acc, s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < ATHREADS / 64; ++i) t += part[i];
        dprobs[row] = live ? t : 0.f;
    }
}

}  // namespace mxl

using namespace mxl;

static bool act_args_ok(const void* a, const void* b, const void* probs, int probs_dtype, int64_t rows, int64_t f, int act) {
    if (rows < 0 || f <= 0 || f % 8 != 0 || rows > 0x7FFFFFFF) return false;
    if (act != MXL_ACT_SILU && act != MXL_ACT_GELU) return false;
    if (probs_dtype != MXL_PROBS_F32 && probs_dtype != MXL_PROBS_BF16) return false;
    return rows == 0 || (a && b && probs);
}

extern "C" int mxl_glu_probs_fwd(const void* x_bf16, const void* probs, int probs_dtype, const uint8_t* row_mask,
                                 int64_t rows, int64_t f, int act, void* y_bf16, void* stream) {
    if (!act_args_ok(x_bf16, y_bf16, probs, probs_dtype, rows, f, act)) return MXL_EINVAL;
    if (rows == 0) return MXL_OK;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const dim3 grid((unsigned)rows), block(ATHREADS);
    hipStream_t st = (hipStream_t)stream;
    if (act == MXL_ACT_SILU)
        hipLaunchKernelGGL((glu_probs_fwd_kernel<MXL_ACT_SILU>), grid, block, 0, st, (const uint16_t*)x_bf16, probs,
                           probs_dtype, row_mask, f, (uint16_t*)y_bf16);
    else
        hipLaunchKernelGGL((glu_probs_fwd_kernel<MXL_ACT_GELU>), grid, block, 0, st, (const uint16_t*)x_bf16, probs,
                           probs_dtype, row_mask, f, (uint16_t*)y_bf16);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

extern "C" int mxl_glu_probs_bwd(const void* dy_bf16, const void* x_bf16, const void* probs, int probs_dtype,
                                 const uint8_t* row_mask, int64_t rows, int64_t f, int act, void* dx_bf16,
                                 void* dprobs_f32, void* stream) {
    if (!act_args_ok(x_bf16, dx_bf16, probs, probs_dtype, rows, f, act)) return MXL_EINVAL;
    if (rows == 0) return MXL_OK;
    if (!dy_bf16 || !dprobs_f32) return MXL_EINVAL;
    if (!device_is_gfx950()) return MXL_ENODEV;
    const dim3 grid((unsigned)rows), block(ATHREADS);
    hipStream_t st = (hipStream_t)stream;
    if (act == MXL_ACT_SILU)
        hipLaunchKernelGGL((glu_probs_bwd_kernel<MXL_ACT_SILU>), grid, block, 0, st, (const uint16_t*)dy_bf16,
                           (const uint16_t*)x_bf16, probs, probs_dtype, row_mask, f, (uint16_t*)dx_bf16,
                           (float*)dprobs_f32);
    else
        hipLaunchKernelGGL((glu_probs_bwd_kernel<MXL_ACT_GELU>), grid, block, 0, st, (const uint16_t*)dy_bf16,
                           (const uint16_t*)x_bf16, probs, probs_dtype, row_mask, f, (uint16_t*)dx_bf16,
                           (float*)dprobs_f32);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}
