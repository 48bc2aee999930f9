// Device-side helpers shared by the MX quantisers and GEMMs (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mxlinear.h"

#include <string.h>

#include <atomic>

namespace mxl {

// Host side: is the current device a gfx950?  The kernels exist for that target only; every entry point
// asks before its first launch on a device (answer cached per device index) and returns MXL_ENODEV otherwise.
inline bool device_is_gfx950() {
    static std::atomic<int> known[64];   // 0 unknown, 1 yes, 2 no
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    const int slot = dev & 63;
    int v = known[slot].load(std::memory_order_relaxed);
    if (v == 0) {
        hipDeviceProp_t pr;
        if (hipGetDeviceProperties(&pr, dev) != hipSuccess) return false;
        v = strncmp(pr.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
        known[slot].store(v, std::memory_order_relaxed);
    }
    return v == 1;
}

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));

constexpr int kFmtE4M3 = MXL_FMT_E4M3;
constexpr int kFmtE2M1 = MXL_FMT_E2M1;
constexpr int kFmtE5M2 = MXL_FMT_E5M2;   // tensor-wise scaled operands only (gradients of the HYBRID format)

// Exponent of the largest normal, its fp32 mantissa field, explicit mantissa bits.
template <int FMT> struct Elem;
template <> struct Elem<kFmtE4M3> {
    static constexpr int emax = 8;
    static constexpr uint32_t maxman = 0x600000u;  // 448 = 1.75 * 2^8
    static constexpr int mbits = 3;
};
template <> struct Elem<kFmtE2M1> {
    static constexpr int emax = 2;
    static constexpr uint32_t maxman = 0x400000u;  // 6 = 1.5 * 2^2
    static constexpr int mbits = 1;
};

// E8M0 byte of a block from the largest bf16 magnitude in it (15-bit pattern).
// Integer arithmetic on the fp32 exponent field only; 255 marks a block that
// holds a NaN or an infinity.
template <int FMT, int SMODE>
__device__ __forceinline__ uint32_t scale_byte(uint32_t amax16) {
    uint32_t b = amax16 << 16;
    if (SMODE == MXL_SCALE_EVEN) b += 1u << (23 - Elem<FMT>::mbits - 1);
    int e = (int)(b >> 23);
    if (SMODE == MXL_SCALE_RCEIL) e += ((b & 0x7FFFFFu) > Elem<FMT>::maxman) ? 1 : 0;
    e -= Elem<FMT>::emax;
    e = e < 0 ? 0 : (e > 254 ? 254 : e);
    return amax16 >= 0x7F80u ? 255u : (uint32_t)e;
}

// 2^(127 - byte) for byte <= 253 (always a normal float).
__device__ __forceinline__ float inv_scale(uint32_t byte) { return __uint_as_float((254u - byte) << 23); }
// 2^(byte - 127) for byte in [1, 254]; byte 0 gives the subnormal 2^-127.
__device__ __forceinline__ float fwd_scale(uint32_t byte) {
    return byte ? __uint_as_float(byte << 23) : __uint_as_float(0x00400000u);
}

__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

// Largest magnitude (as 15-bit patterns) of the two bf16 halves, lane-wise packed.
__device__ __forceinline__ uint32_t pk_absmax(uint32_t acc, uint32_t pair) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    us2 a = __builtin_bit_cast(us2, acc);
    us2 b = __builtin_bit_cast(us2, pair & 0x7FFF7FFFu);
    us2 r = {(unsigned short)(a[0] > b[0] ? a[0] : b[0]), (unsigned short)(a[1] > b[1] ? a[1] : b[1])};
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_max16(uint32_t x, uint32_t y) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    us2 a = __builtin_bit_cast(us2, x);
    us2 b = __builtin_bit_cast(us2, y);
    us2 r = {(unsigned short)(a[0] > b[0] ? a[0] : b[0]), (unsigned short)(a[1] > b[1] ? a[1] : b[1])};
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t hmax16(uint32_t pk) {
    uint32_t lo = pk & 0xFFFFu, hi = pk >> 16;
    return lo > hi ? lo : hi;
}

// Two bf16 (packed) -> two E4M3 bytes in the low 16 bits.  `inv` is the
// power-of-two factor; the clamp makes the hardware convert (round to nearest
// even, NaN on overflow) saturating.
__device__ __forceinline__ uint32_t cvt2_e4m3(uint32_t pair, float inv) {
    float a = __builtin_amdgcn_fmed3f(bf16_lo(pair) * inv, -448.f, 448.f);
    float b = __builtin_amdgcn_fmed3f(bf16_hi(pair) * inv, -448.f, 448.f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xFFFFu;
}
// Four bf16 (two packed pairs) -> four E4M3 bytes.
__device__ __forceinline__ uint32_t cvt4_e4m3(uint32_t p0, uint32_t p1, float inv) {
    float a = __builtin_amdgcn_fmed3f(bf16_lo(p0) * inv, -448.f, 448.f);
    float b = __builtin_amdgcn_fmed3f(bf16_hi(p0) * inv, -448.f, 448.f);
    float c = __builtin_amdgcn_fmed3f(bf16_lo(p1) * inv, -448.f, 448.f);
    float d = __builtin_amdgcn_fmed3f(bf16_hi(p1) * inv, -448.f, 448.f);
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
    return (uint32_t)r;
}
// The same for E5M2 (tensor-wise scaled gradients): multiply, clamp at +-57344, round to nearest even.
__device__ __forceinline__ uint32_t cvt4_e5m2(uint32_t p0, uint32_t p1, float inv) {
    float a = __builtin_amdgcn_fmed3f(bf16_lo(p0) * inv, -57344.f, 57344.f);
    float b = __builtin_amdgcn_fmed3f(bf16_hi(p0) * inv, -57344.f, 57344.f);
    float c = __builtin_amdgcn_fmed3f(bf16_lo(p1) * inv, -57344.f, 57344.f);
    float d = __builtin_amdgcn_fmed3f(bf16_hi(p1) * inv, -57344.f, 57344.f);
    int r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
    return (uint32_t)r;
}
template <int FMT> __device__ __forceinline__ uint32_t cvt4_fp8(uint32_t p0, uint32_t p1, float inv) {
    return FMT == kFmtE5M2 ? cvt4_e5m2(p0, p1, inv) : cvt4_e4m3(p0, p1, inv);
}
// Slow path for a block that holds a NaN/Inf: finite lanes -> signed zero,
// non-finite lanes -> NaN code with the input's sign.
__device__ __forceinline__ uint32_t nonfinite1_e4m3(uint32_t h) {
    uint32_t s = (h >> 8) & 0x80u;
    return ((h & 0x7FFFu) >= 0x7F80u) ? (s | 0x7Fu) : s;
}
__device__ __forceinline__ uint32_t nonfinite4_e4m3(uint32_t p0, uint32_t p1) {
    return nonfinite1_e4m3(p0 & 0xFFFFu) | (nonfinite1_e4m3(p0 >> 16) << 8) | (nonfinite1_e4m3(p1 & 0xFFFFu) << 16) |
           (nonfinite1_e4m3(p1 >> 16) << 24);
}

// Two bf16 (packed) -> two E2M1 nibbles in bits 7:0 (element 0 in bits 3:0).
// The hardware convert divides by `scale` (a power of two), rounds to nearest
// even and saturates at +-6.
__device__ __forceinline__ uint32_t cvt2_e2m1(uint32_t pair, float scale) {
    v2bf h = __builtin_bit_cast(v2bf, pair);
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(0u, h, scale, 0) & 0xFFu;
}
__device__ __forceinline__ uint32_t nonfinite1_e2m1(uint32_t h) {
    uint32_t s = (h >> 12) & 0x8u;
    return ((h & 0x7FFFu) >= 0x7F80u) ? (s | 0x7u) : s;
}
__device__ __forceinline__ uint32_t nonfinite2_e2m1(uint32_t pair) {
    return nonfinite1_e2m1(pair & 0xFFFFu) | (nonfinite1_e2m1(pair >> 16) << 4);
}

// ---- stochastic rounding to E2M1 (gradients of the MXFP4 recipe: rowwise_use_sr / colwise_use_sr of
// quantize_mxfp4_dual, primus/backends/megatron/core/extensions/primus_turbo_mxfp4_local.py:272-288).
// Integer arithmetic throughout so that a CPU restatement reproduces every code:
//   w = |x| * 2^(127 - scale byte)                         (exact: power-of-two scaling of a bf16)
//   w >= 1: the fp32 pattern of w plus a random integer below 2^22, cut after one mantissa bit
//           (round up with probability = the dropped fraction), saturating at 6;
//   w <  1: floor(w * 2^23) plus the same random integer, cut at 2^22  -> 0, 0.5 or 1.
// Random bits: a counter-based hash, 16 bits per element, two elements per 32-bit word.
__device__ __forceinline__ uint32_t sr_mix(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7FEB352Du;
    x ^= x >> 15;
    x *= 0x846CA68Bu;
    x ^= x >> 16;
    return x;
}
__device__ __forceinline__ uint32_t sr_word(uint64_t counter, uint64_t seed, uint32_t stream) {
    const uint32_t h = sr_mix((uint32_t)counter ^ (uint32_t)seed);
    return sr_mix(h + (uint32_t)(counter >> 32) * 0x9E3779B9u + (uint32_t)(seed >> 32) + stream * 0x85EBCA6Bu);
}
__device__ __forceinline__ uint32_t sr1_e2m1(float x, float inv, uint32_t rnd16) {
    const float w = fabsf(x) * inv;
    const uint32_t sign = (__float_as_uint(x) >> 28) & 0x8u;
    const uint32_t add = rnd16 << 6;
    uint32_t mag;
    if (w < 1.f) {
        mag = ((uint32_t)(w * 8388608.f) + add) >> 22;
    } else {
        mag = ((__float_as_uint(w) + add) >> 22) - 252u;
        mag = mag > 7u ? 7u : mag;
    }
    return sign | mag;
}
// two bf16 (packed) -> two nibbles in bits 7:0, element 0 (random bits 15:0) in bits 3:0
__device__ __forceinline__ uint32_t sr2_e2m1(uint32_t pair, float inv, uint32_t rnd) {
    return sr1_e2m1(bf16_lo(pair), inv, rnd & 0xFFFFu) | (sr1_e2m1(bf16_hi(pair), inv, rnd >> 16) << 4);
}

// ---- gated activation of the expert MLP (shared by the activation kernels and the fused
// activation + quantisation path, so that both round identically) ----
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    v2bf h = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, h);
}
template <int ACT> __device__ __forceinline__ float act_fwd(float g) {
    // hardware exp2 and reciprocal (about 1 ulp each in fp32, far inside the bf16 rounding of the result); the
    // IEEE division and the range handling of expf would make the fused quantiser ALU-bound
    if (ACT == MXL_ACT_SILU) return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
    // 0.5 g erfc(-g / sqrt 2); erfc (not 1 + erf): no cancellation in the negative tail.  erfc(z), z >= 0, from
    // the rational-exponential fit t exp(-z^2 + P(t)), t = 1 / (1 + z / 2) (fractional error below 1.2e-7
    // everywhere, Numerical Recipes 6.2), with the hardware reciprocal and exp2: the library erfcf would make
    // the fused quantiser ALU-bound.
    const float x = g * -0.70710678118654752f, z = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(1.f + 0.5f * z);
    float p = 0.17087277f;
    p = p * t - 0.82215223f;
    p = p * t + 1.48851587f;
    p = p * t - 1.13520398f;
    p = p * t + 0.27886807f;
    p = p * t - 0.18628806f;
    p = p * t + 0.09678418f;
    p = p * t + 0.37409196f;
    p = p * t + 1.00002368f;
    p = p * t - 1.26551223f;
    const float e = t * __builtin_amdgcn_exp2f((p - z * z) * 1.4426950408889634f);
    return 0.5f * g * (x >= 0.f ? e : 2.f - e);
}
__device__ __forceinline__ float load_prob(const void* probs, int probs_bf16, int64_t row) {
    if (probs_bf16) return __uint_as_float((uint32_t)((const uint16_t*)probs)[row] << 16);
    return ((const float*)probs)[row];
}
// 8 outputs act(g) * u * p from 8 gate and 8 linear bf16 values, rounded once to bf16
template <int ACT> __device__ __forceinline__ uint4 glu8(const uint4& g, const uint4& u, float p) {
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float lo = act_fwd<ACT>(bf16_lo(gw[k])) * bf16_lo(uw[k]) * p;
        const float hi = act_fwd<ACT>(bf16_hi(gw[k])) * bf16_hi(uw[k]) * p;
        ow[k] = pack_bf16(lo, hi);
    }
    return make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// ---- RMSNorm (shared by the normalisation kernels and the fused normalisation + quantisation path) ----
// 8 outputs (x * rstd) * w from 8 input and 8 weight bf16 values, fp32 products in that order, rounded once
__device__ __forceinline__ uint4 norm8(const uint4& x, const uint4& wv, float rstd) {
    const uint32_t xw[4] = {x.x, x.y, x.z, x.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
        ow[k] = pack_bf16(bf16_lo(xw[k]) * rstd * bf16_lo(ww[k]), bf16_hi(xw[k]) * rstd * bf16_hi(ww[k]));
    return make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// ---- shared by the quantisers ----
// The quantisers stream: every input byte is read once and every output byte written once, by one
// workgroup.  Non-temporal accesses keep that traffic from displacing the scale words in L2, which
// do have to wait there for their neighbours (the 8 x 8 supertile order of the quantisers' grids).
typedef uint32_t qu32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t qu32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store16_streaming(void* d, const uint4& v) {
    const qu32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (qu32x4*)d);
}
__device__ __forceinline__ void store8_streaming(void* d, const uint2& v) {
    const qu32x2 t = {v.x, v.y};
    __builtin_nontemporal_store(t, (qu32x2*)d);
}
__device__ __forceinline__ void store4_streaming(void* d, uint32_t v) { __builtin_nontemporal_store(v, (uint32_t*)d); }
__device__ __forceinline__ uint4 load16_streaming(const void* s) {
    const qu32x4 t = __builtin_nontemporal_load((const qu32x4*)s);
    return make_uint4(t.x, t.y, t.z, t.w);
}

__device__ __forceinline__ uint32_t dpp_xor1(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t dpp_xor2(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
}
// the other two steps of a maximum over the 16 lanes of a DPP row: lane i <-> 7 - i inside each half row, lane i <-> 15 - i
__device__ __forceinline__ uint32_t dpp_half_mirror(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
}
__device__ __forceinline__ uint32_t dpp_mirror(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true);  // row_mirror
}

}  // namespace mxl
