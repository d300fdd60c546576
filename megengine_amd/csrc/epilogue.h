// Fused requantisation epilogue shared by every ConvBias kernel.
//
// Arithmetic contract (one separately rounded IEEE binary32 operation per step, exactly the
// order of naive::ConvBiasForwardImpl, dnn/src/naive/conv_bias/opr_impl.cpp:21-98, with the
// dtype conversions of dnn/include/megdnn/dtype.h:845-853,:897):
//     r = float(sfb) * s_bias            sfb = int32 accumulator + bias
//     r = r + float(z) * s_z             only when z is present
//     r = act(r)                         RELU: r <= 0 ? 0 : r;  H_SWISH: r*min(max(r+3,0),6)*(1/6)
//     v = roundf(r / s_dst)              true division, ties away from zero
//     dst = (int8) min(max(-128, v), 127)
//
// The "fast" form below produces the same bits with no hardware divide:
//   * division by the per-tensor constant s_dst: with y_hi = RN(1/s_dst), y_lo = RN(1/s_dst - y_hi)
//       q0 = fma(r, y_hi, r * y_lo)      faithful quotient (error << 1 ulp before its rounding)
//       e  = fma(-q0, s_dst, r)          exact residual
//       q  = fma(e, y_hi, q0)            correctly rounded r / s_dst (Markstein's correction step)
//   * RELU is folded into the clamp: for s_dst > 0, r <= 0 gives q <= 0 which clamps to 0.
//   * roundf + clamp + convert: clamp first, then trunc(q + copysign(pred(0.5), q)); for
//     |q| <= 128 the sum is exact except below 0.5 where pred(0.5) keeps it under 1.  After a RELU
//     clamp q >= 0 and the hardware's round-to-plus-infinity conversion does the same in one step.
// The host only selects the fast form when the scales are positive, normal and small enough
// that no intermediate overflows (see epi_fast_ok in capi.hip); otherwise kernels run the
// literal form with the IEEE divide.
//
// The "linear" form (NL_LIN; IDENTITY or RELU without z) is one fused multiply-add:
//     dst = floor(min(max(fma(float(sfb), c, d), lo), 127.5))
// Without z the contract above is a non-decreasing step function of the integer sfb with at most 255
// steps, and so is this form for c > 0.  Two non-decreasing step functions are equal on every integer
// iff each step of one sits at the same integer as the corresponding step of the other, so the host
// finds the 255 step positions of the contract by bisection, chooses (c, d) from them and then
// checks every step of the candidate against them with the device's own arithmetic (epi_solve_linear
// in capi.hip).  Only a pair (c, d) that passes is ever handed to a kernel; when none passes, the
// fast form runs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

struct EpiParams {
    float s_b, s_z, s_d;
    float y_hi, y_lo;
    int nonline;  // MI355_NL_*
    int has_z;
    int fast;     // 1: fast form allowed
    int lin;      // 1: linear form verified for (s_b, s_d, nonline); implies fast && !has_z
    float lin_c, lin_d, lin_lo;
};

// NL_LIN is not an activation of the interface: it selects the linear form in the kernels' epilogue templates
enum { NL_IDENTITY = 0, NL_RELU = 1, NL_H_SWISH = 3, NL_LIN = 4 };

__device__ __forceinline__ float act_f32(float r, int nl) {
    if (nl == NL_RELU) return r <= 0.f ? 0.f : r;
    if (nl == NL_H_SWISH) {
        float t = r + 3.f;
        t = fminf(fmaxf(t, 0.f), 6.f);
        float m = r * t;
        return m * (1.f / 6.f);
    }
    return r;
}

// literal form, any scales (also the only form for QuantizedS32 dst)
__device__ __forceinline__ int requant_s8_exact(int sfb, bool has_z, int z, const EpiParams& e) {
    float r = (float)sfb * e.s_b;
    if (has_z) {
        float zf = (float)z * e.s_z;
        r = r + zf;
    }
    r = act_f32(r, e.nonline);
    float v = r / e.s_d;
    v = __builtin_roundf(v);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int)v;
}

__device__ __forceinline__ int requant_s32_exact(int sfb, bool has_z, int z, const EpiParams& e) {
    float r = (float)sfb * e.s_b;
    if (has_z) {
        float zf = (float)z * e.s_z;
        r = r + zf;
    }
    r = act_f32(r, e.nonline);
    float v = r / e.s_d;
    v = __builtin_roundf(v);
    v = fminf(fmaxf(-2147483648.f, v), 2147483520.f);
    return (int)v;
}

// fast form; NL and HAS_Z are compile-time so the inner loops carry no branches
template <int NL, bool HAS_Z>
__device__ __forceinline__ int requant_s8_fast(int sfb, int z, const EpiParams& e) {
    if (NL == NL_LIN) {
        float x = __builtin_fmaf((float)sfb, e.lin_c, e.lin_d);
        x = __builtin_amdgcn_fmed3f(x, e.lin_lo, 127.5f);
        int o;
        asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(o) : "v"(x));  // (int)floor(x): x is finite and inside [-128, 127.5]
        return o;
    }
    float r = (float)sfb * e.s_b;
    if (HAS_Z) {
        float zf = (float)z * e.s_z;
        r = r + zf;
    }
    if (NL == NL_H_SWISH) {
        float t = r + 3.f;
        t = fminf(fmaxf(t, 0.f), 6.f);
        float m = r * t;
        r = m * (1.f / 6.f);
    }
    float t0 = r * e.y_lo;
    float q0 = __builtin_fmaf(r, e.y_hi, t0);
    float res = __builtin_fmaf(-q0, e.s_d, r);
    float q = __builtin_fmaf(res, e.y_hi, q0);
    int out;
    if (NL == NL_RELU) {
        q = __builtin_amdgcn_fmed3f(q, 0.f, 127.f);  // q is finite here: same as min(max(q, 0), 127)
        // floor(q + 0.5) computed exactly by the hardware (round to nearest, ties to +infinity): for q >= 0 that is
        // round-half-away, one instruction instead of add + truncate.  Equal to (int)(q + 0.49999997f) on every
        // float in [0, 127] (checked exhaustively on gfx950).
        asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(out) : "v"(q));
    } else {
        q = __builtin_amdgcn_fmed3f(q, -128.f, 127.f);
        out = (int)(q + __builtin_copysignf(0.49999997f, q));
    }
    return out;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);  // b.b0 a.b0
    uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// 4 accumulators (consecutive channels) + packed z word -> packed int8x4
template <int NL, bool HAS_Z>
__device__ __forceinline__ uint32_t requant4_fast(int a0, int a1, int a2, int a3, uint32_t zw,
                                                  const EpiParams& e) {
    int z0 = 0, z1 = 0, z2 = 0, z3 = 0;
    if (HAS_Z) {
        z0 = (int)(int8_t)(zw);
        z1 = (int)(int8_t)(zw >> 8);
        z2 = (int)(int8_t)(zw >> 16);
        z3 = (int)zw >> 24;
    }
    int r0 = requant_s8_fast<NL, HAS_Z>(a0, z0, e);
    int r1 = requant_s8_fast<NL, HAS_Z>(a1, z1, e);
    int r2 = requant_s8_fast<NL, HAS_Z>(a2, z2, e);
    int r3 = requant_s8_fast<NL, HAS_Z>(a3, z3, e);
    return pack4(r0, r1, r2, r3);
}

__device__ __forceinline__ uint32_t requant4_exact(int a0, int a1, int a2, int a3, uint32_t zw,
                                                   const EpiParams& e) {
    bool hz = e.has_z != 0;
    int r0 = requant_s8_exact(a0, hz, (int)(int8_t)(zw), e);
    int r1 = requant_s8_exact(a1, hz, (int)(int8_t)(zw >> 8), e);
    int r2 = requant_s8_exact(a2, hz, (int)(int8_t)(zw >> 16), e);
    int r3 = requant_s8_exact(a3, hz, (int)zw >> 24, e);
    return pack4(r0, r1, r2, r3);
}

// runtime dispatch used by the bandwidth-bound kernels (one uniform branch per call site)
__device__ __forceinline__ uint32_t requant4(int a0, int a1, int a2, int a3, uint32_t zw, const EpiParams& e) {
    if (!e.fast) return requant4_exact(a0, a1, a2, a3, zw, e);
    if (e.lin) return requant4_fast<NL_LIN, false>(a0, a1, a2, a3, zw, e);
    if (e.has_z) {
        switch (e.nonline) {
            case NL_RELU: return requant4_fast<NL_RELU, true>(a0, a1, a2, a3, zw, e);
            case NL_H_SWISH: return requant4_fast<NL_H_SWISH, true>(a0, a1, a2, a3, zw, e);
            default: return requant4_fast<NL_IDENTITY, true>(a0, a1, a2, a3, zw, e);
        }
    }
    switch (e.nonline) {
        case NL_RELU: return requant4_fast<NL_RELU, false>(a0, a1, a2, a3, zw, e);
        case NL_H_SWISH: return requant4_fast<NL_H_SWISH, false>(a0, a1, a2, a3, zw, e);
        default: return requant4_fast<NL_IDENTITY, false>(a0, a1, a2, a3, zw, e);
    }
}

}  // namespace mi355
