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
//   * division by the per-tensor constant s_dst: with the reciprocal as an unevaluated sum of two floats,
//     y_hi = RN(1/s_dst), y_lo = RN(1/s_dst - y_hi) (computed in double precision on the host),
//       t = r * y_lo                     the part of the quotient that y_hi misses (24 bits below it)
//       q = fma(r, y_hi, t)              r (y_hi + y_lo) rounded once: less than one ulp from r / s_dst
//     Such a quotient can change the result only next to a rounding boundary of roundf; the host proves the form
//     for every dst scale before a kernel may use it (epi_prove_quotient in capi.hip).
//   * RELU is folded into the clamp: for s_dst > 0, r <= 0 gives q <= 0 which clamps to 0.
//   * roundf + clamp + convert: clamp first, then trunc(q + copysign(pred(0.5), q)); for
//     |q| <= 128 the sum is exact except below 0.5 where pred(0.5) keeps it under 1.  After a RELU
//     clamp q >= 0 and the hardware's round-to-plus-infinity conversion does the same in one step.
//   * the four results of a dword are packed by the conversions themselves: the SDWA form of the convert writes the low
//     byte of its integer result into byte k of the destination and keeps the other bytes (no v_perm afterwards).
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
//
// The "residual table" form (NL_ZLIN; IDENTITY or RELU with z) is the linear form with an offset per residual value:
//     dst = floor(min(max(fma(float(sfb), c, tab[z]), lo), 127.5))          tab: 256 floats in LDS
// For each of the 256 values of z the contract is a step function of sfb as above; the host finds the steps of all 256,
// one slope c and an offset per z, and checks every step of every z with the device's arithmetic (epi_solve_table in
// capi.hip).  Five vector instructions and an LDS read per output instead of nine; scale triples without a proof
// (small s_bias / s_dst) run the fast form.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

struct EpiParams {
    float s_b, s_z, s_d;
    float y_hi;   // RN(1 / s_d)
    float y_lo;   // RN(1 / s_d - y_hi)
    int nonline;  // MI355_NL_*
    int has_z;
    int fast;     // 1: fast form allowed
    int lin;      // 1: linear form verified for (s_b, s_d, nonline); implies fast && !has_z
    float lin_c, lin_d, lin_lo;
    int zlin;     // 1: residual table form (set by the launch code of a kernel that holds the table; slope in lin_c)
};

// NL_LIN is not an activation of the interface: it selects the linear form in the kernels' epilogue templates
// and NL_ZLIN the residual table form
enum { NL_IDENTITY = 0, NL_RELU = 1, NL_H_SWISH = 3, NL_LIN = 4, NL_ZLIN = 5 };

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

// fast form; NL and HAS_Z are compile-time so the inner loops carry no branches.  Returns the value that the final
// conversion takes: clamped for NL_LIN (floor follows) and NL_RELU (round half up follows), clamped and moved half a
// unit away from zero otherwise (truncation follows).
template <int NL, bool HAS_Z>
__device__ __forceinline__ float requant_fast_value(int sfb, int z, const EpiParams& e) {
    if (NL == NL_LIN) {
        float x = __builtin_fmaf((float)sfb, e.lin_c, e.lin_d);
        return __builtin_amdgcn_fmed3f(x, e.lin_lo, 127.5f);  // finite and inside [-128, 127.5]
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
    float t = r * e.y_lo;
    float q = __builtin_fmaf(r, e.y_hi, t);
    if (NL == NL_RELU) return __builtin_amdgcn_fmed3f(q, 0.f, 127.f);  // q is finite here: same as min(max(q, 0), 127)
    q = __builtin_amdgcn_fmed3f(q, -128.f, 127.f);
    return q + __builtin_copysignf(0.49999997f, q);
}

// The final conversion of result K of a dword, written into byte K of `o` (the other bytes are kept; K = 0 clears them):
//   NL_LIN   floor            v_cvt_flr_i32_f32
//   NL_RELU  floor(x + 0.5)   v_cvt_rpi_i32_f32: exact (no intermediate rounding), for x >= 0 that is round-half-away; equal
//                             to (int)(x + 0.49999997f) on every float in [0, 127] (checked exhaustively on gfx950)
//   others   truncation       v_cvt_i32_f32
// Every result lies in [-128, 127]: its low byte is the int8 value.
template <int NL, int K>
__device__ __forceinline__ void convert_into_byte(uint32_t& o, float x) {
    static_assert(K >= 0 && K < 4, "byte of a dword");
    if (K == 0) {
        if (NL == NL_LIN)
            asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(o) : "v"(x));
        else if (NL == NL_RELU)
            asm("v_cvt_rpi_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(o) : "v"(x));
        else
            asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(o) : "v"(x));
    } else if (NL == NL_LIN) {
        if (K == 1) asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 2) asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 3) asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
    } else if (NL == NL_RELU) {
        if (K == 1) asm("v_cvt_rpi_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 2) asm("v_cvt_rpi_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 3) asm("v_cvt_rpi_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
    } else {
        if (K == 1) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 2) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
        if (K == 3) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o) : "v"(x));
    }
}

// one result, as an int (the generic one-thread-per-output kernel)
template <int NL, bool HAS_Z>
__device__ __forceinline__ int requant_s8_fast(int sfb, int z, const EpiParams& e) {
    const float x = requant_fast_value<NL, HAS_Z>(sfb, z, e);
    int o;
    if (NL == NL_LIN)
        asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(o) : "v"(x));
    else if (NL == NL_RELU)
        asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(o) : "v"(x));
    else
        o = (int)x;
    return o;
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
    const float x0 = requant_fast_value<NL, HAS_Z>(a0, z0, e);
    const float x1 = requant_fast_value<NL, HAS_Z>(a1, z1, e);
    const float x2 = requant_fast_value<NL, HAS_Z>(a2, z2, e);
    const float x3 = requant_fast_value<NL, HAS_Z>(a3, z3, e);
    uint32_t o;
    convert_into_byte<NL, 0>(o, x0);
    convert_into_byte<NL, 1>(o, x1);
    convert_into_byte<NL, 2>(o, x2);
    convert_into_byte<NL, 3>(o, x3);
    return o;
}

// residual table form: zt = the table in LDS, zw = the four residual bytes of the four accumulators
__device__ __forceinline__ uint32_t requant4_table(int a0, int a1, int a2, int a3, uint32_t zw, const EpiParams& e,
                                                   const float* zt) {
    const float x0 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)a0, e.lin_c, zt[zw & 0xffu]), e.lin_lo, 127.5f);
    const float x1 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)a1, e.lin_c, zt[(zw >> 8) & 0xffu]), e.lin_lo, 127.5f);
    const float x2 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)a2, e.lin_c, zt[(zw >> 16) & 0xffu]), e.lin_lo, 127.5f);
    const float x3 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)a3, e.lin_c, zt[zw >> 24]), e.lin_lo, 127.5f);
    uint32_t o;
    convert_into_byte<NL_LIN, 0>(o, x0);
    convert_into_byte<NL_LIN, 1>(o, x1);
    convert_into_byte<NL_LIN, 2>(o, x2);
    convert_into_byte<NL_LIN, 3>(o, x3);
    return o;
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
