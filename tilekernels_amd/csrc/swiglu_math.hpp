// fp32 SwiGLU arithmetic shared by the forward and backward kernels (gfx950).
#pragma once

#include "tk_device.hpp"

namespace tk {

// exp(-g) and g / (1 + exp(-g)) in fp32, built on v_exp_f32 / v_rcp_f32 (about 1 ulp each).
// The reference's CPU evaluation (vectorised exp, IEEE division) is itself only faithful to about
// 1 ulp in exp, so bit equality is not defined for these ops; what can be matched is everything after
// the exp: 1 + e is one IEEE addition, the quotient is corrected to (almost always) the IEEE
// quotient, and the products that follow are single roundings in the reference's order.
//
// exp(-g) = 2^(g * -log2 e).  Rounding that product would put |g|*2^-24 of absolute error into the
// exponent, so the constant is split into hi + lo and the lo part is applied to first order:
// 2^(g*hi + g*lo) = 2^(g*hi) * (1 + g*lo*ln 2).
//   bf16 input: hi keeps 15 significant bits, so g*hi is exact for an 8-bit significand
//   fp32 input: the rounding error of g*hi is recovered with an fma and joins the lo term
// The gate is capped at -88 inside the exponential only (the CPU's exp overflows to inf at -88.7 and
// its quotient becomes -0): e and 1 + e then stay finite, the reciprocal underflows and the corrected
// quotient is -0 or a value below 1e-36, never inf * 0.
#ifndef TK_SWIGLU_NEWTON
#define TK_SWIGLU_NEWTON 1
#endif

// max(g, -88) on the bit pattern: negative floats order like their patterns as unsigned integers, and
// every non-negative float has a smaller pattern than -88, so one integer min does it.  (A float max
// would cost a second instruction: its operand is an unpacked bit pattern that the compiler has to
// canonicalise first.)  NaNs with the sign bit set come out as -88, other NaNs pass through.
__device__ __forceinline__ float floor_at_minus_88(float g) {
    const uint32_t b = f2u(g);
    return u2f(b < 0xC2B00000u ? b : 0xC2B00000u);
}

template <typename InT> __device__ __forceinline__ float exp_neg(float g);

template <> __device__ __forceinline__ float exp_neg<bf16_t>(float g) {
    constexpr float nh = -1.44268798828125f;             // -log2(e) cut to 15 significant bits (0xBFB8AA00)
    constexpr float nl_ln2 = -4.8884952e-06f;            // (-log2(e) - nh) * ln 2
    const float gc = floor_at_minus_88(g);
    const float e0 = __builtin_amdgcn_exp2f(gc * nh);    // exact product
    return __builtin_fmaf(e0, gc * nl_ln2, e0);
}

template <> __device__ __forceinline__ float exp_neg<float>(float g) {
    constexpr float nh = -1.4426950216293335f;           // float(-log2 e)
    constexpr float nl = -1.9259629911266175e-8f;        // -log2 e - nh
    const float gc = floor_at_minus_88(g);
    const float th = gc * nh;
    const float tl = __builtin_fmaf(gc, nl, __builtin_fmaf(gc, nh, -th));
    const float e0 = __builtin_amdgcn_exp2f(th);
    return __builtin_fmaf(e0, tl * 0.6931471805599453f, e0);
}

// g / d from r ~ 1/d: one Newton step on the quotient (two fmas)
__device__ __forceinline__ float quotient_with(float g, float d, float r) {
    const float q0 = g * r;
#if TK_SWIGLU_NEWTON
    return __builtin_fmaf(__builtin_fmaf(-d, q0, g), r, q0);
#else
    return q0;
#endif
}
__device__ __forceinline__ float quotient(float g, float d) { return quotient_with(g, d, __builtin_amdgcn_rcpf(d)); }

// 1 / d for finite d >= 1: v_rcp_f32 plus one Newton step (two fmas), which lands on the correctly
// rounded reciprocal in all but a vanishing share of cases
__device__ __forceinline__ float reciprocal(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}

// silu(g) * u
template <typename InT> __device__ __forceinline__ float silu_mul(float g, float u) {
    return quotient(g, 1.0f + exp_neg<InT>(g)) * u;
}

}  // namespace tk
