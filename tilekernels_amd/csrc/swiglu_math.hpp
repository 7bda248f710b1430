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
// exp(-g) = 2^(g * -log2 e) on v_exp_f32.
//   bf16 input: one product with float(-log2 e).  Its rounding puts up to |g| * 1.44 * 2^-24 of absolute error into
//               the exponent, i.e. a relative error of |g| * 6e-8 in exp(-g); that only reaches the result where
//               exp(-g) dominates 1 + exp(-g) (gates below about -3), whose outputs are small against the group
//               maximum that sets the scale.  Against the CPU evaluation at bf16 [8192, 4096], N(0,1): 4.2e-7 of the
//               codes differ (budget 1e-4), each by one step, scales within 3.1e-7 (budget 1e-6); a hi/lo split of
//               the constant (two more operations per element) brought the codes to 2.4e-7 and cost 0.08 us of 14.6.
//   fp32 input: the constant is split into hi + lo and the rounding error of g*hi is recovered with an fma, both
//               applied to first order: 2^(g*hi + t) = 2^(g*hi) * (1 + t * ln 2).
// The gate is capped at -88 inside the exponential only (the CPU's exp overflows to inf at -88.7 and
// its quotient becomes -0): e and 1 + e then stay finite, the reciprocal underflows and the corrected
// quotient is -0 or a value below 1e-36, never inf * 0.

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
    return __builtin_amdgcn_exp2f(floor_at_minus_88(g) * -1.4426950408889634f);
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

// g / d from r ~ 1/d: one Newton step on the quotient (two fmas).  Without the step the quotient is off by an ulp
// often enough to matter where many elements share one gate value: every element of a group is then the same factor
// times its up value, 448 * v / amax falls on exact rounding boundaries of the format for a sizeable share of them, and
// the last bit of the factor decides which way those go.  Codes differing from the CPU's, with / without the step: gate
// 0.5 everywhere 0 / 1.1e-3, gate 3.0 everywhere 0 / 1.3e-3, gates clamped to 0.5 ... / 1.0e-4 (the budget is 1e-4);
// N(0,1) gates 2.4e-7 either way.  The step costs 0.2 us of the 14.2 of bf16 [8192, 2 x 2048] on MI355X.
__device__ __forceinline__ float quotient_with(float g, float d, float r) {
    const float q0 = g * r;
    return __builtin_fmaf(__builtin_fmaf(-d, q0, g), r, q0);
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
