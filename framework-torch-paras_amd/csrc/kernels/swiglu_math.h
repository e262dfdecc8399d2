// silu(gate) * up for one element, with the rounding of the reference's host
// engine: fp64 evaluation, then double -> float -> T
// (csrc/ops/fused_ops.cpp:185-190).  Shared by the streaming SwiGLU kernel and
// the MoE expert GEMM epilogue.
//
// For the 16-bit dtypes the value is computed in two tiers:
//   fast  fp32 evaluation with a proven relative error bound kFastRelErr; the
//         result is accepted when both ends of the error interval round to
//         the same 16-bit value, which means the fp64 result rounds there too;
//   exact the fp64 formula, taken by the few lanes whose interval straddles a
//         rounding boundary (about 1 element in 1000) or whose gate lies
//         outside the range the bound was derived for.
// The output therefore equals the fp64-then-round definition everywhere, not
// only within a tolerance.  fp32/fp64 tensors use the fp64 formula directly.
#pragma once

#include <hip/hip_runtime.h>

#include "core/device_math.h"

namespace paras {

// Bound on |fast - exact| / |exact| for gate in [kFastGateMin, kFastGateMax]:
// the exponent argument g*log2(e) carries at most |g*log2e| * 2^-23 absolute
// error (product rounding + constant), i.e. <= 8.1e-7 relative on exp for
// g >= -8 (for g > 0 the term exp(-g) <= 1 is damped by 1/(1+e)); v_exp_f32,
// the add, v_rcp_f32 and the two multiplies add < 5e-7.  2^-19 = 1.9e-6
// covers the sum with margin.
constexpr float kFastRelErr  = 1.9073486328125e-06f;  // 2^-19
constexpr float kFastGateMin = -8.0f;
constexpr float kFastGateMax = 60.0f;

template <typename T>
__device__ __forceinline__ typename Elem<T>::store_t swiglu_exact(float g, float u) {
    const double gd = static_cast<double>(g);
    const double s  = gd / (1.0 + exp(-gd));
    return Elem<T>::from_f64(s * static_cast<double>(u));
}

template <typename T>
__device__ __forceinline__ typename Elem<T>::store_t swiglu_one(typename Elem<T>::store_t gs,
                                                                  typename Elem<T>::store_t us) {
    using E = Elem<T>;
    if constexpr (sizeof(typename E::store_t) == 2) {
        const float g = E::to_f32(gs);
        const float u = E::to_f32(us);
        const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
        const float y = g * __builtin_amdgcn_rcpf(1.0f + e) * u;
        const auto lo = E::from_f32(y * (1.0f - kFastRelErr));
        const auto hi = E::from_f32(y * (1.0f + kFastRelErr));
        // NaN gates fail the range test and take the exact tier.  A result in
        // fp32's denormal range has no relative bound, so it is only accepted
        // when it is an exact zero (zero gate or zero up).
        const bool sized = (fabsf(y) >= 1e-30f) || (g == 0.0f) || (u == 0.0f);
        const bool ok = (lo == hi) && (g >= kFastGateMin) && (g <= kFastGateMax) && sized;
        // Return the rounding of y itself: it lies between lo and hi, and unlike
        // them it keeps the sign of a zero result (the compiler may form lo/hi
        // with a fused multiply-add-convert whose +0 addend drops it).
        if (__builtin_expect(ok, 1)) return E::from_f32(y);
        return swiglu_exact<T>(g, u);
    } else {
        const double g = E::to_f64(gs);
        const double s = g / (1.0 + exp(-g));
        return E::from_f64(s * E::to_f64(us));
    }
}

}  // namespace paras
