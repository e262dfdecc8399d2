// Element math shared by the streaming kernels: results that equal the
// reference host engine's "evaluate in fp64, narrow double -> float -> T"
// (csrc/ops/fused_ops.cpp:72-84,185-190) at fp32 cost.
//
// Two tiers for the 16-bit dtypes:
//   fast   the value is computed in fp32 with a proven relative error bound.
//          If the fp32 result is further from every 16-bit rounding boundary
//          than that bound, the fp64 result narrows to the same 16-bit value,
//          so the fp32 result is narrowed and used.
//   exact  otherwise (about 1 element in 1000) the fp64 formula is evaluated.
// The output therefore equals the fp64-then-narrow definition everywhere, not
// only within a tolerance.  fp32 / fp64 tensors use the fp64 formula directly.
//
// The distance test works on the bits of the fp32 result: a 16-bit type with
// M explicit mantissa bits drops the low (23-M) bits; the rounding boundary
// sits at half of that field.  `ulps` is the error bound in fp32 ulps.
#pragma once

#include <hip/hip_runtime.h>

#include "core/device_math.h"

namespace paras {

template <typename T> struct Narrow16;
template <> struct Narrow16<bf16_t> {
    static constexpr std::uint32_t kMask = 0xFFFFu, kHalf = 0x8000u;
    // normal range of the result in which the dropped field has fixed width
    static constexpr float kMinNormal = 1e-30f, kMaxFinite = 3.0e38f;
};
template <> struct Narrow16<f16_t> {
    static constexpr std::uint32_t kMask = 0x1FFFu, kHalf = 0x1000u;
    static constexpr float kMinNormal = 6.2e-5f /* > 2^-14 */, kMaxFinite = 65000.0f;
};

// True when narrowing `y` (fp32, relative error <= ulps fp32 ulps) to T is safe.
template <typename T>
__device__ __forceinline__ bool narrow_is_safe(float y, std::uint32_t ulps) {
    const std::uint32_t b = __builtin_bit_cast(std::uint32_t, y);
    const std::uint32_t f = b & Narrow16<T>::kMask;
    const bool near = (f - (Narrow16<T>::kHalf - ulps)) <= 2u * ulps;  // unsigned wrap: one compare
    const float a = fabsf(y);
    const bool ranged = (a >= Narrow16<T>::kMinNormal) && (a <= Narrow16<T>::kMaxFinite);  // false for NaN
    return !near && ranged;
}

// ---- SwiGLU ------------------------------------------------------------------
// Error of the fp32 evaluation for gate in [kFastGateMin, kFastGateMax]: the
// exponent argument g*log2(e) carries at most |g*log2e| * 2^-23 absolute error
// (product rounding + constant), i.e. <= 8.1e-7 relative on exp for g >= -8
// (for g > 0 the term exp(-g) <= 1 is damped by 1/(1+e)); v_exp_f32, the add,
// v_rcp_f32 and the two multiplies add < 5e-7.  2^-19 = 1.9e-6 relative covers
// the sum with margin; that is 16 fp32 ulps at the bottom of a binade and 32
// at the top, so 32 is used.
constexpr std::uint32_t kSwigluUlps = 32;
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
        // |g - 26| <= 34  <=>  -8 <= g <= 60; false for a NaN gate.
        const bool ok = narrow_is_safe<T>(y, kSwigluUlps) && (fabsf(g - 26.0f) <= 34.0f);
        if (__builtin_expect(ok, 1)) return E::from_f32_finite(y);
        // A zero gate or zero up gives an exact signed zero (or NaN against an
        // infinity) in fp32 as in fp64; keep zero padding off the fp64 path.
        if (y == 0.0f && (g == 0.0f || u == 0.0f)) return E::from_f32(y);
        return swiglu_exact<T>(g, u);
    } else {
        const double g = E::to_f64(gs);
        const double s = g / (1.0 + exp(-g));
        return E::from_f64(s * E::to_f64(us));
    }
}

// SwiGLU of two fp32 accumulators (a GEMM epilogue): T(silu(T(a0)) * T(a1)) with the narrowing
// of a0 and a1 done by the conversion instruction on the common path.  That instruction differs
// from the host's narrowing for NaNs only, a NaN gate or up value makes y a NaN, and a NaN y fails
// the range test: whatever does not pass goes through swiglu_one on the software-narrowed values.
template <typename T>
__device__ __forceinline__ typename Elem<T>::store_t swiglu_from_acc(float a0, float a1) {
    using E = Elem<T>;
    static_assert(sizeof(typename E::store_t) == 2, "16-bit dtypes only");
    const float g = E::to_f32(E::from_f32_finite(a0));
    const float u = E::to_f32(E::from_f32_finite(a1));
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
    const float y = g * __builtin_amdgcn_rcpf(1.0f + e) * u;
    const bool ok = narrow_is_safe<T>(y, kSwigluUlps) && (fabsf(g - 26.0f) <= 34.0f);
    if (__builtin_expect(ok, 1)) return E::from_f32_finite(y);
    return swiglu_one<T>(E::from_f32(a0), E::from_f32(a1));
}

// The common tier of four of them at once (V: a vector of four floats), without a branch in between, so
// the exp / rcp chains overlap in a wave that has its SIMD to itself.  Returns whether all four passed
// their bounds: o then holds the results; otherwise the caller sends the four through swiglu_from_acc.
template <typename T, typename V>
__device__ __forceinline__ bool swiglu4_common_tier(const V a0, const V a1, typename Elem<T>::store_t (&o)[4]) {
    using E = Elem<T>;
    static_assert(sizeof(typename E::store_t) == 2, "16-bit dtypes only");
    bool ok = true;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const float g = E::to_f32(E::from_f32_finite(a0[r]));
        const float u = E::to_f32(E::from_f32_finite(a1[r]));
        const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
        const float y = g * __builtin_amdgcn_rcpf(1.0f + e) * u;
        ok = ok & (narrow_is_safe<T>(y, kSwigluUlps) & (fabsf(g - 26.0f) <= 34.0f));
        o[r] = E::from_f32_finite(y);
    }
    return ok;
}
template <typename T, typename V>
__device__ __forceinline__ void swiglu4_from_acc(const V a0, const V a1, typename Elem<T>::store_t (&o)[4]) {
    if (__builtin_expect(swiglu4_common_tier<T>(a0, a1, o), 1)) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = swiglu_from_acc<T>(a0[r], a1[r]);
}

// ---- SwiGLU backward -----------------------------------------------------------
// Host definition (csrc/ops/fused_ops.cpp:218-226), in fp64:
//   s = 1/(1+exp(-g));  dup = (dy*g)*s;  dgate = (dy*u) * (s * (1 + g*(1-s)))
// Fast tier in fp32 with e = exp2(-g*log2e), r = rcp(1+e) (= s), e*r (= 1-s, formed without the
// cancellation of 1-s), q = 1 + g*(e*r).  Error bounds in units of 2^-24 relative (one rounding
// = 1, v_exp_f32 / v_rcp_f32 = 2), with w = 1-s and Ee = 2|g| + 2 the error of e (argument
// rounding, amplified by |g|, plus the instruction's own):
//   r:      w*Ee + 3            (the error of e enters 1+e damped by w)
//   dup:    w*Ee + 5
//   e*r:    s*Ee + 4            (the errors of e in e and in r partly cancel)
//   q:      absolute |g e r| (s*Ee + 5) + |q|, i.e. relative rho (s*Ee + 5) + 1, rho = |g e r| / |q|
//   dgate:  w*Ee + 7 + rho (s*Ee + 5)
// q crosses zero near g = -1.278: rho grows without bound there and those elements take the exact
// tier.  The bounds are used with a factor 1.5 and 3 units of margin.  A relative error of E units
// is less than E fp32 ulps of the result, which is what narrow_is_safe takes.
template <typename T>
__device__ __forceinline__ void swiglu_bwd_exact(float dy, float g, float u, typename Elem<T>::store_t& dgate,
                                                 typename Elem<T>::store_t& dup) {
    const double dyd = static_cast<double>(dy), gd = static_cast<double>(g), ud = static_cast<double>(u);
    const double s = 1.0 / (1.0 + exp(-gd));
    dup = Elem<T>::from_f64(dyd * gd * s);
    dgate = Elem<T>::from_f64(dyd * ud * (s * (1.0 + gd * (1.0 - s))));
}

// Fast tier for one element of a 16-bit tensor: the fp32 results and whether each may be narrowed.
template <typename T>
__device__ __forceinline__ void swiglu_bwd_fast(float dy, float g, float u, float& yg, float& yu, bool& ok_g, bool& ok_u) {
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
    const float r = __builtin_amdgcn_rcpf(1.0f + e);
    const float er = e * r;
    yu = (dy * g) * r;
    const float ger = g * er;
    const float q = 1.0f + ger;
    yg = (dy * u) * (r * q);
    const float ee = fmaf(2.0f, fabsf(g), 2.0f);
    const float eu = fmaf(er, ee, 5.0f);
    const float rho = fabsf(ger) * __builtin_amdgcn_rcpf(fabsf(q));
    const float eg = fmaf(rho, fmaf(r, ee, 5.0f), eu + 2.0f);
    const bool in_range = (fabsf(g - 26.0f) <= 34.0f) && (rho < 4096.0f);     // -8 <= g <= 60, q well away from zero; false for NaN
    const std::uint32_t ulps_u = static_cast<std::uint32_t>(fmaf(1.5f, eu, 3.0f));
    const std::uint32_t ulps_g = static_cast<std::uint32_t>(fmaf(1.5f, in_range ? eg : 0.0f, 3.0f));
    ok_u = in_range && narrow_is_safe<T>(yu, ulps_u);
    ok_g = in_range && narrow_is_safe<T>(yg, ulps_g);
    // exact signed zeros need no fp64 (zero padding stays on the fast tier)
    ok_u = ok_u || (yu == 0.0f && (dy == 0.0f || g == 0.0f));
    ok_g = ok_g || (yg == 0.0f && (dy == 0.0f || u == 0.0f) && in_range);
}

// ---- RMSNorm output ------------------------------------------------------------
// out = T(x * rstd * w).  fp32: fl(fl(x*fl(rstd))*w) is within 3 * 2^-24
// relative of the exact product (three roundings), i.e. at most 3 fp32 ulps; 4 is used.
constexpr std::uint32_t kScaleUlps = 4;

template <typename T>
__device__ __forceinline__ typename Elem<T>::store_t scale_one(typename Elem<T>::store_t xs, float rs32, double rs64,
                                                                 typename Elem<T>::store_t ws) {
    using E = Elem<T>;
    if constexpr (sizeof(typename E::store_t) == 2) {
        const float x = E::to_f32(xs), w = E::to_f32(ws);
        const float y = x * rs32 * w;
        if (__builtin_expect(narrow_is_safe<T>(y, kScaleUlps), 1)) return E::from_f32_finite(y);
        if (y == 0.0f && (x == 0.0f || w == 0.0f)) return E::from_f32(y);  // exact signed zero
        return E::from_f64(static_cast<double>(x) * rs64 * static_cast<double>(w));
    } else {
        return E::from_f64(E::to_f64(xs) * rs64 * E::to_f64(ws));
    }
}


// Eight 16-bit elements at once (one 16-byte vector of x and of w), fast tier
// only, straight-line: returns the packed fp32-path results and sets `fix` when
// any element sits next to a rounding boundary or outside the normal range.
// The caller passes flagged vectors through scale_vec16_fix before storing.
template <typename T>
__device__ __forceinline__ u32x4 scale_vec16_fast(u32x4 xv, u32x4 wv, float rs32, bool& fix) {
    using E = Elem<T>;
    static_assert(sizeof(typename E::store_t) == 2, "16-bit dtypes only");
    // distance of the dropped field from the rounding boundary, biased so that
    // "within kScaleUlps" reads (field + bias) & mask <= 2*kScaleUlps; the
    // smallest of the eight decides for the vector
    constexpr std::uint32_t kBias = kScaleUlps - Narrow16<T>::kHalf;
    u32x4 o;
    float amin = 1.0f, amax = 1.0f;
    std::uint32_t dmin = 0xFFFFu;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const float y0 = E::to_f32(static_cast<std::uint16_t>(xv[p])) * rs32 * E::to_f32(static_cast<std::uint16_t>(wv[p]));
        const float y1 = E::to_f32(static_cast<std::uint16_t>(xv[p] >> 16)) * rs32 * E::to_f32(static_cast<std::uint16_t>(wv[p] >> 16));
        const std::uint32_t d0 = (__builtin_bit_cast(std::uint32_t, y0) + kBias) & Narrow16<T>::kMask;
        const std::uint32_t d1 = (__builtin_bit_cast(std::uint32_t, y1) + kBias) & Narrow16<T>::kMask;
        dmin = min(dmin, min(d0, d1));
        amin = fminf(amin, fminf(fabsf(y0), fabsf(y1)));
        amax = fmaxf(amax, fmaxf(fabsf(y0), fabsf(y1)));
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        if constexpr (sizeof(T) == sizeof(bf16_t) && __is_same(T, bf16_t)) {
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            o[p] = __builtin_bit_cast(std::uint32_t, __builtin_convertvector((f32x2){y0, y1}, bf16x2));
        } else {
            typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
            o[p] = __builtin_bit_cast(std::uint32_t, __builtin_convertvector((f32x2){y0, y1}, f16x2));
        }
    }
    fix = (dmin <= 2 * kScaleUlps) || !(amin >= Narrow16<T>::kMinNormal && amax <= Narrow16<T>::kMaxFinite);
    return o;
}

// Replaces the elements of one result vector whose fp32 value was not safe to
// narrow with the exact fp64 product.  Rare (about one vector in a thousand
// per lane), so it is written as a rolled loop over the 8 elements: one exact
// product is live at a time and the hot loop keeps its registers.
template <typename T>
__device__ __forceinline__ u32x4 scale_vec16_fix(u32x4 xv, u32x4 wv, u32x4 o, float rs32, double rs64) {
    using E = Elem<T>;
#pragma unroll 1
    for (int j = 0; j < 8; ++j) {
        const int p = j >> 1, sh = (j & 1) * 16;
        const std::uint16_t xs = static_cast<std::uint16_t>(xv[p] >> sh), ws = static_cast<std::uint16_t>(wv[p] >> sh);
        const float x = E::to_f32(xs), w = E::to_f32(ws);
        const float y = x * rs32 * w;
        if (narrow_is_safe<T>(y, kScaleUlps)) continue;
        const bool zero = (y == 0.0f) && (x == 0.0f || w == 0.0f);  // an exact signed zero needs no fp64
        const std::uint32_t r = zero ? E::from_f32(y) : E::from_f64(static_cast<double>(x) * rs64 * static_cast<double>(w));
        o[p] = (o[p] & ~(0xFFFFu << sh)) | (r << sh);
    }
    return o;
}

}  // namespace paras
