// Device-side helpers for gfx950: storage-type conversions with the rounding
// the reference's host engine has, 16-byte vector access, and wavefront
// (64-lane) reductions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace paras {

constexpr int kWave = 64;

// ---- storage types ---------------------------------------------------------
// Storage is raw bits; arithmetic happens in float or double.
struct bf16_t { std::uint16_t bits; };
struct f16_t  { std::uint16_t bits; };

typedef float    float4_t  __attribute__((ext_vector_type(4)));
typedef float    float16_t __attribute__((ext_vector_type(16)));
typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef std::uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16   bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8  __attribute__((ext_vector_type(8)));
typedef short    i16x4  __attribute__((ext_vector_type(4)));

// float -> bf16 bits, round to nearest even; NaN becomes 0x7FC0 (what
// c10::BFloat16's round_to_nearest_even produces on the host).
__device__ __forceinline__ std::uint16_t f32_to_bf16_bits(float f) {
    const std::uint32_t u = __builtin_bit_cast(std::uint32_t, f);
    if (f != f) return 0x7FC0;
    return static_cast<std::uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(std::uint16_t b) {
    return __builtin_bit_cast(float, static_cast<std::uint32_t>(b) << 16);
}
// float -> half as v_cvt_f16_f32 rounds (to nearest even).  The value is made opaque first: left
// to itself the compiler fuses a preceding fp32 multiply into v_fma_mixlo_f16 with a +0 addend,
// which turns a product of -0 into +0.  A NaN keeps its payload here; the host's c10::Half writes
// sign | 0x7E00 (f32_to_f16_bits_host below).
__device__ __forceinline__ std::uint16_t f32_to_f16_bits(float f) {
    asm("" : "+v"(f));
    const _Float16 h = static_cast<_Float16>(f);
    return __builtin_bit_cast(std::uint16_t, h);
}
__device__ __forceinline__ std::uint16_t f32_to_f16_bits_host(float f) {
    const std::uint16_t h = f32_to_f16_bits(f);
    const std::uint32_t u = __builtin_bit_cast(std::uint32_t, f);
    return f != f ? static_cast<std::uint16_t>(((u >> 16) & 0x8000u) | 0x7E00u) : h;
}
__device__ __forceinline__ float f16_bits_to_f32(std::uint16_t b) {
    return static_cast<float>(__builtin_bit_cast(_Float16, b));
}

// Per-dtype traits: `store_t` is what sits in HBM.
template <typename T> struct Elem;
template <> struct Elem<float> {
    using store_t = float;
    static constexpr int kVec = 4;  // elements per 16-byte access
    __device__ static __forceinline__ float  to_f32(float v) { return v; }
    __device__ static __forceinline__ double to_f64(float v) { return static_cast<double>(v); }
    __device__ static __forceinline__ float  from_f32(float v) { return v; }
    // double -> T exactly as static_cast<float>(double) on the host.
    __device__ static __forceinline__ float  from_f64(double v) { return static_cast<float>(v); }
};
template <> struct Elem<double> {
    using store_t = double;
    static constexpr int kVec = 2;
    __device__ static __forceinline__ float  to_f32(double v) { return static_cast<float>(v); }
    __device__ static __forceinline__ double to_f64(double v) { return v; }
    __device__ static __forceinline__ double from_f32(float v) { return static_cast<double>(v); }
    __device__ static __forceinline__ double from_f64(double v) { return v; }
};
template <> struct Elem<bf16_t> {
    using store_t = std::uint16_t;
    static constexpr int kVec = 8;
    __device__ static __forceinline__ float  to_f32(std::uint16_t v) { return bf16_bits_to_f32(v); }
    __device__ static __forceinline__ double to_f64(std::uint16_t v) { return static_cast<double>(bf16_bits_to_f32(v)); }
    __device__ static __forceinline__ std::uint16_t from_f32(float v) { return f32_to_bf16_bits(v); }
    // Same rounding through v_cvt_pk_bf16_f32, for values known not to be NaN
    // (the hardware keeps a NaN's payload, the host canonicalises it).
    __device__ static __forceinline__ std::uint16_t from_f32_finite(float v) {
        return __builtin_bit_cast(std::uint16_t, static_cast<__bf16>(v));
    }
    // The host path converts double -> float -> bf16 (c10::BFloat16 has only a
    // float constructor), i.e. two roundings; keep both.
    __device__ static __forceinline__ std::uint16_t from_f64(double v) { return f32_to_bf16_bits(static_cast<float>(v)); }
};
template <> struct Elem<f16_t> {
    using store_t = std::uint16_t;
    static constexpr int kVec = 8;
    __device__ static __forceinline__ float  to_f32(std::uint16_t v) { return f16_bits_to_f32(v); }
    __device__ static __forceinline__ double to_f64(std::uint16_t v) { return static_cast<double>(f16_bits_to_f32(v)); }
    __device__ static __forceinline__ std::uint16_t from_f32(float v) { return f32_to_f16_bits_host(v); }
    // for values known not to be NaN
    __device__ static __forceinline__ std::uint16_t from_f32_finite(float v) { return f32_to_f16_bits(v); }
    // Two roundings as on the host (double -> float -> half); the conversion to half keeps its
    // input opaque, so the compiler cannot merge them into one double -> half rounding.
    __device__ static __forceinline__ std::uint16_t from_f64(double v) { return f32_to_f16_bits_host(static_cast<float>(v)); }
};

// ---- wavefront reductions ----------------------------------------------------
// Butterfly over all 64 lanes; every lane ends with the full result.
template <typename T, typename Op>
__device__ __forceinline__ T wave_allreduce(T v, Op op) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, kWave));
    return v;
}
// Sum of a double over the 64 lanes, every lane gets the result.  The generic butterfly
// above goes through the LDS crossbar (ds_bpermute) twelve times in a dependent chain; this one
// stays in the VALU: four DPP exchanges inside each row of 16 lanes (quad swaps, then the
// half-row and row mirrors, which pair up equal partial sums), then the four row sums are read
// with v_readlane and added.
template <int kCtrl>
__device__ __forceinline__ double dpp_move_f64(double v) {
    const std::uint64_t b = __builtin_bit_cast(std::uint64_t, v);
    const int lo = static_cast<int>(b), hi = static_cast<int>(b >> 32);
    const int lo2 = __builtin_amdgcn_update_dpp(lo, lo, kCtrl, 0xf, 0xf, false);
    const int hi2 = __builtin_amdgcn_update_dpp(hi, hi, kCtrl, 0xf, 0xf, false);
    return __builtin_bit_cast(double, (static_cast<std::uint64_t>(static_cast<std::uint32_t>(hi2)) << 32) |
                                          static_cast<std::uint32_t>(lo2));
}
__device__ __forceinline__ double readlane_f64(double v, int lane) {
    const std::uint64_t b = __builtin_bit_cast(std::uint64_t, v);
    const std::uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(b), lane);
    const std::uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(b >> 32), lane);
    return __builtin_bit_cast(double, (static_cast<std::uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ double wave_sum(double v) {
    v += dpp_move_f64<0xB1>(v);    // quad_perm [1,0,3,2]: lane ^ 1
    v += dpp_move_f64<0x4E>(v);    // quad_perm [2,3,0,1]: lane ^ 2
    v += dpp_move_f64<0x141>(v);   // row_half_mirror: the other quad of the half row
    v += dpp_move_f64<0x140>(v);   // row_mirror: the other half of the row
    return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}
__device__ __forceinline__ float wave_sum(float v) {
    return wave_allreduce(v, [](float a, float b) { return a + b; });
}
__device__ __forceinline__ float wave_max(float v) {
    return wave_allreduce(v, [](float a, float b) { return fmaxf(a, b); });
}

// ---- workgroup barrier for LDS traffic only -----------------------------------
// __syncthreads() carries a release fence over every address space: the wave waits for all of
// its global loads and stores in flight before it meets the others, which serialises a loop that
// requested the next row from memory before reducing the current one.  This barrier orders LDS
// accesses only (s_waitcnt lgkmcnt(0); s_barrier): use it where the data exchanged lives in LDS.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- 16-byte global access ---------------------------------------------------
__device__ __forceinline__ u32x4 load16(const void* p) {
    return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ void store16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
// Non-temporal variants for data touched once: keep streams out of L2's way.
__device__ __forceinline__ u32x4 load16_nt(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void store16_nt(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

}  // namespace paras
