// Pieces shared by the flash-attention forward kernels (sdpa_flash.hip: 32 queries per
// wavefront, two wavefronts per SIMD, every mask form; sdpa_flash_wide.hip: 64 queries per
// wavefront, one wavefront per SIMD, head size 128 without a user mask).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "core/device_math.h"

namespace paras {
namespace flash {

constexpr int kBN = 64;    // keys per tile

typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

struct FlashParams {
    const std::uint16_t* q;
    const std::uint16_t* k;
    const std::uint16_t* v;
    std::uint16_t*       out;
    float*               lse;
    long qs_b, qs_h, qs_l;  // element strides
    long ks_b, ks_h, ks_l;
    long vs_b, vs_h, vs_l;
    int  B, Hq, Hkv, Lq, Lk;
    int  n_qblocks;
    float scale_log2;  // scale * log2(e)
    float scale;
    // optional mask over [B, Hq, Lq, Lk] (element strides; 0 = broadcast): bytes (nonzero = attend)
    // or additive values of the tensor dtype
    const unsigned char* mask;
    long ms_b, ms_h, ms_q, ms_k;
    float score_scale; // the caller's scale as given; the masked variants apply it themselves and run with scale = 1
    unsigned magic_nq, magic_hq, magic_rep;   // ceil(2^32 / d) for d = n_qblocks, Hq, Hq / Hkv (set by the wide kernel's launcher)
};

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    // The same instruction with its register files chosen by hand (see sdpa_flash_wide.hip):
    // scores accumulate in VGPRs with the query operand in AGPRs, outputs accumulate in AGPRs.
    __device__ static __forceinline__ void score_first(float16_t& d, i16x8 a, i16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
    }
    __device__ static __forceinline__ void score_acc(float16_t& d, i16x8 a, i16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
    }
    __device__ static __forceinline__ void out_acc(float16_t& d, i16x8 a, u32x4 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(d) : "v"(a), "v"(b));
    }
    __device__ static __forceinline__ std::uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(std::uint32_t, __builtin_convertvector(v, bf16x2));
    }
};
template <> struct Mma<f16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ void score_first(float16_t& d, i16x8 a, i16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
    }
    __device__ static __forceinline__ void score_acc(float16_t& d, i16x8 a, i16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
    }
    __device__ static __forceinline__ void out_acc(float16_t& d, i16x8 a, u32x4 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(d) : "v"(a), "v"(b));
    }
    __device__ static __forceinline__ std::uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(std::uint32_t, __builtin_convertvector(v, f16x2));
    }
};

// Exchange between the two half-waves that share a query: v_permlane32_swap
// swaps lanes 32..63 of its first register with lanes 0..31 of its second.
// Fed the same value twice it leaves the lower half's value in every lane of
// the first register and the upper half's value in every lane of the second.
// Written as inline asm because the compiler's builtin for it returns the
// first result twice (seen with ROCm 7.2's hipcc); the s_nop pairs cover the
// VALU-write -> permlane-read and permlane-write -> VALU-read wait states the
// hazard recognizer cannot see inside an asm block.
__device__ __forceinline__ void half_swap(float x, float& lo, float& hi) {
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lo = a;
    hi = b;
}
__device__ __forceinline__ float half_swap_max(float x) {
    float lo, hi;
    half_swap(x, lo, hi);
    return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_swap_sum(float x) {
    float lo, hi;
    half_swap(x, lo, hi);
    return lo + hi;
}

// Workgroup index -> (batch * head, query tile, heaviest first): consecutive workgroup ids go to
// consecutive XCDs, so the heads are dealt to the XCDs in pairs and each XCD walks the query
// tiles of its pair from the last (longest under the causal rule) to the first.
__device__ __forceinline__ void map_workgroup(int idx, int BH, int nq, int& bh, int& qblock) {
    int qi;
    if (BH % 16 == 0) {
        const int xcd = idx & 7, j = idx >> 3;
        const int g = j / (2 * nq), r = j % (2 * nq);
        bh = (2 * g + (r & 1)) * 8 + xcd;
        qi = r >> 1;
    } else if (BH % 8 == 0) {
        const int xcd = idx & 7, j = idx >> 3;
        bh = (j / nq) * 8 + xcd;
        qi = j % nq;
    } else {
        bh = idx / nq;
        qi = idx % nq;
    }
    qblock = nq - 1 - qi;
}

// 64 queries per wavefront (sdpa_flash_wide.hip): head size 128, causal or unmasked.
constexpr int kWideBM = 256;   // queries per workgroup of that kernel
bool wide_supported(long B, long Hq, long Lq, long Lk, int D, int mask_kind, bool causal);
int  launch_flash_wide(FlashParams p, bool causal, bool is_bf16, hipStream_t s);

}  // namespace flash
}  // namespace paras
