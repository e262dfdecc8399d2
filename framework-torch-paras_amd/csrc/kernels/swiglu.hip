// Fused SwiGLU forward/backward and rotate_half for gfx950.
//
// out = silu(gate) * up with the host engine's rounding (see
// kernels/swiglu_math.h for how the fp64 definition is met at fp32 cost).
//
// Layout: flat contiguous streams, 16 bytes per lane per access, kUnroll
// independent non-temporal accesses per stream in flight per lane, one chunk
// per workgroup (tens of thousands of short workgroups stream better here
// than a persistent grid-stride loop).
#include <hip/hip_runtime.h>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/swiglu_math.h"

namespace paras {
namespace {

constexpr int kBlock  = 256;
constexpr int kUnroll = 4;  // 16-byte vectors per stream per lane per iteration

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_fwd_vec(
    const typename Elem<T>::store_t* __restrict__ gate, const typename Elem<T>::store_t* __restrict__ up,
    typename Elem<T>::store_t* __restrict__ out, long nvec) {
    using E = Elem<T>;
    using S = typename E::store_t;
    constexpr int V = E::kVec;
    const long stride = static_cast<long>(gridDim.x) * kBlock * kUnroll;
    for (long base = static_cast<long>(blockIdx.x) * kBlock * kUnroll + threadIdx.x; base < nvec;
         base += stride) {
        u32x4 gv[kUnroll], uv[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const long i = base + static_cast<long>(k) * kBlock;
            if (i < nvec) {
                gv[k] = load16_nt(gate + i * V);
                uv[k] = load16_nt(up + i * V);
            }
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const long i = base + static_cast<long>(k) * kBlock;
            if (i < nvec) {
                const S* ge = reinterpret_cast<const S*>(&gv[k]);
                const S* ue = reinterpret_cast<const S*>(&uv[k]);
                u32x4 o;
                S* oe = reinterpret_cast<S*>(&o);
#pragma unroll
                for (int j = 0; j < V; ++j) oe[j] = swiglu_one<T>(ge[j], ue[j]);
                store16_nt(out + i * V, o);
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_fwd_any(
    const typename Elem<T>::store_t* __restrict__ gate, const typename Elem<T>::store_t* __restrict__ up,
    typename Elem<T>::store_t* __restrict__ out, long first, long n) {
    const long stride = static_cast<long>(gridDim.x) * kBlock;
    for (long i = first + static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
        out[i] = swiglu_one<T>(gate[i], up[i]);
}

// Backward (csrc/ops/fused_ops.cpp:218-226), fp64 as on the host:
//   s = 1/(1+exp(-g)); dup = dy*g*s; dgate = dy*u*(s*(1+g*(1-s)))
template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_any(
    const typename Elem<T>::store_t* __restrict__ go, const typename Elem<T>::store_t* __restrict__ gate,
    const typename Elem<T>::store_t* __restrict__ up, typename Elem<T>::store_t* __restrict__ ggate,
    typename Elem<T>::store_t* __restrict__ gup, long n) {
    using E = Elem<T>;
    const long stride = static_cast<long>(gridDim.x) * kBlock;
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        const double dy = E::to_f64(go[i]);
        const double g  = E::to_f64(gate[i]);
        const double u  = E::to_f64(up[i]);
        const double s  = 1.0 / (1.0 + exp(-g));
        gup[i]   = E::from_f64(dy * g * s);
        ggate[i] = E::from_f64(dy * u * (s * (1.0 + g * (1.0 - s))));
    }
}

// 16-bit tensors, 16-byte aligned: eight elements per lane and access.  Every element goes through
// the fp32 fast tier; the few whose result sits next to a rounding boundary (or outside the fast
// tier's range) are collected in a bit mask and redone in fp64 in a loop that runs as often as the
// lane with the most of them needs -- usually not at all, sometimes once.
template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_vec(const std::uint16_t* __restrict__ go,
                                                         const std::uint16_t* __restrict__ gate,
                                                         const std::uint16_t* __restrict__ up,
                                                         std::uint16_t* __restrict__ ggate,
                                                         std::uint16_t* __restrict__ gup, long nvec) {
    using E = Elem<T>;
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < nvec; i += static_cast<long>(gridDim.x) * kBlock) {
        const u32x4 dv = load16_nt(go + i * 8), gv = load16_nt(gate + i * 8), uv = load16_nt(up + i * 8);
        const std::uint16_t* de = reinterpret_cast<const std::uint16_t*>(&dv);
        const std::uint16_t* ge = reinterpret_cast<const std::uint16_t*>(&gv);
        const std::uint16_t* ue = reinterpret_cast<const std::uint16_t*>(&uv);
        std::uint16_t og[8], ou[8];
        unsigned redo = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float yg, yu;
            bool ok_g, ok_u;
            swiglu_bwd_fast<T>(E::to_f32(de[j]), E::to_f32(ge[j]), E::to_f32(ue[j]), yg, yu, ok_g, ok_u);
            og[j] = E::from_f32_finite(yg);
            ou[j] = E::from_f32_finite(yu);
            redo |= (ok_g && ok_u) ? 0u : (1u << j);
        }
        while (redo != 0) {
            const int j = __builtin_ctz(redo);
            redo &= redo - 1;
            std::uint16_t d16 = 0, g16 = 0, u16 = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (k == j) { d16 = de[k]; g16 = ge[k]; u16 = ue[k]; }
            std::uint16_t xg, xu;
            swiglu_bwd_exact<T>(E::to_f32(d16), E::to_f32(g16), E::to_f32(u16), xg, xu);
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (k == j) { og[k] = xg; ou[k] = xu; }
        }
        u32x4 wg, wu;
#pragma unroll
        for (int p2 = 0; p2 < 4; ++p2) {
            wg[p2] = og[2 * p2] | (static_cast<std::uint32_t>(og[2 * p2 + 1]) << 16);
            wu[p2] = ou[2 * p2] | (static_cast<std::uint32_t>(ou[2 * p2 + 1]) << 16);
        }
        store16_nt(ggate + i * 8, wg);
        store16_nt(gup + i * 8, wu);
    }
}

// rotate_half (csrc/ops/fused_ops.cpp:254-263, 290-299): out[.., c] takes
// x[.., c+half] (negated for forward) when c < half, else x[.., c-half]
// (negated for backward).  Negation flips the sign bit, which is what
// -(double)v rounded back gives for every finite value and infinity; a NaN
// stays a NaN.
// A 16-bit NaN as the host writes it after its trip through double: bf16 0x7FC0, half sign | 0x7E00
// (kind 1 / 2; anything else passes through).
__device__ __forceinline__ std::uint32_t host_nan16(std::uint32_t h, int kind) {
    if (kind == 1) return (h & 0x7FFFu) > 0x7F80u ? 0x7FC0u : h;
    if (kind == 2) return (h & 0x7FFFu) > 0x7C00u ? ((h & 0x8000u) | 0x7E00u) : h;
    return h;
}
template <typename S>
__global__ __launch_bounds__(kBlock) void rotate_half_any(const S* __restrict__ x, S* __restrict__ out,
                                                          long n, long D, int backward, int nan_kind) {
    const long half = D / 2;
    const long stride = static_cast<long>(gridDim.x) * kBlock;
    constexpr S kSign = static_cast<S>(S{1} << (sizeof(S) * 8 - 1));
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        const long col = i % D;
        const bool first = col < half;
        const S v = x[first ? i + half : i - half];
        const bool negate = backward ? !first : first;
        S r = negate ? static_cast<S>(v ^ kSign) : v;
        // the negated half goes through double on the host and comes back as its 16-bit types
        // write a NaN; the other half is copied as it is
        if constexpr (sizeof(S) == 2) r = negate ? static_cast<S>(host_nan16(r, nan_kind)) : r;
        out[i] = r;
    }
}

// 16-bit elements, D a multiple of 16, 16-byte aligned: one 16-byte vector per lane, the
// partner vector sits half a row away, the sign flips are one XOR per register.
__global__ __launch_bounds__(kBlock) void rotate_half_vec16(const std::uint16_t* __restrict__ x,
                                                            std::uint16_t* __restrict__ out, long nvec,
                                                            int vec_per_row, int backward, int nan_kind) {
    const int half = vec_per_row / 2;
    const long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= nvec) return;
    const int col = static_cast<int>(i % vec_per_row);
    const bool first = col < half;
    u32x4 v = load16_nt(x + (first ? i + half : i - half) * 8);
    const bool negate = backward ? !first : first;
    if (negate) {
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] ^= 0x80008000u;
    }
    // The negated half goes through double on the host and comes back as its 16-bit types write
    // a NaN (the other half is copied as it is).  Rare, so behind a wave-uniform test: an exponent
    // field of all ones in any of the eight elements, i.e. a NaN or an infinity.
    const std::uint32_t exp_mask = nan_kind == 1 ? 0x7F807F80u : 0x7C007C00u;
    bool special = false;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const std::uint32_t e = v[k] & exp_mask;
        special = special || (e & 0xFFFFu) == (exp_mask & 0xFFFFu) || (e >> 16) == (exp_mask >> 16);
    }
    if (__builtin_amdgcn_ballot_w64(special && negate) != 0) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (negate) v[k] = host_nan16(v[k] & 0xFFFFu, nan_kind) | (host_nan16(v[k] >> 16, nan_kind) << 16);
    }
    store16_nt(out + i * 8, v);
}

int stream_grid(long work_items_per_block_iter, long total) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto* st = DeviceContext::instance().device(dev);
    const long cus = st ? st->compute_units : 256;
    const long cap = cus * 8;
    const long need = (total + work_items_per_block_iter - 1) / work_items_per_block_iter;
    const long g = need < cap ? need : cap;
    return static_cast<int>(g < 1 ? 1 : g);
}

template <typename T>
int launch_swiglu_fwd(const void* gate, const void* up, void* out, long n, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    constexpr int V = Elem<T>::kVec;
    const auto* g = static_cast<const S*>(gate);
    const auto* u = static_cast<const S*>(up);
    auto* o = static_cast<S*>(out);
    const bool aligned = ((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) |
                           reinterpret_cast<uintptr_t>(out)) % 16) == 0;
    long done = 0;
    if (aligned && n >= V) {
        const long nvec = n / V;
        long blocks = (nvec + kBlock * kUnroll - 1) / (kBlock * kUnroll);
        if (blocks > 0x7fffffffL) blocks = 0x7fffffffL;  // the kernel grid-strides beyond that
        hipLaunchKernelGGL((swiglu_fwd_vec<T>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, s, g, u, o, nvec);
        PARAS_HIP_TRY(hipGetLastError());
        done = nvec * V;
    }
    if (done < n) {
        hipLaunchKernelGGL((swiglu_fwd_any<T>), dim3(stream_grid(kBlock, n - done)), dim3(kBlock), 0, s, g,
                           u, o, done, n);
        PARAS_HIP_TRY(hipGetLastError());
    }
    return PARAS_OK;
}

template <typename T>
int launch_swiglu_bwd(const void* go, const void* gate, const void* up, void* ggate, void* gup, long n,
                      hipStream_t s) {
    using S = typename Elem<T>::store_t;
    const auto* d = static_cast<const S*>(go);
    const auto* g = static_cast<const S*>(gate);
    const auto* u = static_cast<const S*>(up);
    auto* og = static_cast<S*>(ggate);
    auto* ou = static_cast<S*>(gup);
    long done = 0;
    if constexpr (sizeof(S) == 2) {
        const bool aligned = ((reinterpret_cast<uintptr_t>(go) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) |
                               reinterpret_cast<uintptr_t>(ggate) | reinterpret_cast<uintptr_t>(gup)) % 16) == 0;
        if (aligned && n >= 8) {
            const long nvec = n / 8;
            long blocks = (nvec + kBlock - 1) / kBlock;
            if (blocks > 0x7fffffffL) blocks = 0x7fffffffL;  // the kernel grid-strides beyond that
            hipLaunchKernelGGL((swiglu_bwd_vec<T>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, s, d, g, u, og, ou, nvec);
            PARAS_HIP_TRY(hipGetLastError());
            done = nvec * 8;
        }
    }
    if (done < n) {
        hipLaunchKernelGGL((swiglu_bwd_any<T>), dim3(stream_grid(kBlock, n - done)), dim3(kBlock), 0, s, d + done, g + done,
                           u + done, og + done, ou + done, n - done);
        PARAS_HIP_TRY(hipGetLastError());
    }
    return PARAS_OK;
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(n >= 0, "paras_swiglu_fwd: negative size");
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(gate && up && out, "paras_swiglu_fwd: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    switch (dtype) {
        case PARAS_F32:  return launch_swiglu_fwd<float>(gate, up, out, n, s);
        case PARAS_F64:  return launch_swiglu_fwd<double>(gate, up, out, n, s);
        case PARAS_BF16: return launch_swiglu_fwd<bf16_t>(gate, up, out, n, s);
        case PARAS_F16:  return launch_swiglu_fwd<f16_t>(gate, up, out, n, s);
        default: return fail(PARAS_ERR_INVALID, "paras_swiglu_fwd: unknown dtype %d", dtype);
    }
}

int paras_swiglu_bwd(const void* grad_out, const void* gate, const void* up, void* grad_gate,
                     void* grad_up, int64_t n, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(n >= 0, "paras_swiglu_bwd: negative size");
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(grad_out && gate && up && grad_gate && grad_up, "paras_swiglu_bwd: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    switch (dtype) {
        case PARAS_F32:  return launch_swiglu_bwd<float>(grad_out, gate, up, grad_gate, grad_up, n, s);
        case PARAS_F64:  return launch_swiglu_bwd<double>(grad_out, gate, up, grad_gate, grad_up, n, s);
        case PARAS_BF16: return launch_swiglu_bwd<bf16_t>(grad_out, gate, up, grad_gate, grad_up, n, s);
        case PARAS_F16:  return launch_swiglu_bwd<f16_t>(grad_out, gate, up, grad_gate, grad_up, n, s);
        default: return fail(PARAS_ERR_INVALID, "paras_swiglu_bwd: unknown dtype %d", dtype);
    }
}

int paras_rotate_half(const void* x, void* out, int64_t rows, int64_t D, int backward, int dtype,
                      void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && D >= 0, "paras_rotate_half: negative shape");
    PARAS_REQUIRE(D % 2 == 0, "paras rotate_half: last dimension must be even");
    const long n = rows * D;
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(x && out, "paras_rotate_half: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    const dim3 grid(stream_grid(kBlock, n)), block(kBlock);
    switch (dtype) {
        case PARAS_F32:
            hipLaunchKernelGGL((rotate_half_any<uint32_t>), grid, block, 0, s, static_cast<const uint32_t*>(x),
                               static_cast<uint32_t*>(out), n, (long)D, backward, 0);
            break;
        case PARAS_F64:
            hipLaunchKernelGGL((rotate_half_any<uint64_t>), grid, block, 0, s, static_cast<const uint64_t*>(x),
                               static_cast<uint64_t*>(out), n, (long)D, backward, 0);
            break;
        case PARAS_BF16:
        case PARAS_F16:
            if (D % 16 == 0 && D / 8 <= 0x7fffffff && n / 8 <= 0x7fffffffL * kBlock &&
                ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
                const long nvec = n / 8;
                hipLaunchKernelGGL(rotate_half_vec16, dim3(static_cast<unsigned>((nvec + kBlock - 1) / kBlock)), block, 0, s,
                                   static_cast<const uint16_t*>(x), static_cast<uint16_t*>(out), nvec,
                                   static_cast<int>(D / 8), backward, dtype == PARAS_BF16 ? 1 : 2);
            } else {
                hipLaunchKernelGGL((rotate_half_any<uint16_t>), grid, block, 0, s, static_cast<const uint16_t*>(x),
                                   static_cast<uint16_t*>(out), n, (long)D, backward, dtype == PARAS_BF16 ? 1 : 2);
            }
            break;
        default: return fail(PARAS_ERR_INVALID, "paras_rotate_half: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // extern "C"
