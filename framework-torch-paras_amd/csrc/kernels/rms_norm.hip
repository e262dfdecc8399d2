// Fused RMSNorm forward/backward for gfx950.
//
// Arithmetic follows the reference's host engine (csrc/ops/fused_ops.cpp:67-85,
// 105-156): everything is evaluated in fp64 and narrowed once to the tensor
// dtype (double -> float -> T).
//
// Forward: one 256-thread workgroup per row (grid = rows, so tens of
// thousands of independent workgroups keep HBM requests in flight).  Each
// thread owns NV 16-byte vectors of the row, loaded once with non-temporal
// loads and kept in registers between the sum-of-squares pass and the scaling
// pass; the four wave sums meet in LDS.  The sum of squares and rstd are fp64
// (the fp32 rstd output then matches the host bit for bit); the scaled outputs
// of 16-bit tensors take the fp32 fast tier of kernels/swiglu_math.h and fall
// back to the fp64 product only next to a rounding boundary, so they too are
// bit-identical to the host engine's.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/swiglu_math.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

// Sum over the workgroup; result valid in every thread.  `slots` is LDS of 2 * kWavesPerBlock
// doubles used as two alternating sets: a call uses set `parity & 1`, so the readers of one call
// never race with the writers of the next and a single barrier per call is enough (the set is
// reused only two calls later, with this call's barrier in between).
template <int NW = kWavesPerBlock>
__device__ __forceinline__ double block_sum(double v, double* slots, int parity) {
    v = wave_sum(v);
    if constexpr (NW == 1) return v;
    double* set = slots + (parity & 1) * NW;
    if ((threadIdx.x & (kWave - 1)) == 0) set[threadIdx.x / kWave] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += set[i];
    return t;
}

// The same for a number of waves known only at run time (sets of 16).
__device__ __forceinline__ double block_sum_any(double v, double* slots, int parity, int nw) {
    v = wave_sum(v);
    double* set = slots + (parity & 1) * 16;
    if ((threadIdx.x & (kWave - 1)) == 0) set[threadIdx.x / kWave] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < nw; ++i) t += set[i];
    return t;
}

// 1/sqrt(v) in fp64 from the hardware estimate and two Newton steps (error of a
// few 1e-16 relative: the fp32 rstd and every narrowed output are what the
// correctly rounded 1.0/sqrt(v) gives, since neither can see the last bit of
// a double).  Zero, infinite, NaN and subnormal arguments take the plain form.
__device__ __forceinline__ double rsqrt_f64(double v) {
    if (!(v > 1e-300 && v < 1e300)) return 1.0 / sqrt(v);
    double r = __builtin_amdgcn_rsq(v);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const double e = fma(-v * r, r, 1.0);
        r = fma(0.5 * r, e, r);
    }
    return r;
}

// Register-resident row: H == vectors per row * kVec, vectors per row <= BLOCK*NV.  The workgroup is
// sized to the row (128 threads for a row of 1024 16-bit elements, 1024 for one of 16384), at most two
// vectors per thread: four need more than the 64 registers that eight waves per SIMD leave.
// PIPE (short rows): a workgroup walks many rows and asks for its next row before it works on the
// current one -- a workgroup per row of 2 or 4 KB is bound by the rate at which workgroups start.
// BLOCK = 0: the workgroup size is whatever the launch says (a multiple of 64 up to 1024), for rows
// that would leave much of a power-of-two workgroup idle (5120 elements: 320 threads).
// Waves per SIMD the kernel is compiled for: eight (64 registers), except that the walking form
// with two vectors per thread keeps a second row in registers, which only bf16 fits into 64 (the
// others would park the row they have just asked for in scratch memory, i.e. wait for it at once).
template <typename T, int NV, bool PIPE>
constexpr int fwd_waves_per_simd() {
    if (!PIPE || NV < 2 || __is_same(T, bf16_t)) return 8;
    return __is_same(T, f16_t) ? 6 : 4;
}
template <typename T, int NV, int BLOCK, bool PIPE = false>
__global__ __launch_bounds__((BLOCK == 0 ? 1024 : BLOCK), (fwd_waves_per_simd<T, NV, PIPE>())) void rms_norm_fwd_vec(
    const typename Elem<T>::store_t* __restrict__ x, const typename Elem<T>::store_t* __restrict__ w,
    typename Elem<T>::store_t* __restrict__ out, float* __restrict__ rstd, long rows, int H,
    double eps, double inv_h) {
    using E = Elem<T>;
    using S = typename E::store_t;
    constexpr int V = E::kVec;
    __shared__ double slots[2 * ((BLOCK == 0 ? 1024 : BLOCK) / kWave)];
    const int block = BLOCK == 0 ? static_cast<int>(blockDim.x) : BLOCK;

    const int nvec = H / V;  // 16-byte vectors per row
    u32x4 wv[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * block;
        if (c < nvec) wv[i] = load16(w + static_cast<long>(c) * V);  // shared by every row: an L2 hit
    }
    // A NaN result must come out as the host's 16-bit types write it, which the fast tier's
    // conversion instructions do not do, and its range test does not see a NaN (min / max skip
    // them).  NaNs can only come from a weight that is not finite or from a row whose rstd is
    // not an ordinary positive number (a NaN or an infinity in the row, or a row of zeros with
    // eps = 0): both are known without looking at the elements.
    bool w_odd[NV];
    if constexpr (sizeof(S) == 2) {
        constexpr std::uint32_t kExp = __is_same(T, bf16_t) ? 0x7F80u : 0x7C00u;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            w_odd[i] = false;
            const int c = threadIdx.x + i * block;
            if (c < nvec) {
#pragma unroll
                for (int p = 0; p < 4; ++p)
                    w_odd[i] = w_odd[i] || ((wv[i][p] & kExp) == kExp) || (((wv[i][p] >> 16) & kExp) == kExp);
            }
        }
    }
    int sum_calls = 0;
    auto load_row = [&](long r, u32x4 (&dst)[NV]) {
        const S* xr = x + r * H;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * block;
            if (c < nvec) dst[i] = load16_nt(xr + static_cast<long>(c) * V);
        }
    };
    u32x4 xv[NV], xn[NV];
    if (PIPE && blockIdx.x < rows) load_row(blockIdx.x, xv);
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        S* outr = out + r * H;
        if constexpr (PIPE) {
            if (r + gridDim.x < rows) load_row(r + gridDim.x, xn);
        } else {
            load_row(r, xv);
        }
        double ss = 0.0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * block;
            if (c < nvec) {
                const S* e = reinterpret_cast<const S*>(&xv[i]);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const double v = E::to_f64(e[j]);
                    ss = fma(v, v, ss);
                }
            }
        }
        if constexpr (BLOCK == 0) ss = block_sum_any(ss, slots, sum_calls++, block / kWave);
        else ss = block_sum<(BLOCK == 0 ? 1 : BLOCK) / kWave>(ss, slots, sum_calls++);
        // 16-bit tensors: mean by the reciprocal and the refined rsqrt (outputs
        // cannot see the difference); fp32 / fp64 tensors: the host's own form.
        const double rs = sizeof(S) == 2 ? rsqrt_f64(fma(ss, inv_h, eps)) : 1.0 / sqrt(ss / static_cast<double>(H) + eps);
        const float rs32 = static_cast<float>(rs);
        if (threadIdx.x == 0) rstd[r] = rs32;
        if constexpr (sizeof(S) == 2) {
            const bool row_odd = !(rs32 > 0.0f && rs32 <= 3.4028234663852886e38f);
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = threadIdx.x + i * block;
                if (c < nvec) {
                    bool fix;
                    u32x4 o = scale_vec16_fast<T>(xv[i], wv[i], rs32, fix);
                    fix = fix || row_odd || w_odd[i];
                    if (__builtin_expect(fix, 0)) o = scale_vec16_fix<T>(xv[i], wv[i], o, rs32, rs);
                    store16_nt(outr + static_cast<long>(c) * V, o);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = threadIdx.x + i * block;
                if (c < nvec) {
                    const S* e  = reinterpret_cast<const S*>(&xv[i]);
                    const S* we = reinterpret_cast<const S*>(&wv[i]);
                    u32x4 o;
                    S* oe = reinterpret_cast<S*>(&o);
#pragma unroll
                    for (int j = 0; j < V; ++j) oe[j] = scale_one<T>(e[j], rs32, rs, we[j]);
                    store16_nt(outr + static_cast<long>(c) * V, o);
                }
            }
        }
        if constexpr (PIPE) {
#pragma unroll
            for (int i = 0; i < NV; ++i) xv[i] = xn[i];
        }
    }
}

// Rows of at most 64 vectors (per-head norms: 128 elements): TPR lanes per row, 64 / TPR rows per
// wave, no LDS and no barrier; the sum of squares meets over the row's lanes by exchanges inside the
// wave.  Persistent, the next group of rows requested before the current one is worked on.
template <typename T, int TPR>
__global__ __launch_bounds__(256, 8) void rms_norm_fwd_small(
    const typename Elem<T>::store_t* __restrict__ x, const typename Elem<T>::store_t* __restrict__ w,
    typename Elem<T>::store_t* __restrict__ out, float* __restrict__ rstd, long rows, int H,
    double eps, double inv_h) {
    using E = Elem<T>;
    using S = typename E::store_t;
    constexpr int V = E::kVec;
    constexpr int RPW = kWave / TPR;                      // rows per wave
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int sub = lane % TPR, rsel = lane / TPR;
    const int nvec = H / V;
    const bool have = sub < nvec;
    u32x4 wv = u32x4{0u, 0u, 0u, 0u};
    if (have) wv = load16(w + static_cast<long>(sub) * V);
    bool w_odd = false;
    if constexpr (sizeof(S) == 2) {
        constexpr std::uint32_t kExp = __is_same(T, bf16_t) ? 0x7F80u : 0x7C00u;
#pragma unroll
        for (int p = 0; p < 4; ++p) w_odd = w_odd || ((wv[p] & kExp) == kExp) || (((wv[p] >> 16) & kExp) == kExp);
    }
    const long step = static_cast<long>(gridDim.x) * (256 / kWave) * RPW;
    long r = (static_cast<long>(blockIdx.x) * (256 / kWave) + wave) * RPW + rsel;
    auto fetch = [&](long row) -> u32x4 {
        return (have && row < rows) ? load16_nt(x + row * H + static_cast<long>(sub) * V) : u32x4{0u, 0u, 0u, 0u};
    };
    u32x4 xv = fetch(r);
    for (; r - rsel < rows; r += step) {                  // wave-uniform: the wave's first row
        const u32x4 xn = fetch(r + step);
        const bool live = have && r < rows;
        double ss = 0.0;
        {
            const S* e = reinterpret_cast<const S*>(&xv);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const double v = E::to_f64(e[j]);
                ss = fma(v, v, ss);
            }
        }
#pragma unroll
        for (int off = TPR / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
        const double rs = sizeof(S) == 2 ? rsqrt_f64(fma(ss, inv_h, eps)) : 1.0 / sqrt(ss / static_cast<double>(H) + eps);
        const float rs32 = static_cast<float>(rs);
        if (sub == 0 && r < rows) rstd[r] = rs32;
        if (live) {
            S* outr = out + r * H + static_cast<long>(sub) * V;
            if constexpr (sizeof(S) == 2) {
                const bool row_odd = !(rs32 > 0.0f && rs32 <= 3.4028234663852886e38f);
                bool fix;
                u32x4 o = scale_vec16_fast<T>(xv, wv, rs32, fix);
                fix = fix || row_odd || w_odd;
                if (__builtin_expect(fix, 0)) o = scale_vec16_fix<T>(xv, wv, o, rs32, rs);
                store16_nt(outr, o);
            } else {
                const S* e  = reinterpret_cast<const S*>(&xv);
                const S* we = reinterpret_cast<const S*>(&wv);
                u32x4 o;
                S* oe = reinterpret_cast<S*>(&o);
#pragma unroll
                for (int j = 0; j < V; ++j) oe[j] = scale_one<T>(e[j], rs32, rs, we[j]);
                store16_nt(outr, o);
            }
        }
        xv = xn;
    }
}

// Any H, any alignment: scalar accesses, row re-read for the second pass.
template <typename T>
__global__ __launch_bounds__(kBlock) void rms_norm_fwd_any(
    const typename Elem<T>::store_t* __restrict__ x, const typename Elem<T>::store_t* __restrict__ w,
    typename Elem<T>::store_t* __restrict__ out, float* __restrict__ rstd, long rows, long H,
    double eps) {
    using E = Elem<T>;
    __shared__ double slots[2 * kWavesPerBlock];
    int sum_calls = 0;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        const auto* xr = x + r * H;
        auto* outr = out + r * H;
        double ss = 0.0;
        for (long j = threadIdx.x; j < H; j += kBlock) {
            const double v = E::to_f64(xr[j]);
            ss = fma(v, v, ss);
        }
        ss = block_sum(ss, slots, sum_calls++);
        const double rs = 1.0 / sqrt(ss / static_cast<double>(H) + eps);
        if (threadIdx.x == 0) rstd[r] = static_cast<float>(rs);
        for (long j = threadIdx.x; j < H; j += kBlock)
            outr[j] = E::from_f64(E::to_f64(xr[j]) * rs * E::to_f64(w[j]));
    }
}

// ---- backward ---------------------------------------------------------------
// dx: one workgroup per row (dot over the row, then the elementwise formula).
// dw: column sums over all rows.  Pass 1 writes, per row-slab, a partial fp64
// column sum into the workspace; pass 2 adds the slabs in slab order, so the
// result does not depend on scheduling.
template <typename T>
__global__ __launch_bounds__(kBlock) void rms_norm_bwd_dx(
    const typename Elem<T>::store_t* __restrict__ go, const typename Elem<T>::store_t* __restrict__ x,
    const typename Elem<T>::store_t* __restrict__ w, const float* __restrict__ rstd,
    typename Elem<T>::store_t* __restrict__ gx, long rows, long H) {
    using E = Elem<T>;
    __shared__ double slots[2 * kWavesPerBlock];
    int sum_calls = 0;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        const auto* gr = go + r * H;
        const auto* xr = x + r * H;
        auto* gxr = gx + r * H;
        const double rr = static_cast<double>(rstd[r]);
        double dot = 0.0;
        for (long j = threadIdx.x; j < H; j += kBlock)
            dot += E::to_f64(gr[j]) * E::to_f64(w[j]) * E::to_f64(xr[j]);
        dot = block_sum(dot, slots, sum_calls++);
        const double coef = rr * rr * rr / static_cast<double>(H);
        for (long j = threadIdx.x; j < H; j += kBlock) {
            const double gj = E::to_f64(gr[j]), wj = E::to_f64(w[j]), xj = E::to_f64(xr[j]);
            gxr[j] = E::from_f64(gj * wj * rr - coef * xj * dot);
        }
    }
}

constexpr int kDwSlabRows = 16;   // rows per partial column sum; the workspace is sized by it (the one-pass kernel may use fewer, larger groups)

template <typename T>
__global__ __launch_bounds__(kBlock) void rms_norm_bwd_dw_partial(
    const typename Elem<T>::store_t* __restrict__ go, const typename Elem<T>::store_t* __restrict__ x,
    const float* __restrict__ rstd, double* __restrict__ partial, long rows, long H) {
    using E = Elem<T>;
    // slabs along grid x (up to 2^31 - 1 of them), columns along grid y
    const long j = static_cast<long>(blockIdx.y) * kBlock + threadIdx.x;
    const long slab = blockIdx.x;
    if (j >= H) return;
    const long r0 = slab * kDwSlabRows;
    const long r1 = r0 + kDwSlabRows < rows ? r0 + kDwSlabRows : rows;
    double acc = 0.0;
    for (long r = r0; r < r1; ++r)
        acc += E::to_f64(go[r * H + j]) * E::to_f64(x[r * H + j]) * static_cast<double>(rstd[r]);
    partial[slab * H + j] = acc;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void rms_norm_bwd_dw_final(
    const double* __restrict__ partial, typename Elem<T>::store_t* __restrict__ gw, long slabs,
    long H) {
    using E = Elem<T>;
    const long j = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (j >= H) return;
    double acc = 0.0;
    for (long s = 0; s < slabs; ++s) acc += partial[s * H + j];
    gw[j] = E::from_f64(acc);
}

// ---- the row arithmetic of the one-pass backward kernels (one 16-byte vector of 8 elements) ----
// First half: widen g and x, accumulate the row's dot product and the column sums.
template <typename T>
__device__ __forceinline__ void bwd_vec_first(u32x4 gv, u32x4 xv, const double (&w64)[8], double rr, double& dot,
                                              double (&dw)[8], double (&g64)[8], double (&x64)[8]) {
    const std::uint16_t* ge = reinterpret_cast<const std::uint16_t*>(&gv);
    const std::uint16_t* xe = reinterpret_cast<const std::uint16_t*>(&xv);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        g64[j] = Elem<T>::to_f64(ge[j]);
        x64[j] = Elem<T>::to_f64(xe[j]);
        const double q = g64[j] * x64[j];
        dot = fma(q, w64[j], dot);
        dw[j] = fma(q, rr, dw[j]);
    }
}
// Second half: grad_x = T(g*w*rstd - x*(coef*dot)), narrowed double -> float -> T by the conversion
// instructions; a vector in which a NaN turns up (or infinities of both signs) is narrowed again in
// software, which canonicalises NaNs the way the host's types do.  The test is wave-uniform so that
// the software narrowing stays behind a branch instead of being evaluated and selected away.
template <typename T>
__device__ __forceinline__ u32x4 bwd_narrow_vec(const float (&y)[8]) {
    float nan_probe = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) nan_probe += y[j];
    u32x4 o;
    typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        if constexpr (__is_same(T, bf16_t)) {
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            o[p] = __builtin_bit_cast(std::uint32_t, __builtin_convertvector((f32x2){y[2 * p], y[2 * p + 1]}, bf16x2));
        } else {
            typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
            o[p] = __builtin_bit_cast(std::uint32_t, __builtin_convertvector((f32x2){y[2 * p], y[2 * p + 1]}, f16x2));
        }
    }
    if (__builtin_amdgcn_ballot_w64(nan_probe != nan_probe) != 0) {
        asm volatile("" ::: "memory");           // not to be evaluated ahead of the branch
        std::uint16_t* oe = reinterpret_cast<std::uint16_t*>(&o);
#pragma unroll
        for (int j = 0; j < 8; ++j) oe[j] = Elem<T>::from_f32(y[j]);
    }
    return o;
}
template <typename T>
__device__ __forceinline__ u32x4 bwd_vec_second(const double (&g64)[8], const double (&x64)[8], const double (&w64)[8], double rr,
                                                double cd) {
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = static_cast<float>(fma(g64[j] * w64[j], rr, -(x64[j] * cd)));
    return bwd_narrow_vec<T>(y);
}
// rstd^3 / H as the host forms it; the division is a multiplication when H is a power of two.
__device__ __forceinline__ double bwd_coef(double rr, int H, bool h_pow2, double inv_h) {
    double coef = rr * rr * rr;
    if (h_pow2) {
        coef *= inv_h;
    } else {
        asm volatile("" ::: "memory");           // keeps the division out of the power-of-two path
        coef = coef / static_cast<double>(H);
    }
    return coef;
}

// 16-bit tensors with 16-byte aligned rows of at most BLOCK*NV vectors: dx and the partial
// column sums in ONE pass over grad_out and x.  A workgroup owns every G-th row (G workgroups); each
// thread keeps the same NV vectors of every row (and of w, as doubles), so its 8*NV column sums
// live in registers across its rows, and the next row's vectors are requested before the current
// row's reduction.  Arithmetic in fp64, arranged so that every product that is exact on the host
// is exact here and every rounding the host makes is made here:
//   q = g*x (16-bit significands: exact), dot += q*w and dw += q*rstd (fma: the products are
//   exact in fp64 -- at most 40 significant bits -- so only the additions round, as on the host);
//   grad_x = fma(g*w, rstd, -(x * (coef*dot))): g*w*rstd is exact, so the one rounding of the
//   fma is the host's rounding of the difference; x*(coef*dot) differs from the host's
//   (coef*x)*dot in the last bit of a double at most, like the dot product's summation order.
// The result is narrowed double -> float -> T with the conversion instructions (two roundings to
// nearest even, as on the host); a vector in which a NaN turns up is narrowed again in software,
// which canonicalises NaNs the way the host's types do.
// One vector per thread needs ~100 registers: rows are spread over 256, 512 or 1024 threads.
// kFull: every thread of the workgroup owns a vector (H == 8 * BLOCK * NV).  Then no memory
// instruction sits under a lane mask and the compiler can count exactly which of them a wait has
// to cover: with a mask it waits, before the next row, for the row's own store as well.
// BLOCK == 0: the workgroup is as wide as the launch makes it (a whole number of waves, every
// thread with a vector of its own: rows of 512 * n elements that are not a power of two).
template <typename T, int NV, int BLOCK, bool kFull, int kTeams = 1>
__global__ __launch_bounds__(BLOCK == 0 ? 1024 : BLOCK * kTeams, 4) void rms_norm_bwd_fused(
    const std::uint16_t* __restrict__ go, const std::uint16_t* __restrict__ x, const std::uint16_t* __restrict__ w,
    const float* __restrict__ rstd, std::uint16_t* __restrict__ gx, double* __restrict__ partial, long rows, int H) {
    using E = Elem<T>;
    constexpr int V = 8;
    constexpr bool kDyn = BLOCK == 0;
    static_assert(!kDyn || (kTeams == 1 && kFull), "a workgroup of run-time width has one team and no idle thread");
    constexpr int kWaves = kDyn ? 16 : BLOCK / kWave;      // slots per sum (run-time width: the most there can be)
    __shared__ double slots[2 * kTeams * kWaves];
    __shared__ double team_dw[kTeams > 1 ? (kTeams - 1) * BLOCK * NV * V : 1];
    const int nvec = H / V;
    const int block = kDyn ? static_cast<int>(blockDim.x) : BLOCK;
    const int team = kTeams > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / (kDyn ? 1 : BLOCK)) : 0;
    const int tid = kTeams > 1 ? static_cast<int>(threadIdx.x) - team * BLOCK : static_cast<int>(threadIdx.x);
    const long slab = blockIdx.x;
    // Rows are dealt out round-robin: workgroup b takes rows b, b + G, b + 2G, ... (G workgroups),
    // so the rows in flight at any moment are neighbours in memory and spread over every memory
    // channel.  (A contiguous slab per workgroup puts the workgroups, which advance in step, a
    // constant 2^k bytes apart: 82 us instead of 76 for 16384 x 4096.)
    // With kTeams > 1 a workgroup is several teams of BLOCK threads, each with rows of its own (the
    // launcher sees to it that all teams have equally many): one partial sum for all of them, so
    // fewer to write and to add up.
    const long rstep = static_cast<long>(gridDim.x) * kTeams;
    const long r0 = slab * kTeams + team;
    const long r1 = rows;
    const double inv_h = 1.0 / static_cast<double>(H);   // only used where H is a power of two (exact)
    const bool h_pow2 = __builtin_amdgcn_readfirstlane((H & (H - 1)) == 0) != 0;
    bool have[NV];
    // One register set of row vectors: as soon as a row has been widened to doubles, the next row
    // is requested into the same registers (no copies between rows, and the loads have the row's
    // reduction, second half and store to arrive).
    u32x4 gs[NV], xs[NV];
    double w64[NV][V], dw[NV][V];
    auto request = [&](long r) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i]) {
                const int c = tid + i * block;
                gs[i] = load16_nt(go + r * H + static_cast<long>(c) * V);
                xs[i] = load16_nt(x + r * H + static_cast<long>(c) * V);
            }
    };
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = tid + i * block;
        have[i] = kFull || c < nvec;
        u32x4 wv = {0u, 0u, 0u, 0u};
        if (have[i]) wv = load16(w + static_cast<long>(c) * V);
        const std::uint16_t* we = reinterpret_cast<const std::uint16_t*>(&wv);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            w64[i][j] = E::to_f64(we[j]);
            dw[i][j] = 0.0;
        }
    }
    request(r0);
    int sum_calls = 0;
    float rstd_next = rstd[r0];
    auto do_row = [&](long r) __attribute__((always_inline)) {
        const float rstd_now = rstd_next;
        if (r + rstep < r1) rstd_next = rstd[r + rstep];     // requested a row ahead
        const double rr = static_cast<double>(rstd_now);
        double dot = 0.0;
        double g64[NV][V], x64[NV][V];     // stay in registers for the second half of the row
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i]) bwd_vec_first<T>(gs[i], xs[i], w64[i], rr, dot, dw[i], g64[i], x64[i]);
        if (r + rstep < r1) request(r + rstep);
        {   // sum over the workgroup; two alternating slot sets, so one barrier per row
            dot = wave_sum(dot);
            double* slot = slots + ((sum_calls++ & 1) * kTeams + team) * kWaves;
            if ((tid & (kWave - 1)) == 0) slot[tid / kWave] = dot;
            lds_barrier();   // not __syncthreads(): the loads requested above stay in flight across it
            dot = 0.0;
            if constexpr (kDyn) {
                const int nw = block / kWave;
                for (int i = 0; i < nw; ++i) dot += slot[i];
            } else if constexpr (kWaves <= 8) {
#pragma unroll
                for (int i = 0; i < kWaves; ++i) dot += slot[i];
            } else {
                // sixteen waves: four slots at a time, so that the slot values never hold more than
                // eight registers (all sixteen at once push the prefetched row out to scratch memory)
#pragma unroll
                for (int i = 0; i < kWaves; i += 4) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) dot += slot[i + u];
                    asm volatile("" : "+v"(dot) : : "memory");
                }
            }
        }
        const double cd = bwd_coef(rr, H, h_pow2, inv_h) * dot;
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i])
                store16_nt(gx + r * H + static_cast<long>(tid + i * block) * V, bwd_vec_second<T>(g64[i], x64[i], w64[i], rr, cd));
    };
    // The first row is written out in front of the loop: entered straight from the prologue, the
    // loop header would inherit "first loads pending" and the compiler's wait insertion would then
    // make every trip wait for all memory traffic in flight, the previous row's store included;
    // after a peeled row both ways into the header look alike (a row requested, a store in flight).
    do_row(r0);
    for (long r = r0 + rstep; r < r1; r += rstep) do_row(r);
    if constexpr (kTeams > 1) {
        // the other teams hand their column sums to team 0 through LDS; added in team order
        if (team > 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int j = 0; j < V; ++j) team_dw[((team - 1) * NV * V + i * V + j) * BLOCK + tid] = dw[i][j];
        }
        __syncthreads();
        if (team > 0) return;
#pragma unroll
        for (int tm = 1; tm < kTeams; ++tm)
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int j = 0; j < V; ++j) dw[i][j] += team_dw[((tm - 1) * NV * V + i * V + j) * BLOCK + tid];
    }
#pragma unroll
    for (int i = 0; i < NV; ++i)
        if (have[i]) {
            double* dst = partial + slab * H + static_cast<long>(tid + i * block) * V;
#pragma unroll
            for (int j = 0; j < V; ++j) dst[j] = dw[i][j];
        }
}

// Rows of 8193 to 16384 elements, 16-bit tensors: two vectors per thread of a 1024-thread workgroup,
// one workgroup per compute unit.  The registers of rms_norm_bwd_fused do not stretch to two
// vectors (weights and column sums as doubles, the widened row, the row asked for ahead), so the
// column sums live in LDS (128 KB: every thread adds into entries of its own, pairs of doubles 16
// bytes apart from lane to lane), the weights stay 16-bit and are widened at use, and g and x are
// widened twice, before and after the row's dot product is known.  Same arithmetic, same roundings.
template <typename T>
__global__ __launch_bounds__(1024, 4) void rms_norm_bwd_wide(
    const std::uint16_t* __restrict__ go, const std::uint16_t* __restrict__ x, const std::uint16_t* __restrict__ w,
    const float* __restrict__ rstd, std::uint16_t* __restrict__ gx, double* __restrict__ partial, long rows, int H) {
    using E = Elem<T>;
    typedef double f64x2 __attribute__((ext_vector_type(2)));
    constexpr int V = 8, NV = 2, BLOCK = 1024, kWaves = BLOCK / kWave;
    __shared__ f64x2 dw_lds[V / 2][NV * BLOCK];
    __shared__ double slots[2 * kWaves];
    const int tid = threadIdx.x;
    const int nvec = H / V;
    const double inv_h = 1.0 / static_cast<double>(H);
    const bool h_pow2 = __builtin_amdgcn_readfirstlane((H & (H - 1)) == 0) != 0;
    bool have[NV];
    u32x4 wv[NV], gs[NV], xs[NV], gn[NV], xn[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = tid + i * BLOCK;
        have[i] = c < nvec;
        wv[i] = have[i] ? load16(w + static_cast<long>(c) * V) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int p = 0; p < V / 2; ++p) dw_lds[p][c] = f64x2{0.0, 0.0};
    }
    auto request = [&](long r, u32x4 (&g)[NV], u32x4 (&xx)[NV]) __attribute__((always_inline)) {
        const std::uint16_t* gr = go + r * H;
        const std::uint16_t* xr = x + r * H;
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i]) {
                const unsigned at = static_cast<unsigned>(tid + i * BLOCK) * V;
                g[i] = load16_nt(gr + at);
                xx[i] = load16_nt(xr + at);
            }
    };
    const long rstep = gridDim.x;
    int sum_calls = 0;
    float rstd_carry = 0.0f;
    // One row from the register set (g, xx); the next row goes into the other set (gnext, xnext) as
    // soon as this one has arrived.  Two elements at a time, in element order, each pair finished
    // before the next is widened: all eight at once would not fit beside the row that is on its
    // way.  For the same reason the compiler must not keep widened values from one half of the row
    // to the other, or the widened weights from row to row: the packed registers are passed through
    // empty asm statements, after which it has to widen again.
    auto do_row = [&](long r, u32x4 (&g)[NV], u32x4 (&xx)[NV], u32x4 (&gnext)[NV], u32x4 (&xnext)[NV]) __attribute__((always_inline)) {
        auto forget = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int p = 0; p < 4; ++p) asm volatile("" : "+v"(g[i][p]), "+v"(xx[i][p]), "+v"(wv[i][p]));
        };
        double dot = 0.0;
        forget();                                            // waits for this row, so before the next one is asked for
        asm volatile("" : "+v"(rstd_carry));
        const double rr = static_cast<double>(rstd_carry);
        if (r + rstep < rows) {
            rstd_carry = rstd[r + rstep];                    // asked for with the row it belongs to
            request(r + rstep, gnext, xnext);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i]) {
                const int c = tid + i * BLOCK;
#pragma unroll
                for (int p = 0; p < V / 2; ++p) {
                    f64x2 d = dw_lds[p][c];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const std::uint32_t sh = 16 * h;
                        const double gd = E::to_f64(static_cast<std::uint16_t>(g[i][p] >> sh));
                        const double xd = E::to_f64(static_cast<std::uint16_t>(xx[i][p] >> sh));
                        const double wd = E::to_f64(static_cast<std::uint16_t>(wv[i][p] >> sh));
                        const double q = gd * xd;
                        dot = fma(q, wd, dot);
                        d[h] = fma(q, rr, d[h]);
                    }
                    dw_lds[p][c] = d;
                    asm volatile("" : "+v"(dot) : : "memory");
                }
            }
        {
            dot = wave_sum(dot);
            double* slot = slots + (sum_calls++ & 1) * kWaves;
            if ((tid & (kWave - 1)) == 0) slot[tid / kWave] = dot;
            lds_barrier();
            dot = 0.0;
#pragma unroll
            for (int i = 0; i < kWaves; i += 4) {
#pragma unroll
                for (int u = 0; u < 4; ++u) dot += slot[i + u];
                asm volatile("" : "+v"(dot) : : "memory");
            }
        }
        const double cd = bwd_coef(rr, H, h_pow2, inv_h) * dot;
        forget();
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (have[i]) {
                float y[V];
#pragma unroll
                for (int p = 0; p < V / 2; ++p) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const std::uint32_t sh = 16 * h;
                        const double gd = E::to_f64(static_cast<std::uint16_t>(g[i][p] >> sh));
                        const double xd = E::to_f64(static_cast<std::uint16_t>(xx[i][p] >> sh));
                        const double wd = E::to_f64(static_cast<std::uint16_t>(wv[i][p] >> sh));
                        y[2 * p + h] = static_cast<float>(fma(gd * wd, rr, -(xd * cd)));
                    }
                    asm volatile("" : "+v"(y[2 * p]), "+v"(y[2 * p + 1]));
                }
                store16_nt(gx + r * H + static_cast<unsigned>(tid + i * BLOCK) * V, bwd_narrow_vec<T>(y));
            }
    };
    long r = blockIdx.x;
    if (r < rows) {
        rstd_carry = rstd[r];
        request(r, gs, xs);
    }
    while (r < rows) {
        do_row(r, gs, xs, gn, xn);
        r += rstep;
        if (r >= rows) break;
        do_row(r, gn, xn, gs, xs);
        r += rstep;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i)
        if (have[i]) {
            const int c = tid + i * BLOCK;
            double* dst = partial + static_cast<long>(blockIdx.x) * H + static_cast<long>(c) * V;
#pragma unroll
            for (int p = 0; p < V / 2; ++p) {
                const f64x2 d = dw_lds[p][c];
                dst[2 * p] = d[0];
                dst[2 * p + 1] = d[1];
            }
        }
}

// Rows of at most 64 vectors (per-head norms: 128 elements), 16-bit tensors: TPR lanes per row,
// 64 / TPR rows per wave, each lane group walking rows of its own with the next one requested
// ahead; the row's dot product meets over its lanes by exchanges inside the wave, so the row loop
// has no LDS and no barrier.  The same arithmetic as rms_norm_bwd_fused; the column sums of the
// workgroup's 4 * 64 / TPR lane groups are added in LDS, in group order, into one partial sum.
template <typename T, int TPR>
__global__ __launch_bounds__(256, 4) void rms_norm_bwd_small(
    const std::uint16_t* __restrict__ go, const std::uint16_t* __restrict__ x, const std::uint16_t* __restrict__ w,
    const float* __restrict__ rstd, std::uint16_t* __restrict__ gx, double* __restrict__ partial, long rows, int H) {
    using E = Elem<T>;
    constexpr int V = 8, RPW = kWave / TPR, kGroups = (256 / kWave) * RPW;
    __shared__ double dw_lds[kGroups][TPR * V];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int sub = lane % TPR, rsel = lane / TPR;
    const int nvec = H / V;
    const bool have = sub < nvec;
    const double inv_h = 1.0 / static_cast<double>(H);
    const bool h_pow2 = __builtin_amdgcn_readfirstlane((H & (H - 1)) == 0) != 0;
    double w64[V], dw[V];
    {
        u32x4 wv = {0u, 0u, 0u, 0u};
        if (have) wv = load16(w + static_cast<long>(sub) * V);
        const std::uint16_t* we = reinterpret_cast<const std::uint16_t*>(&wv);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            w64[j] = E::to_f64(we[j]);
            dw[j] = 0.0;
        }
    }
    const long step = static_cast<long>(gridDim.x) * kGroups;
    long r = (static_cast<long>(blockIdx.x) * (256 / kWave) + wave) * RPW + rsel;
    auto fetch = [&](const std::uint16_t* base, long row) -> u32x4 {
        return (have && row < rows) ? load16_nt(base + row * H + static_cast<long>(sub) * V) : u32x4{0u, 0u, 0u, 0u};
    };
    u32x4 gv = fetch(go, r), xv = fetch(x, r);
    float rstd_now = r < rows ? rstd[r] : 0.0f;
    for (; r - rsel < rows; r += step) {                  // wave-uniform: the wave's first row
        const u32x4 gn = fetch(go, r + step), xn = fetch(x, r + step);
        const float rstd_nx = r + step < rows ? rstd[r + step] : 0.0f;
        const bool live = have && r < rows;
        const double rr = static_cast<double>(rstd_now);
        double dot = 0.0, g64[V], x64[V];
        if (live) bwd_vec_first<T>(gv, xv, w64, rr, dot, dw, g64, x64);
#pragma unroll
        for (int off = TPR / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, kWave);
        const double cd = bwd_coef(rr, H, h_pow2, inv_h) * dot;
        if (live) store16_nt(gx + r * H + static_cast<long>(sub) * V, bwd_vec_second<T>(g64, x64, w64, rr, cd));
        gv = gn;
        xv = xn;
        rstd_now = rstd_nx;
    }
    if (have) {
#pragma unroll
        for (int j = 0; j < V; ++j) dw_lds[wave * RPW + rsel][sub * V + j] = dw[j];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < H; c += 256) {
        double t = 0.0;
#pragma unroll 8
        for (int k = 0; k < kGroups; ++k) t += dw_lds[k][c];
        partial[static_cast<long>(blockIdx.x) * H + c] = t;
    }
}

// Column sums of the slabs in a fixed order: thread (column c of kDwFinalCols, lane l of
// kDwFinalLanes) adds slabs l, l + kDwFinalLanes, ... and the lane sums meet in LDS in lane order.
// A workgroup's columns are one 128-byte line of every slab row, so no line is fetched by two
// workgroups (on two XCDs, twice).
constexpr int kDwFinalCols = 16, kDwFinalLanes = 64;
template <typename T>
__global__ __launch_bounds__(kDwFinalLanes * kDwFinalCols) void rms_norm_bwd_dw_final_wide(
    const double* __restrict__ partial, typename Elem<T>::store_t* __restrict__ gw, long slabs, long H) {
    using E = Elem<T>;
    __shared__ double part[kDwFinalLanes][kDwFinalCols];
    const int c = threadIdx.x % kDwFinalCols, l = threadIdx.x / kDwFinalCols;
    const long j = static_cast<long>(blockIdx.x) * kDwFinalCols + c;
    double acc = 0.0;
    if (j < H) {
        // eight loads in flight at a time, added in slab order
        long sl = l;
        for (; sl + 7 * kDwFinalLanes < slabs; sl += 8 * kDwFinalLanes) {
            double v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(sl + u * kDwFinalLanes) * H + j];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; sl < slabs; sl += kDwFinalLanes) acc += partial[sl * H + j];
    }
    part[l][c] = acc;
    __syncthreads();
    if (l == 0 && j < H) {
        double t = 0.0;
#pragma unroll 8
        for (int k = 0; k < kDwFinalLanes; ++k) t += part[k][c];
        gw[j] = E::from_f64(t);
    }
}

int grid_for_rows(long rows) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto* st = DeviceContext::instance().device(dev);
    const long cus = st ? st->compute_units : 256;
    const long cap = cus * 256;  // far more workgroups than fit at once: the dispatcher keeps every CU fed
    return static_cast<int>(rows < cap ? rows : cap);
}

template <typename T>
int launch_fwd(const void* x, const void* w, void* out, float* rstd, long rows, long H,
               double eps, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    constexpr int V = Elem<T>::kVec;
    const auto* xs = static_cast<const S*>(x);
    const auto* ws = static_cast<const S*>(w);
    auto* os = static_cast<S*>(out);
    const int grid = grid_for_rows(rows);
    const bool aligned = (H % V == 0) && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                                           reinterpret_cast<uintptr_t>(out)) % 16 == 0);
    const long nvec = H / V;
#define PARAS_RMS_FWD(NV_, BLOCK_)                                                                                  \
    hipLaunchKernelGGL((rms_norm_fwd_vec<T, NV_, BLOCK_>), dim3(grid), dim3(BLOCK_), 0, s, xs, ws, os, rstd, rows, \
                       (int)H, eps, 1.0 / static_cast<double>(H))
    // short rows: sixteen workgroups' worth of rows per CU at a time, each workgroup walking its share
    int dev_id = 0;
    (void)hipGetDevice(&dev_id);
    auto* dst_ = DeviceContext::instance().device(dev_id);
    const long pipe_cap = (dst_ ? dst_->compute_units : 256) * 16;
    const int pgrid = static_cast<int>(rows < pipe_cap ? rows : pipe_cap);
#define PARAS_RMS_FWD_PIPE(NV_, BLOCK_)                                                                                   \
    hipLaunchKernelGGL((rms_norm_fwd_vec<T, NV_, BLOCK_, true>), dim3(pgrid), dim3(BLOCK_), 0, s, xs, ws, os, rstd, rows, \
                       (int)H, eps, 1.0 / static_cast<double>(H))
#define PARAS_RMS_FWD_SMALL(TPR_)                                                                                      \
    do {                                                                                                              \
        const long groups = (rows + (4 * (kWave / TPR_)) - 1) / (4 * (kWave / TPR_));                                 \
        const int sgrid = static_cast<int>(groups < pipe_cap ? groups : pipe_cap);                                    \
        hipLaunchKernelGGL((rms_norm_fwd_small<T, TPR_>), dim3(sgrid), dim3(256), 0, s, xs, ws, os, rstd, rows, (int)H, \
                           eps, 1.0 / static_cast<double>(H));                                                        \
    } while (0)
    if (aligned && nvec <= 8)         PARAS_RMS_FWD_SMALL(8);
    else if (aligned && nvec <= 16)   PARAS_RMS_FWD_SMALL(16);
    else if (aligned && nvec <= 32)   PARAS_RMS_FWD_SMALL(32);
    else if (aligned && nvec <= 64)   PARAS_RMS_FWD_SMALL(64);
    else if (aligned && nvec <= 128)  PARAS_RMS_FWD_PIPE(1, 128);
    else if (aligned && nvec <= 256)  PARAS_RMS_FWD_PIPE(1, 256);
#undef PARAS_RMS_FWD_PIPE
#undef PARAS_RMS_FWD_SMALL
    else if (aligned && nvec <= 2048) {
        int fit = static_cast<int>(((nvec + 1) / 2 + 63) / 64 * 64);     // threads that two vectors each fill
        if (fit > 256) fit = (fit + 127) / 128 * 128;      // an even number of waves: 5120 elements run 12 % faster on 384 threads than on 320
        // Wider than 256 threads: as many workgroups as are resident at once (eight waves per SIMD),
        // each walking its rows with the next one requested ahead.  With few, long rows a workgroup
        // per row leaves the chip half empty while the first rows arrive and the last ones drain
        // (8192 rows of 8192: 56 -> 52 us, 4096 of 16384: 59 -> 51 us); at 256 threads it is the
        // other way round (46 us against 47.5).
        const long fit_resident = (dst_ ? dst_->compute_units : 256) * ((4 * fwd_waves_per_simd<T, 2, true>()) / (fit / kWave));
        const int fgrid = static_cast<int>(rows < fit_resident ? rows : fit_resident);
        if (fit == 256)       PARAS_RMS_FWD(2, 256);
        else if (fit == 512)
            hipLaunchKernelGGL((rms_norm_fwd_vec<T, 2, 512, true>), dim3(fgrid), dim3(512), 0, s, xs, ws, os, rstd, rows, (int)H, eps,
                               1.0 / static_cast<double>(H));
        else if (fit == 1024)
            hipLaunchKernelGGL((rms_norm_fwd_vec<T, 2, 1024, true>), dim3(fgrid), dim3(1024), 0, s, xs, ws, os, rstd, rows, (int)H, eps,
                               1.0 / static_cast<double>(H));
        else if (fit > 256)
            hipLaunchKernelGGL((rms_norm_fwd_vec<T, 2, 0, true>), dim3(fgrid), dim3(fit), 0, s, xs, ws, os, rstd, rows, (int)H, eps,
                               1.0 / static_cast<double>(H));
        else
            hipLaunchKernelGGL((rms_norm_fwd_vec<T, 2, 0>), dim3(grid), dim3(fit), 0, s, xs, ws, os, rstd, rows, (int)H, eps,
                               1.0 / static_cast<double>(H));
    }
#undef PARAS_RMS_FWD
    else
        hipLaunchKernelGGL((rms_norm_fwd_any<T>), dim3(grid), dim3(kBlock), 0, s, xs, ws, os, rstd, rows, H, eps);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

template <typename T>
int launch_bwd(const void* go, const void* x, const void* w, const float* rstd, void* gx,
               void* gw, void* workspace, long rows, long H, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    long slabs = (rows + kDwSlabRows - 1) / kDwSlabRows;
    PARAS_REQUIRE(slabs <= 0x7fffffffL, "paras_rms_norm_bwd: too many rows");
    if constexpr (sizeof(S) == 2) {
        const bool aligned = (H % 8 == 0) && ((reinterpret_cast<uintptr_t>(go) | reinterpret_cast<uintptr_t>(x) |
                                               reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(gx)) % 16 == 0);
        const long nvec = H / 8;
        if (aligned && nvec <= 64) {
            // short rows: several rows per wave; as many workgroups as are resident at once (four
            // per compute unit), never more than the workspace has partial sums for
            int dev = 0;
            (void)hipGetDevice(&dev);
            auto* dst = DeviceContext::instance().device(dev);
            const long resident = (dst ? dst->compute_units : 256) * 4;
            const unsigned sgrid = static_cast<unsigned>(slabs < resident ? slabs : resident);
            auto* part = static_cast<double*>(workspace);
#define PARAS_BWD_SMALL(TPR_)                                                                                            \
    hipLaunchKernelGGL((rms_norm_bwd_small<T, TPR_>), dim3(sgrid), dim3(256), 0, s, static_cast<const std::uint16_t*>(go), \
                       static_cast<const std::uint16_t*>(x), static_cast<const std::uint16_t*>(w), rstd,                \
                       static_cast<std::uint16_t*>(gx), part, rows, (int)H)
            if (nvec <= 8)       PARAS_BWD_SMALL(8);
            else if (nvec <= 16) PARAS_BWD_SMALL(16);
            else if (nvec <= 32) PARAS_BWD_SMALL(32);
            else                 PARAS_BWD_SMALL(64);
#undef PARAS_BWD_SMALL
            PARAS_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL((rms_norm_bwd_dw_final_wide<T>), dim3(static_cast<unsigned>((H + kDwFinalCols - 1) / kDwFinalCols)), dim3(kDwFinalLanes * kDwFinalCols), 0, s,
                               part, static_cast<S*>(gw), static_cast<long>(sgrid), H);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
        if (aligned && nvec > 1024 && nvec <= 2048) {
            int dev = 0;
            (void)hipGetDevice(&dev);
            auto* dst = DeviceContext::instance().device(dev);
            const long cus = dst ? dst->compute_units : 256;
            const unsigned wgrid = static_cast<unsigned>(slabs < cus ? slabs : cus);     // one partial sum each: the workspace has `slabs`
            auto* part = static_cast<double*>(workspace);
            hipLaunchKernelGGL((rms_norm_bwd_wide<T>), dim3(wgrid), dim3(1024), 0, s, static_cast<const std::uint16_t*>(go),
                               static_cast<const std::uint16_t*>(x), static_cast<const std::uint16_t*>(w), rstd,
                               static_cast<std::uint16_t*>(gx), part, rows, (int)H);
            PARAS_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL((rms_norm_bwd_dw_final_wide<T>), dim3(static_cast<unsigned>((H + kDwFinalCols - 1) / kDwFinalCols)), dim3(kDwFinalLanes * kDwFinalCols), 0, s,
                               part, static_cast<S*>(gw), static_cast<long>(wgrid), H);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
        if (aligned && nvec <= 512 * 2) {
            const auto* g16 = static_cast<const std::uint16_t*>(go);
            const auto* x16 = static_cast<const std::uint16_t*>(x);
            const auto* w16 = static_cast<const std::uint16_t*>(w);
            auto* gx16 = static_cast<std::uint16_t*>(gx);
            auto* part = static_cast<double*>(workspace);
            // One workgroup per kDwSlabRows rows (the workspace is sized for that many partial sums)
            // up to what is resident at once (four waves per SIMD: 4, 2 or 1 workgroups per compute
            // unit): beyond that a workgroup takes more rows instead, so the partial sums to write and
            // to add up stop growing.
            int dev = 0;
            (void)hipGetDevice(&dev);
            auto* dst = DeviceContext::instance().device(dev);
            const long cus = dst ? dst->compute_units : 256;
            // rows of a whole number of waves that are not 256, 512 or 1024 vectors: a workgroup of
            // exactly that many threads
            const bool exact_width = nvec % kWave == 0 && nvec != kBlock && nvec != 512 && nvec != 1024;
            const long wg_waves = exact_width ? nvec / kWave : (nvec <= kBlock ? 4 : nvec <= 512 ? 8 : 16);
            const long resident = (16 / wg_waves) * cus;
            const bool plenty = slabs >= resident;
            if (plenty) slabs = resident;
            // Rows of 2048 or 4096 elements, plenty of them: workgroups of 1024 threads in teams of
            // one row's width (4 x 256 or 2 x 512), one workgroup per compute unit, when the rows
            // divide evenly among the teams.
            const bool teams = (nvec == 512 || nvec == kBlock) && plenty && rows % resident == 0;
            if (teams) slabs = cus;
            const dim3 grid(static_cast<unsigned>(slabs));
#define PARAS_BWD_LAUNCH(BLOCK_, FULL_) \
    hipLaunchKernelGGL((rms_norm_bwd_fused<T, 1, BLOCK_, FULL_>), grid, dim3(BLOCK_), 0, s, g16, x16, w16, rstd, gx16, part, rows, (int)H)
#define PARAS_BWD_LAUNCH_TEAMS(BLOCK_) \
    hipLaunchKernelGGL((rms_norm_bwd_fused<T, 1, BLOCK_, true, 1024 / BLOCK_>), grid, dim3(1024), 0, s, g16, x16, w16, rstd, gx16, part, rows, (int)H)
            if (exact_width)
                hipLaunchKernelGGL((rms_norm_bwd_fused<T, 1, 0, true>), grid, dim3(static_cast<unsigned>(nvec)), 0, s, g16, x16, w16, rstd, gx16, part, rows, (int)H);
            else if (teams && nvec == 512) PARAS_BWD_LAUNCH_TEAMS(512);
            else if (teams)          PARAS_BWD_LAUNCH_TEAMS(kBlock);
            else if (nvec == kBlock) PARAS_BWD_LAUNCH(kBlock, true);
            else if (nvec < kBlock)  PARAS_BWD_LAUNCH(kBlock, false);
            else if (nvec == 512)    PARAS_BWD_LAUNCH(512, true);
            else if (nvec < 512)     PARAS_BWD_LAUNCH(512, false);
            else if (nvec == 1024)   PARAS_BWD_LAUNCH(1024, true);   // rows of up to 8192 elements
            else                     PARAS_BWD_LAUNCH(1024, false);
#undef PARAS_BWD_LAUNCH_TEAMS
#undef PARAS_BWD_LAUNCH
            PARAS_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL((rms_norm_bwd_dw_final_wide<T>), dim3(static_cast<unsigned>((H + kDwFinalCols - 1) / kDwFinalCols)), dim3(kDwFinalLanes * kDwFinalCols), 0, s,
                               part, static_cast<S*>(gw), slabs, H);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
    }
    const unsigned gx_blocks = static_cast<unsigned>((H + kBlock - 1) / kBlock);
    PARAS_REQUIRE(gx_blocks <= 65535, "paras_rms_norm_bwd: rows of more than %d elements are not supported", 65535 * kBlock);   // before any launch
    hipLaunchKernelGGL((rms_norm_bwd_dx<T>), dim3(grid_for_rows(rows)), dim3(kBlock), 0, s,
                       static_cast<const S*>(go), static_cast<const S*>(x), static_cast<const S*>(w),
                       rstd, static_cast<S*>(gx), rows, H);
    PARAS_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((rms_norm_bwd_dw_partial<T>), dim3(static_cast<unsigned>(slabs), gx_blocks),
                       dim3(kBlock), 0, s, static_cast<const S*>(go), static_cast<const S*>(x), rstd,
                       static_cast<double*>(workspace), rows, H);
    PARAS_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((rms_norm_bwd_dw_final_wide<T>), dim3(static_cast<unsigned>((H + kDwFinalCols - 1) / kDwFinalCols)), dim3(kDwFinalLanes * kDwFinalCols), 0, s,
                       static_cast<const double*>(workspace), static_cast<S*>(gw), slabs, H);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_rms_norm_fwd(const void* x, const void* w, void* out, float* rstd, int64_t rows,
                       int64_t H, double eps, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && H >= 0, "paras_rms_norm_fwd: negative shape");
    if (rows == 0 || H == 0) return PARAS_OK;
    PARAS_REQUIRE(x && w && out && rstd, "paras_rms_norm_fwd: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    switch (dtype) {
        case PARAS_F32:  return launch_fwd<float>(x, w, out, rstd, rows, H, eps, s);
        case PARAS_F64:  return launch_fwd<double>(x, w, out, rstd, rows, H, eps, s);
        case PARAS_BF16: return launch_fwd<bf16_t>(x, w, out, rstd, rows, H, eps, s);
        case PARAS_F16:  return launch_fwd<f16_t>(x, w, out, rstd, rows, H, eps, s);
        default: return fail(PARAS_ERR_INVALID, "paras_rms_norm_fwd: unknown dtype %d", dtype);
    }
}

size_t paras_rms_norm_bwd_workspace(int64_t rows, int64_t H) {
    if (rows <= 0 || H <= 0) return 0;
    const int64_t slabs = (rows + paras::kDwSlabRows - 1) / paras::kDwSlabRows;
    return static_cast<size_t>(slabs) * static_cast<size_t>(H) * sizeof(double);
}

int paras_rms_norm_bwd(const void* grad_out, const void* x, const void* w, const float* rstd,
                       void* grad_x, void* grad_w, void* workspace, int64_t rows, int64_t H,
                       int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && H >= 0, "paras_rms_norm_bwd: negative shape");
    if (rows == 0 || H == 0) return PARAS_OK;
    PARAS_REQUIRE(grad_out && x && w && rstd && grad_x && grad_w && workspace,
                  "paras_rms_norm_bwd: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    switch (dtype) {
        case PARAS_F32:  return launch_bwd<float>(grad_out, x, w, rstd, grad_x, grad_w, workspace, rows, H, s);
        case PARAS_F64:  return launch_bwd<double>(grad_out, x, w, rstd, grad_x, grad_w, workspace, rows, H, s);
        case PARAS_BF16: return launch_bwd<bf16_t>(grad_out, x, w, rstd, grad_x, grad_w, workspace, rows, H, s);
        case PARAS_F16:  return launch_bwd<f16_t>(grad_out, x, w, rstd, grad_x, grad_w, workspace, rows, H, s);
        default: return fail(PARAS_ERR_INVALID, "paras_rms_norm_bwd: unknown dtype %d", dtype);
    }
}

}  // extern "C"
