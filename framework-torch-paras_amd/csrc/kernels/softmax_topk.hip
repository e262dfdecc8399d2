// Row softmax and row top-k on the device, with the reference host engine's
// arithmetic (csrc/ops/pointwise_ops.cpp:926-981 and :1292-1381):
//
//   softmax  per row, in fp64: m = max_j v_j; s = sum_j exp(v_j - m);
//            out_j = T_out( exp(v_j - m) / s ).  T_out is the input dtype, or
//            fp32 for 16-bit inputs when the caller asks (half_to_float).
//   top-k    the k largest (or smallest) of a row in sorted order, ties to the
//            lower index, found as the reference does: slot s takes the best
//            element that comes after slot s-1 in (value, index) order.
//            Comparisons are on the values widened to double, so they are
//            exact for every float dtype; indices are int64.
//
// Rows of up to 256 elements: one wave per row, the row in registers.  Longer rows: one
// workgroup per row; the softmax re-reads it from L2 between passes, the top-k keeps one
// candidate per thread and refreshes only the one that was taken (fp64 rows: a pass per slot).
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "paras_hip.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

__device__ __forceinline__ double wave_max_f64(double v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmax(v, __shfl_xor(v, off, kWave));
    return v;
}

// Any row length: three passes over the row (it stays in L2), kThreads threads per row -- 1024 for
// the long rows of which there are few (vocabulary-sized logits), so that a row has a CU's worth
// of wavefronts behind its fp64 exponentials.
template <typename TI, typename TO, int kThreads>
__global__ __launch_bounds__(kThreads) void softmax_rows_kernel(const typename Elem<TI>::store_t* __restrict__ x,
                                                                typename Elem<TO>::store_t* __restrict__ out, long n) {
    using EI = Elem<TI>;
    using EO = Elem<TO>;
    constexpr int kNW = kThreads / kWave;
    __shared__ double slots[kNW];
    const auto* xr = x + static_cast<long>(blockIdx.x) * n;
    auto* outr = out + static_cast<long>(blockIdx.x) * n;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;

    double m = -INFINITY;
    for (long j = threadIdx.x; j < n; j += kThreads) {
        const double v = EI::to_f64(xr[j]);
        if (v > m) m = v;                       // as the host: a NaN never replaces the max
    }
    m = wave_max_f64(m);
    if (lane == 0) slots[wave] = m;
    __syncthreads();
    m = slots[0];
#pragma unroll
    for (int i = 1; i < kNW; ++i) m = fmax(m, slots[i]);
    __syncthreads();

    double s = 0.0;
    for (long j = threadIdx.x; j < n; j += kThreads) s += exp(EI::to_f64(xr[j]) - m);
    s = wave_sum(s);
    if (lane == 0) slots[wave] = s;
    __syncthreads();
    s = 0.0;
#pragma unroll
    for (int i = 0; i < kNW; ++i) s += slots[i];

    for (long j = threadIdx.x; j < n; j += kThreads) outr[j] = EO::from_f64(exp(EI::to_f64(xr[j]) - m) / s);
}

// Rows of up to kBlock * EPT elements: the same, with each thread's exponentials kept in
// registers between the sum and the division (one fp64 exp per element instead of two, one read
// of the row instead of three).
template <typename TI, typename TO, int EPT>
__global__ __launch_bounds__(kBlock) void softmax_rows_reg_kernel(const typename Elem<TI>::store_t* __restrict__ x,
                                                                  typename Elem<TO>::store_t* __restrict__ out, int n) {
    using EI = Elem<TI>;
    using EO = Elem<TO>;
    __shared__ double slots[2][kWaves];
    const auto* xr = x + static_cast<long>(blockIdx.x) * n;
    auto* outr = out + static_cast<long>(blockIdx.x) * n;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    double v[EPT];
    double m = -INFINITY;
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int j = threadIdx.x + i * kBlock;
        v[i] = j < n ? EI::to_f64(xr[j]) : -INFINITY;
        if (j < n && v[i] > m) m = v[i];        // as the host: a NaN never replaces the max
    }
    m = wave_max_f64(m);
    if (lane == 0) slots[0][wave] = m;
    __syncthreads();
    m = slots[0][0];
#pragma unroll
    for (int i = 1; i < kWaves; ++i) m = fmax(m, slots[0][i]);
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int j = threadIdx.x + i * kBlock;
        v[i] = j < n ? exp(v[i] - m) : 0.0;
        sum += v[i];
    }
    sum = wave_sum(sum);
    if (lane == 0) slots[1][wave] = sum;
    __syncthreads();
    sum = 0.0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) sum += slots[1][i];
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int j = threadIdx.x + i * kBlock;
        if (j < n) outr[j] = EO::from_f64(v[i] / sum);
    }
}

// 16-bit and fp32 rows of up to 32768 elements in whole 16-byte pieces, 16-byte aligned, output in the
// input's dtype: the same arithmetic as softmax_rows_reg_kernel in fewer instructions (that kernel
// spends two thirds of its 113 per element on widening, narrowing and the tests of a ragged row).
// A thread takes NV pieces (eight 16-bit elements or four floats) with 16-byte loads and stores; the
// maximum is taken on floats (the widening is exact and v_max_f32 passes a NaN by, as the host's
// `v > m` does); the difference to it, the exponential, the sum and the division are in fp64 as
// before; 16-bit quotients are narrowed double -> float -> T by the conversion instructions when
// the sum is a positive finite number (every quotient then lies in [0, 1]), and with the host's NaN
// rules otherwise.  BLK threads per row (64, 128, 256 or 1024: the fewest that cover the row with
// at most 32 elements each, since every thread pays for its exponentials whether the row reaches
// it or not).
template <typename T, int NV, int BLK>
__global__ __launch_bounds__(BLK) void softmax_rows_vec_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                               typename Elem<T>::store_t* __restrict__ out, int n) {
    using E = Elem<T>;
    using S = typename E::store_t;
    constexpr int kBlock = BLK, kWaves = BLK / kWave;
    constexpr int EPV = 16 / static_cast<int>(sizeof(S));          // elements per piece
    static_assert(EPV == 8 || EPV == 4, "16-bit or 32-bit elements");
    __shared__ float m_slots[kWaves];
    __shared__ double s_slots[kWaves];
    const S* xr = x + static_cast<long>(blockIdx.x) * n;
    S* outr = out + static_cast<long>(blockIdx.x) * n;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int pieces = n / EPV;
    // minus infinity in every element, for the lanes past the row's end
    constexpr std::uint32_t kFill = EPV == 4 ? 0xFF800000u : (std::is_same<T, bf16_t>::value ? 0xFF80FF80u : 0xFC00FC00u);
    float f[NV][EPV];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int pc = threadIdx.x + i * kBlock;
        u32x4 w = {kFill, kFill, kFill, kFill};
        if (pc < pieces) w = *reinterpret_cast<const u32x4*>(xr + EPV * pc);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            if constexpr (EPV == 4) {
                const std::uint32_t bits = w[e];
                f[i][e] = __builtin_bit_cast(float, bits);
            }
            else                    f[i][e] = E::to_f32(static_cast<S>(w[e >> 1] >> (16 * (e & 1))));
            m = __builtin_fmaxf(m, f[i][e]);
        }
    }
    m = wave_max(m);
    if (lane == 0) m_slots[wave] = m;
    __syncthreads();
    m = m_slots[0];
#pragma unroll
    for (int i = 1; i < kWaves; ++i) m = __builtin_fmaxf(m, m_slots[i]);
    const double md = static_cast<double>(m);
    double ex[NV][EPV], sum = 0.0;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            ex[i][e] = exp(static_cast<double>(f[i][e]) - md);       // (lanes past the row's end: exp(-inf - m) = 0, or a NaN when the sum is one anyway)
            sum += ex[i][e];
        }
    sum = wave_sum(sum);
    if (lane == 0) s_slots[wave] = sum;
    __syncthreads();
    sum = 0.0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) sum += s_slots[i];
    const bool plain = sum > 0.0 && sum <= 1.0e300;        // wave-uniform (false for a NaN)
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int pc = threadIdx.x + i * kBlock;
        u32x4 w;
        if constexpr (EPV == 4) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float q = static_cast<float>(ex[i][e] / sum);
                w[e] = __builtin_bit_cast(std::uint32_t, q);
            }
        } else {
            std::uint16_t o[8];
            if (plain) {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = E::from_f32_finite(static_cast<float>(ex[i][e] / sum));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = E::from_f64(ex[i][e] / sum);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = o[2 * q] | (static_cast<std::uint32_t>(o[2 * q + 1]) << 16);
        }
        if (pc < pieces) *reinterpret_cast<u32x4*>(outr + EPV * pc) = w;
    }
}

// Rows in whole 16-byte pieces at 16-byte aligned addresses, up to 32768 elements, same dtype out: the kernel above.
template <typename T>
bool launch_softmax_vec(const void* x, void* out, long rows, long n, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    constexpr long EPV = 16 / sizeof(S);
    if (n % EPV != 0 || n > 32 * 1024 || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) != 0) return false;
    const dim3 g(static_cast<unsigned>(rows));
    const auto* xs = static_cast<const S*>(x);
    auto* os = static_cast<S*>(out);
    const long pieces = n / EPV;
    constexpr int kMost = 32 / EPV;        // pieces per thread at most: 32 exponentials in registers
    if (pieces <= 64)        hipLaunchKernelGGL((softmax_rows_vec_kernel<T, 1, 64>), g, dim3(64), 0, s, xs, os, (int)n);
    else if (pieces <= 128)  hipLaunchKernelGGL((softmax_rows_vec_kernel<T, 1, 128>), g, dim3(128), 0, s, xs, os, (int)n);
    else if (pieces <= 256)  hipLaunchKernelGGL((softmax_rows_vec_kernel<T, 1, 256>), g, dim3(256), 0, s, xs, os, (int)n);
    else if (pieces <= 512)  hipLaunchKernelGGL((softmax_rows_vec_kernel<T, 2, 256>), g, dim3(256), 0, s, xs, os, (int)n);
    else if (pieces <= 1024) hipLaunchKernelGGL((softmax_rows_vec_kernel<T, 4, 256>), g, dim3(256), 0, s, xs, os, (int)n);
    else if (pieces <= 256 * kMost)  hipLaunchKernelGGL((softmax_rows_vec_kernel<T, kMost, 256>), g, dim3(256), 0, s, xs, os, (int)n);
    else                     hipLaunchKernelGGL((softmax_rows_vec_kernel<T, kMost, 1024>), g, dim3(1024), 0, s, xs, os, (int)n);
    return true;
}

// (value, index) order of the reference: larger value first (smaller when !largest), then lower index.
__device__ __forceinline__ bool comes_before(double va, long ia, double vb, long ib, bool largest) {
    return largest ? (va > vb || (va == vb && ia < ib)) : (va < vb || (va == vb && ia < ib));
}

template <typename T>
__global__ __launch_bounds__(kBlock) void topk_rows_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                           typename Elem<T>::store_t* __restrict__ values,
                                                           long* __restrict__ indices, long n, long k, int largest_i) {
    using E = Elem<T>;
    __shared__ double v_slots[kWaves];
    __shared__ long   i_slots[kWaves];
    const bool largest = largest_i != 0;
    const auto* xr = x + static_cast<long>(blockIdx.x) * n;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;

    // NaNs.  The host scans a row from the left and an element replaces the running best only if
    // it compares greater (or equal with a lower index): a NaN therefore never replaces anything and
    // is never "after" the previous slot -- it can only be chosen by being the scan's first element,
    // x[0] in slot 0.  The slot after that finds no element "after" a NaN (index -1, value 0), and
    // the one after it goes on from (0, -1) like from any other previous slot.  In a parallel
    // search that is: NaNs take no part, except that a NaN x[0] is slot 0.
    const bool first_is_nan = n > 0 && E::to_f64(xr[0]) != E::to_f64(xr[0]);
    double prev_v = 0.0;
    long prev_i = -1;
    for (long s = 0; s < k; ++s) {
        double best_v = 0.0;
        long best_i = -1;
        for (long j = threadIdx.x; j < n; j += kBlock) {
            const double v = E::to_f64(xr[j]);
            if (v != v) continue;
            // strictly after the previous slot in (value, index) order
            if (s > 0 && !comes_before(prev_v, prev_i, v, j, largest)) continue;
            if (best_i < 0 || comes_before(v, j, best_v, best_i, largest)) {
                best_v = v;
                best_i = j;
            }
        }
        // wave, then workgroup argbest; index -1 marks "none"
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const double ov = __shfl_xor(best_v, off, kWave);
            const long oi = __shfl_xor(best_i, off, kWave);
            if (oi >= 0 && (best_i < 0 || comes_before(ov, oi, best_v, best_i, largest))) {
                best_v = ov;
                best_i = oi;
            }
        }
        if (lane == 0) {
            v_slots[wave] = best_v;
            i_slots[wave] = best_i;
        }
        __syncthreads();
        best_v = v_slots[0];
        best_i = i_slots[0];
#pragma unroll
        for (int i = 1; i < kWaves; ++i) {
            if (i_slots[i] >= 0 && (best_i < 0 || comes_before(v_slots[i], i_slots[i], best_v, best_i, largest))) {
                best_v = v_slots[i];
                best_i = i_slots[i];
            }
        }
        __syncthreads();
        if (first_is_nan && s == 0) {
            best_i = 0;
            best_v = E::to_f64(xr[0]);
        }
        if (threadIdx.x == 0) {
            // no eligible element: the host engine reports index -1 and value 0
            values[static_cast<long>(blockIdx.x) * k + s] = E::from_f64(best_i >= 0 ? best_v : 0.0);   // (a NaN as the host narrows it)
            indices[static_cast<long>(blockIdx.x) * k + s] = best_i;
        }
        if (best_i < 0) best_v = 0.0;
        prev_v = best_v;
        prev_i = best_i;
    }
}

// ---- long rows of bf16 / fp16 / fp32 (vocabulary-sized logits, k a few dozen): the same result
// without a pass over the row per slot.  An element becomes one 64-bit key, its value made
// monotone in the upper half and 2^32 - 1 - index in the lower, so that "comes before" in the
// reference's (value, index) order is "has the larger key" and "strictly after the previous slot"
// is "key below the previous slot's key"; NaNs get key 0 = no element, -0 is keyed as +0 (the
// reference compares them equal and lets the index decide).  Thread t owns the 16-byte groups of
// elements t, t + kThreads, ... and keeps the best key of them that is still below the bound.
// A slot is then: the best of the wavefronts' bests (LDS), and only the thread that owned it looks
// for its next candidate -- its wavefront does that together, a group per lane.  When nothing is
// left (NaNs, or k beyond the eligible elements) the reference reports (0, -1) and carries on from
// there, i.e. with the bound at (value 0, index -1): every thread scans again.
typedef unsigned long long u64;

template <typename T>
__device__ __forceinline__ u64 topk_key(typename Elem<T>::store_t raw, long j, bool largest) {
    const float f = Elem<T>::to_f32(raw);
    if (f != f) return 0ull;
    std::uint32_t u = __builtin_bit_cast(std::uint32_t, f);
    if ((u << 1) == 0u) u = 0u;                                    // -0 -> +0
    std::uint32_t mono = (u >> 31) ? ~u : (u | 0x80000000u);
    if (!largest) mono = ~mono;
    return (static_cast<u64>(mono) << 32) | static_cast<u64>(0xFFFFFFFFu - static_cast<std::uint32_t>(j));
}

// Maximum of a 64-bit key over the wave, in every lane, without the LDS crossbar: four DPP
// exchanges inside each row of 16 lanes, then the four row maxima through v_readlane.
template <int kCtrl>
__device__ __forceinline__ u64 dpp_move_u64(u64 v) {
    const int lo = static_cast<int>(v), hi = static_cast<int>(v >> 32);
    const int lo2 = __builtin_amdgcn_update_dpp(lo, lo, kCtrl, 0xf, 0xf, false);
    const int hi2 = __builtin_amdgcn_update_dpp(hi, hi, kCtrl, 0xf, 0xf, false);
    return (static_cast<u64>(static_cast<std::uint32_t>(hi2)) << 32) | static_cast<std::uint32_t>(lo2);
}
__device__ __forceinline__ u64 readlane_u64(u64 v, int lane) {
    const std::uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(v), lane);
    const std::uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(v >> 32), lane);
    return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ u64 wave_max_u64(u64 v) {
    auto mx = [](u64 a, u64 b) { return a > b ? a : b; };
    v = mx(v, dpp_move_u64<0xB1>(v));    // quad_perm [1,0,3,2]: lane ^ 1
    v = mx(v, dpp_move_u64<0x4E>(v));    // quad_perm [2,3,0,1]: lane ^ 2
    v = mx(v, dpp_move_u64<0x141>(v));   // row_half_mirror
    v = mx(v, dpp_move_u64<0x140>(v));   // row_mirror
    return mx(mx(readlane_u64(v, 0), readlane_u64(v, 16)), mx(readlane_u64(v, 32), readlane_u64(v, 48)));
}

template <typename T, int kThreads>
__global__ __launch_bounds__(kThreads) void topk_rows_select_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                                    typename Elem<T>::store_t* __restrict__ values,
                                                                    long* __restrict__ indices, long n, long k, int largest_i) {
    using E = Elem<T>;
    using S = typename E::store_t;
    constexpr int kNW = kThreads / kWave;
    __shared__ u64 wbest[kNW];
    const bool largest = largest_i != 0;
    const S* xr = x + static_cast<long>(blockIdx.x) * n;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    constexpr int GE = 16 / static_cast<int>(sizeof(S));          // elements per 16-byte group
    const long ngroups = (n + GE - 1) / GE;
    // rows that start on a 16-byte boundary and are whole groups long: one load per group
    const bool wide = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && n % GE == 0;

    // best key below `bound` among the elements of group g
    auto group_best = [&](long g, u64 bound) -> u64 {
        u64 best = 0ull;
        const long j0 = g * GE;
        if (wide) {
            const u32x4 v = load16(xr + j0);
            const S* e = reinterpret_cast<const S*>(&v);
#pragma unroll
            for (int i = 0; i < GE; ++i) {
                const u64 key = topk_key<T>(e[i], j0 + i, largest);
                if (key < bound && key > best) best = key;
            }
        } else {
#pragma unroll
            for (int i = 0; i < GE; ++i) {
                const long j = j0 + i;
                if (j < n) {
                    const u64 key = topk_key<T>(xr[j], j, largest);
                    if (key < bound && key > best) best = key;
                }
            }
        }
        return best;
    };
    auto scan_own = [&](u64 bound) -> u64 {
        u64 best = 0ull;
        for (long g = tid; g < ngroups; g += kThreads) {
            const u64 b = group_best(g, bound);
            best = b > best ? b : best;
        }
        return best;
    };
    // the bound "after (value 0, index -1)": every element whose value key does not exceed that of 0
    const u64 zero_bound = ((topk_key<T>(static_cast<S>(0), 0, largest) >> 32) + 1ull) << 32;

    const bool first_is_nan = n > 0 && E::to_f64(xr[0]) != E::to_f64(xr[0]);
    u64 bound = ~0ull, mine = 0ull;
    bool rescan_all = true;
    for (long s = 0; s < k; ++s) {
        S* vout = values + static_cast<long>(blockIdx.x) * k + s;
        long* iout = indices + static_cast<long>(blockIdx.x) * k + s;
        if (first_is_nan && s < 2) {
            // a NaN first element is slot 0; nothing comes "after" a NaN, so slot 1 is (0, -1)
            if (tid == 0) {
                *vout = s == 0 ? E::from_f64(E::to_f64(xr[0])) : E::from_f64(0.0);
                *iout = s == 0 ? 0 : -1;
            }
            bound = zero_bound;
            rescan_all = true;
            continue;
        }
        if (rescan_all) {
            mine = scan_own(bound);
            const u64 wb = wave_max_u64(mine);
            if (lane == 0) wbest[wave] = wb;
            rescan_all = false;
        }
        __syncthreads();
        u64 best = 0ull;
        int best_wave = 0;
#pragma unroll
        for (int w = 0; w < kNW; ++w) {
            const u64 c = wbest[w];
            if (c > best) {
                best = c;
                best_wave = w;
            }
        }
        __syncthreads();                                   // everyone has read the wavefronts' bests
        if (best == 0ull) {                                // nothing eligible: (0, -1), go on from there
            if (tid == 0) {
                *vout = E::from_f64(0.0);
                *iout = -1;
            }
            bound = zero_bound;
            rescan_all = true;
            continue;
        }
        const long idx = static_cast<long>(0xFFFFFFFFu - static_cast<std::uint32_t>(best));
        if (tid == 0) {
            *vout = xr[idx];
            *iout = idx;
        }
        bound = best;
        if (wave == best_wave) {
            // the lane whose candidate was taken gets its next one: its groups, a group per lane
            const u64 owners = __ballot(mine == best);
            const int owner_lane = __ffsll(static_cast<long long>(owners)) - 1;
            const long owner_tid = static_cast<long>(wave) * kWave + owner_lane;
            u64 next = 0ull;
            for (long g = owner_tid + static_cast<long>(lane) * kThreads; g < ngroups; g += static_cast<long>(kWave) * kThreads) {
                const u64 b = group_best(g, bound);
                next = b > next ? b : next;
            }
            next = wave_max_u64(next);
            if (lane == owner_lane) mine = next;
            const u64 wb = wave_max_u64(mine);
            if (lane == 0) wbest[wave] = wb;
        }
    }
}

// ---- short rows (n <= 64 * EPL): one wave per row, four rows per workgroup, the row in
// registers (lane l holds elements l, l + 64, ...), no LDS and no barrier.  Router logits and
// other rows of a few dozen elements would otherwise leave most of a 256-thread workgroup idle.
template <typename TI, typename TO, int EPL>
__global__ __launch_bounds__(kBlock) void softmax_rows_wave_kernel(const typename Elem<TI>::store_t* __restrict__ x,
                                                                   typename Elem<TO>::store_t* __restrict__ out, long rows, int n) {
    using EI = Elem<TI>;
    using EO = Elem<TO>;
    const int lane = threadIdx.x % kWave;
    const long row = static_cast<long>(blockIdx.x) * kWaves + threadIdx.x / kWave;
    if (row >= rows) return;                    // whole waves leave: nothing below synchronises the workgroup
    const auto* xr = x + row * n;
    auto* outr = out + row * n;
    double v[EPL];
    double m = -INFINITY;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int j = lane + i * kWave;
        v[i] = j < n ? EI::to_f64(xr[j]) : -INFINITY;
        if (j < n && v[i] > m) m = v[i];        // as the host: a NaN never replaces the max
    }
    m = wave_max_f64(m);
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int j = lane + i * kWave;
        v[i] = j < n ? exp(v[i] - m) : 0.0;
        sum += v[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int j = lane + i * kWave;
        if (j < n) outr[j] = EO::from_f64(v[i] / sum);
    }
}

template <typename T, int EPL>
__global__ __launch_bounds__(kBlock) void topk_rows_wave_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                                typename Elem<T>::store_t* __restrict__ values,
                                                                long* __restrict__ indices, long rows, int n, int k, int largest_i) {
    using E = Elem<T>;
    const bool largest = largest_i != 0;
    const int lane = threadIdx.x % kWave;
    const long row = static_cast<long>(blockIdx.x) * kWaves + threadIdx.x / kWave;
    if (row >= rows) return;
    const auto* xr = x + row * n;
    double v[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int j = lane + i * kWave;
        v[i] = j < n ? E::to_f64(xr[j]) : 0.0;
    }
    // (NaNs take no part in the search, except that a NaN x[0] is slot 0: see topk_rows_kernel)
    const double x0 = __shfl(v[0], 0, kWave);
    const bool first_is_nan = x0 != x0;
    double prev_v = 0.0;
    long prev_i = -1;
    for (int s = 0; s < k; ++s) {
        double best_v = 0.0;
        long best_i = -1;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const long j = lane + i * kWave;
            if (j >= n || v[i] != v[i]) continue;
            if (s > 0 && !comes_before(prev_v, prev_i, v[i], j, largest)) continue;   // strictly after the previous slot
            if (best_i < 0 || comes_before(v[i], j, best_v, best_i, largest)) {
                best_v = v[i];
                best_i = j;
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const double ov = __shfl_xor(best_v, off, kWave);
            const long oi = __shfl_xor(static_cast<int>(best_i), off, kWave);
            if (oi >= 0 && (best_i < 0 || comes_before(ov, oi, best_v, best_i, largest))) {
                best_v = ov;
                best_i = oi;
            }
        }
        if (first_is_nan && s == 0) {
            best_i = 0;
            best_v = x0;
        }
        if (lane == 0) {
            // no eligible element: index -1, value 0, as the host engine
            values[row * k + s] = E::from_f64(best_i >= 0 ? best_v : 0.0);   // (a NaN as the host narrows it)
            indices[row * k + s] = best_i;
        }
        if (best_i < 0) best_v = 0.0;
        prev_v = best_v;
        prev_i = best_i;
    }
}

// Short rows of bf16 / fp16 / fp32 with the same keys: a lane holds the keys of its elements, a
// slot is a wave maximum, and the lane that held it writes the element out and retires the key.
template <typename T, int EPL>
__global__ __launch_bounds__(kBlock) void topk_rows_wave_keys_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                                     typename Elem<T>::store_t* __restrict__ values,
                                                                     long* __restrict__ indices, long rows, int n, int k, int largest_i) {
    using E = Elem<T>;
    using S = typename E::store_t;
    const bool largest = largest_i != 0;
    const int lane = threadIdx.x % kWave;
    const long row = static_cast<long>(blockIdx.x) * kWaves + threadIdx.x / kWave;
    if (row >= rows) return;
    const S* xr = x + row * n;
    S raw[EPL];
    u64 orig[EPL], live[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int j = lane + i * kWave;
        raw[i] = j < n ? xr[j] : static_cast<S>(0);
        orig[i] = j < n ? topk_key<T>(raw[i], j, largest) : 0ull;
        live[i] = orig[i];
    }
    const u64 zero_bound = ((topk_key<T>(static_cast<S>(0), 0, largest) >> 32) + 1ull) << 32;
    auto restart = [&]() {                       // go on from (value 0, index -1): everything not above zero is eligible again
#pragma unroll
        for (int i = 0; i < EPL; ++i) live[i] = orig[i] < zero_bound ? orig[i] : 0ull;
    };
    const S x0 = xr[0];
    const bool first_is_nan = E::to_f64(x0) != E::to_f64(x0);
    S* vout = values + row * k;
    long* iout = indices + row * k;
    for (int s = 0; s < k; ++s) {
        if (first_is_nan && s < 2) {
            if (lane == 0) {
                vout[s] = s == 0 ? E::from_f64(E::to_f64(x0)) : E::from_f64(0.0);
                iout[s] = s == 0 ? 0 : -1;
            }
            restart();
            continue;
        }
        u64 m = live[0];
#pragma unroll
        for (int i = 1; i < EPL; ++i) m = live[i] > m ? live[i] : m;
        const u64 best = wave_max_u64(m);
        if (best == 0ull) {
            if (lane == 0) {
                vout[s] = E::from_f64(0.0);
                iout[s] = -1;
            }
            restart();
            continue;
        }
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            if (live[i] == best) {
                vout[s] = raw[i];
                iout[s] = lane + i * kWave;
                live[i] = 0ull;
            }
    }
}

template <typename TI>
int launch_softmax(const void* x, void* out, long rows, long n, int dtype_out, hipStream_t s) {
    using SI = typename Elem<TI>::store_t;
    const dim3 g(static_cast<unsigned>(rows)), b(kBlock);
    if (n <= 4 * kWave) {
        const dim3 gw(static_cast<unsigned>((rows + kWaves - 1) / kWaves));
        const bool widen = dtype_out == PARAS_F32 && sizeof(SI) == 2;
        const auto* xs = static_cast<const SI*>(x);
        if (n <= kWave) {
            if (widen) hipLaunchKernelGGL((softmax_rows_wave_kernel<TI, float, 1>), gw, b, 0, s, xs, static_cast<float*>(out), rows, (int)n);
            else       hipLaunchKernelGGL((softmax_rows_wave_kernel<TI, TI, 1>), gw, b, 0, s, xs, static_cast<SI*>(out), rows, (int)n);
        } else {
            if (widen) hipLaunchKernelGGL((softmax_rows_wave_kernel<TI, float, 4>), gw, b, 0, s, xs, static_cast<float*>(out), rows, (int)n);
            else       hipLaunchKernelGGL((softmax_rows_wave_kernel<TI, TI, 4>), gw, b, 0, s, xs, static_cast<SI*>(out), rows, (int)n);
        }
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    if (n <= 16 * kBlock) {
        const bool widen = dtype_out == PARAS_F32 && sizeof(SI) == 2;
        const auto* xs = static_cast<const SI*>(x);
        if constexpr (sizeof(SI) == 2 || sizeof(SI) == 4) {
            if (!widen && launch_softmax_vec<TI>(x, out, rows, n, s)) {
                PARAS_HIP_TRY(hipGetLastError());
                return PARAS_OK;
            }
        }
        if (n <= 4 * kBlock) {
            if (widen) hipLaunchKernelGGL((softmax_rows_reg_kernel<TI, float, 4>), g, b, 0, s, xs, static_cast<float*>(out), (int)n);
            else       hipLaunchKernelGGL((softmax_rows_reg_kernel<TI, TI, 4>), g, b, 0, s, xs, static_cast<SI*>(out), (int)n);
        } else {
            if (widen) hipLaunchKernelGGL((softmax_rows_reg_kernel<TI, float, 16>), g, b, 0, s, xs, static_cast<float*>(out), (int)n);
            else       hipLaunchKernelGGL((softmax_rows_reg_kernel<TI, TI, 16>), g, b, 0, s, xs, static_cast<SI*>(out), (int)n);
        }
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    if constexpr (sizeof(SI) == 2 || sizeof(SI) == 4) {
        // up to 32768 elements the exponentials of a row still fit the registers of a workgroup (one
        // exponential per element instead of two, one read of the row instead of three)
        if (!(dtype_out == PARAS_F32 && sizeof(SI) == 2) && launch_softmax_vec<TI>(x, out, rows, n, s)) {
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
    }
    const bool widen_long = dtype_out == PARAS_F32 && sizeof(SI) == 2;
    if (rows <= 2048) {           // few long rows: a CU's worth of wavefronts per row
        const dim3 b4(1024);
        if (widen_long) hipLaunchKernelGGL((softmax_rows_kernel<TI, float, 1024>), g, b4, 0, s, static_cast<const SI*>(x), static_cast<float*>(out), n);
        else            hipLaunchKernelGGL((softmax_rows_kernel<TI, TI, 1024>), g, b4, 0, s, static_cast<const SI*>(x), static_cast<SI*>(out), n);
    } else if (widen_long)
        hipLaunchKernelGGL((softmax_rows_kernel<TI, float, kBlock>), g, b, 0, s, static_cast<const SI*>(x), static_cast<float*>(out), n);
    else
        hipLaunchKernelGGL((softmax_rows_kernel<TI, TI, kBlock>), g, b, 0, s, static_cast<const SI*>(x), static_cast<SI*>(out), n);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

template <typename T>
int launch_topk(const void* x, void* values, long* indices, long rows, long n, long k, int largest, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    if (n <= 4 * kWave) {
        const dim3 gw(static_cast<unsigned>((rows + kWaves - 1) / kWaves)), b(kBlock);
        if constexpr (sizeof(S) <= 4) {
            if (n <= kWave)
                hipLaunchKernelGGL((topk_rows_wave_keys_kernel<T, 1>), gw, b, 0, s, static_cast<const S*>(x), static_cast<S*>(values), indices, rows, (int)n, (int)k, largest);
            else
                hipLaunchKernelGGL((topk_rows_wave_keys_kernel<T, 4>), gw, b, 0, s, static_cast<const S*>(x), static_cast<S*>(values), indices, rows, (int)n, (int)k, largest);
        } else if (n <= kWave)
            hipLaunchKernelGGL((topk_rows_wave_kernel<T, 1>), gw, b, 0, s, static_cast<const S*>(x), static_cast<S*>(values), indices, rows, (int)n, (int)k, largest);
        else
            hipLaunchKernelGGL((topk_rows_wave_kernel<T, 4>), gw, b, 0, s, static_cast<const S*>(x), static_cast<S*>(values), indices, rows, (int)n, (int)k, largest);
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    if constexpr (sizeof(S) <= 4) {
        if (n < (1LL << 32)) {
            if (n <= 8192)
                hipLaunchKernelGGL((topk_rows_select_kernel<T, 256>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, s, static_cast<const S*>(x),
                                   static_cast<S*>(values), indices, n, k, largest);
            else
                hipLaunchKernelGGL((topk_rows_select_kernel<T, 1024>), dim3(static_cast<unsigned>(rows)), dim3(1024), 0, s, static_cast<const S*>(x),
                                   static_cast<S*>(values), indices, n, k, largest);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
    }
    hipLaunchKernelGGL((topk_rows_kernel<T>), dim3(static_cast<unsigned>(rows)), dim3(kBlock), 0, s, static_cast<const S*>(x),
                       static_cast<S*>(values), indices, n, k, largest);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_softmax_rows(const void* x, void* out, int64_t rows, int64_t n, int dtype_in, int dtype_out, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && n >= 0, "paras_softmax_rows: negative shape");
    if (rows == 0 || n == 0) return PARAS_OK;
    PARAS_REQUIRE(x && out, "paras_softmax_rows: null pointer");
    PARAS_REQUIRE(rows <= 0x7fffffffLL, "paras_softmax_rows: too many rows");
    PARAS_REQUIRE(dtype_out == dtype_in || (dtype_out == PARAS_F32 && (dtype_in == PARAS_BF16 || dtype_in == PARAS_F16)),
                  "paras_softmax_rows: the output dtype is the input dtype, or fp32 for a 16-bit input");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    switch (dtype_in) {
        case PARAS_F32:  return launch_softmax<float>(x, out, rows, n, dtype_out, s);
        case PARAS_F64:  return launch_softmax<double>(x, out, rows, n, dtype_out, s);
        case PARAS_BF16: return launch_softmax<bf16_t>(x, out, rows, n, dtype_out, s);
        case PARAS_F16:  return launch_softmax<f16_t>(x, out, rows, n, dtype_out, s);
        default: return fail(PARAS_ERR_INVALID, "paras_softmax_rows: unknown dtype %d", dtype_in);
    }
}

int paras_topk_rows(const void* x, void* values, int64_t* indices, int64_t rows, int64_t n, int64_t k, int largest,
                    int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && n >= 0, "paras_topk_rows: negative shape");
    PARAS_REQUIRE(k >= 0 && k <= n, "paras_topk_rows: k out of range");
    if (rows == 0 || k == 0) return PARAS_OK;
    PARAS_REQUIRE(x && values && indices, "paras_topk_rows: null pointer");
    PARAS_REQUIRE(rows <= 0x7fffffffLL, "paras_topk_rows: too many rows");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    long* idx = reinterpret_cast<long*>(indices);
    switch (dtype) {
        case PARAS_F32:  return launch_topk<float>(x, values, idx, rows, n, k, largest, s);
        case PARAS_F64:  return launch_topk<double>(x, values, idx, rows, n, k, largest, s);
        case PARAS_BF16: return launch_topk<bf16_t>(x, values, idx, rows, n, k, largest, s);
        case PARAS_F16:  return launch_topk<f16_t>(x, values, idx, rows, n, k, largest, s);
        default: return fail(PARAS_ERR_INVALID, "paras_topk_rows: unknown dtype %d", dtype);
    }
}

}  // extern "C"
