// Tensor plumbing kernels for the `paras` device: strided copy with optional
// float-type conversion, strided fill, and the two "composed" ops whose
// reference implementations narrow to the tensor dtype after every step.
// The copies keep whole expressions on the device so that the hot-path kernels
// are not surrounded by host bounces; the two composed ops are what
// F.rms_norm and torch_paras::swiglu reach on this device and stream at the
// rate of their fused counterparts for the 16-bit dtypes.
#include <hip/hip_runtime.h>

#include <cmath>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/swiglu_math.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxDims = 8;  // the reference's StridedSpec limit (csrc/core/kernels.h:31)

struct Strided {
    int  ndim;
    long sizes[kMaxDims];
    long src_strides[kMaxDims];
    long dst_strides[kMaxDims];
};

__device__ __forceinline__ void offsets(const Strided& s, long flat, long* so, long* d_o) {
    long a = 0, b = 0;
    for (int d = s.ndim - 1; d >= 0; --d) {
        const long c = flat % s.sizes[d];
        flat /= s.sizes[d];
        a += c * s.src_strides[d];
        b += c * s.dst_strides[d];
    }
    *so = a;
    *d_o = b;
}

template <typename W>
__global__ __launch_bounds__(kBlock) void copy_same_kernel(const W* __restrict__ src, W* __restrict__ dst, long n,
                                                           const Strided s) {
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * kBlock) {
        long a, b;
        offsets(s, i, &a, &b);
        dst[b] = src[a];
    }
}

// Conversion between the four float storage types goes through double, which
// holds every source value exactly, then narrows as the host does.
template <typename TS, typename TD>
__global__ __launch_bounds__(kBlock) void copy_convert_kernel(const typename Elem<TS>::store_t* __restrict__ src,
                                                              typename Elem<TD>::store_t* __restrict__ dst, long n,
                                                              const Strided s) {
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * kBlock) {
        long a, b;
        offsets(s, i, &a, &b);
        if constexpr (sizeof(typename Elem<TS>::store_t) == 8)
            dst[b] = Elem<TD>::from_f64(Elem<TS>::to_f64(src[a]));
        else
            dst[b] = Elem<TD>::from_f32(Elem<TS>::to_f32(src[a]));   // float -> T: one narrowing, as static_cast<T>(float)
    }
}

template <typename W>
__global__ __launch_bounds__(kBlock) void fill_kernel(W* __restrict__ dst, long n, const Strided s, W value) {
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * kBlock) {
        long a, b;
        offsets(s, i, &a, &b);
        dst[b] = value;
    }
}

template <typename T>
__device__ __forceinline__ double narrow(double v) { return Elem<T>::to_f64(Elem<T>::from_f64(v)); }

// aten::rms_norm as the reference composes it (csrc/ops/rms_swiglu_ops.cpp:66-73):
// pow(2) -> mean(keepdim) [sum, then * 1/n] -> + eps -> rsqrt -> x * inv -> * w,
// each step narrowed to T.  One workgroup per row.
template <typename T>
__global__ __launch_bounds__(kBlock) void rms_norm_composed_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                                   const typename Elem<T>::store_t* __restrict__ w,
                                                                   typename Elem<T>::store_t* __restrict__ out, long rows,
                                                                   long H, double eps_narrowed) {
    using E = Elem<T>;
    __shared__ double slots[kBlock / kWave];
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        const auto* xr = x + r * H;
        double acc = 0.0;
        for (long j = threadIdx.x; j < H; j += kBlock) {
            const double v = E::to_f64(xr[j]);
            acc += narrow<T>(v * v);
        }
        acc = wave_sum(acc);
        __syncthreads();
        if ((threadIdx.x & (kWave - 1)) == 0) slots[threadIdx.x / kWave] = acc;
        __syncthreads();
        double sum = 0.0;
        for (int i = 0; i < kBlock / kWave; ++i) sum += slots[i];
        const double s = narrow<T>(sum);
        const double m = narrow<T>(s * (H > 0 ? 1.0 / static_cast<double>(H) : 0.0));
        const double a = narrow<T>(m + 1.0 * eps_narrowed);
        const double inv = narrow<T>(1.0 / sqrt(a));
        for (long j = threadIdx.x; j < H; j += kBlock) {
            double y = narrow<T>(E::to_f64(xr[j]) * inv);
            if (w != nullptr) y = narrow<T>(y * E::to_f64(w[j]));
            out[r * H + j] = E::from_f64(y);
        }
    }
}

// torch_paras::swiglu(x, gate) = x * silu(gate), silu narrowed first
// (csrc/ops/rms_swiglu_ops.cpp:83-86, csrc/ops/pointwise_ops.cpp:460-464).
template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_composed_kernel(const typename Elem<T>::store_t* __restrict__ x,
                                                                 const typename Elem<T>::store_t* __restrict__ gate,
                                                                 typename Elem<T>::store_t* __restrict__ out, long n) {
    using E = Elem<T>;
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * kBlock) {
        const double g = E::to_f64(gate[i]);
        const double s = narrow<T>(g / (1.0 + exp(-g)));
        out[i] = E::from_f64(E::to_f64(x[i]) * s);
    }
}

// ---- 16-bit dtypes, 16-byte aligned rows: the same results at streaming speed.  Every product
// of two 16-bit values is exact in fp32 (at most 22 significant bits), so "multiply in fp64, narrow"
// is one fp32 multiply and one rounding; only the row sum needs fp64.  silu narrowed to T is the
// fused SwiGLU element function with an up value of one.
template <typename T, int NV>
__global__ __launch_bounds__(kBlock, (NV <= 2 ? 8 : 4)) void rms_norm_composed_vec(
    const std::uint16_t* __restrict__ x, const std::uint16_t* __restrict__ w, std::uint16_t* __restrict__ out, long rows,
    int H, double eps_narrowed) {
    using E = Elem<T>;
    constexpr int kWaves = kBlock / kWave;
    __shared__ double slots[2 * kWaves];
    const int nvec = H / 8;
    u32x4 wv[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * kBlock;
        if (w != nullptr && c < nvec) wv[i] = load16(w + static_cast<long>(c) * 8);
    }
    int calls = 0;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        u32x4 xv[NV];
        double acc = 0.0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * kBlock;
            if (c < nvec) {
                xv[i] = load16_nt(x + r * H + static_cast<long>(c) * 8);
                const std::uint16_t* e = reinterpret_cast<const std::uint16_t*>(&xv[i]);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float v = E::to_f32(e[j]);
                    // (the conversion instruction: a NaN's payload does not matter in a sum)
                    acc += static_cast<double>(E::to_f32(E::from_f32_finite(v * v)));
                }
            }
        }
        acc = wave_sum(acc);
        double* set = slots + (calls++ & 1) * kWaves;        // alternating sets: one barrier per row
        if ((threadIdx.x & (kWave - 1)) == 0) set[threadIdx.x / kWave] = acc;
        __syncthreads();
        double sum = 0.0;
#pragma unroll
        for (int i = 0; i < kWaves; ++i) sum += set[i];
        const double s = narrow<T>(sum);
        const double m = narrow<T>(s * (1.0 / static_cast<double>(H)));
        const double a = narrow<T>(m + 1.0 * eps_narrowed);
        const float inv = static_cast<float>(narrow<T>(1.0 / sqrt(a)));
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * kBlock;
            if (c < nvec) {
                const std::uint16_t* e = reinterpret_cast<const std::uint16_t*>(&xv[i]);
                const std::uint16_t* we = reinterpret_cast<const std::uint16_t*>(&wv[i]);
                u32x4 o;
                std::uint16_t* oe = reinterpret_cast<std::uint16_t*>(&o);
                // Narrowing by the conversion instructions; they keep a NaN's payload where the host's
                // types canonicalise it, so a vector with a NaN in it (the probe below; inf - inf also
                // sets it off, harmlessly) is narrowed again in software, behind a wave-uniform branch.
                float probe = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float y1 = E::to_f32(e[j]) * inv;
                    std::uint16_t y = E::from_f32_finite(y1);
                    probe += y1;
                    if (w != nullptr) {
                        const float y2 = E::to_f32(y) * E::to_f32(we[j]);
                        y = E::from_f32_finite(y2);
                        probe += y2;
                    }
                    oe[j] = y;
                }
                if (__builtin_amdgcn_ballot_w64(probe != probe) != 0) {
                    asm volatile("" ::: "memory");           // not to be evaluated ahead of the branch
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        std::uint16_t y = E::from_f32(E::to_f32(e[j]) * inv);
                        if (w != nullptr) y = E::from_f32(E::to_f32(y) * E::to_f32(we[j]));
                        oe[j] = y;
                    }
                }
                store16_nt(out + r * H + static_cast<long>(c) * 8, o);
            }
        }
    }
}

constexpr int kComposedUnroll = 4;   // 16-byte vectors per stream in flight per lane

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_composed_vec(const std::uint16_t* __restrict__ x,
                                                              const std::uint16_t* __restrict__ gate,
                                                              std::uint16_t* __restrict__ out, long nvec) {
    using E = Elem<T>;
    const std::uint16_t one = E::from_f32(1.0f);
    const long stride = static_cast<long>(gridDim.x) * kBlock * kComposedUnroll;
    for (long base = static_cast<long>(blockIdx.x) * kBlock * kComposedUnroll + threadIdx.x; base < nvec; base += stride) {
        u32x4 xv[kComposedUnroll], gv[kComposedUnroll];
#pragma unroll
        for (int k = 0; k < kComposedUnroll; ++k) {
            const long i = base + static_cast<long>(k) * kBlock;
            if (i < nvec) {
                xv[k] = load16_nt(x + i * 8);
                gv[k] = load16_nt(gate + i * 8);
            }
        }
#pragma unroll
        for (int k = 0; k < kComposedUnroll; ++k) {
            const long i = base + static_cast<long>(k) * kBlock;
            if (i < nvec) {
                const std::uint16_t* xe = reinterpret_cast<const std::uint16_t*>(&xv[k]);
                const std::uint16_t* ge = reinterpret_cast<const std::uint16_t*>(&gv[k]);
                u32x4 o;
                std::uint16_t* oe = reinterpret_cast<std::uint16_t*>(&o);
#pragma unroll
                for (int j = 0; j < 8; ++j) oe[j] = E::from_f32(E::to_f32(xe[j]) * E::to_f32(swiglu_one<T>(ge[j], one)));
                store16_nt(out + i * 8, o);
            }
        }
    }
}

// ---- elementwise add / sub / mul / div with broadcasting (the reference's binary_kernel,
// csrc/ops/pointwise_ops.cpp:63-85 with add_out :262-268, sub_out :271-277, mul_out :280-283,
// div_out :299-302): out = T(a op alpha*b) evaluated in double.  For 16-bit tensors with alpha = 1
// add, sub and mul in fp32 give the same bits: a product of two such values is exact in fp32, and a
// sum is either exact in double (then fp32's correctly rounded sum is what double -> float gives)
// or one operand is below a quarter unit in the last place of the other in both.
enum { kOpAdd = 0, kOpSub = 1, kOpMul = 2, kOpDiv = 3 };

template <typename T>
__device__ __forceinline__ typename Elem<T>::store_t binary_one(int op, typename Elem<T>::store_t as, typename Elem<T>::store_t bs,
                                                                 double alpha, bool unit_alpha) {
    using E = Elem<T>;
    if constexpr (sizeof(typename E::store_t) == 2) {
        if (unit_alpha && op != kOpDiv) {
            const float x = E::to_f32(as), y = E::to_f32(bs);
            return E::from_f32(op == kOpAdd ? x + y : op == kOpSub ? x - y : x * y);
        }
    }
    const double x = E::to_f64(as), y = E::to_f64(bs);
    double r;
    switch (op) {
        case kOpAdd: r = x + alpha * y; break;
        case kOpSub: r = x - alpha * y; break;
        case kOpMul: r = x * y; break;
        default:     r = x / y; break;
    }
    return E::from_f64(r);
}

// general form: `s` carries a's strides as src_strides and b's as dst_strides; out is dense
template <typename T>
__global__ __launch_bounds__(kBlock) void binary_strided_kernel(int op, const typename Elem<T>::store_t* __restrict__ a,
                                                                const typename Elem<T>::store_t* __restrict__ b,
                                                                typename Elem<T>::store_t* __restrict__ out, long n, const Strided s,
                                                                double alpha) {
    const bool unit = alpha == 1.0;
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * kBlock) {
        long ao, bo;
        offsets(s, i, &ao, &bo);
        out[i] = binary_one<T>(op, a[ao], b[bo], alpha, unit);
    }
}

// 16-bit tensors, out and a dense, b dense or one value or one row repeated (period `brow` vectors,
// 0 = one value): eight elements per thread
template <typename T>
__global__ __launch_bounds__(kBlock) void binary_vec16_kernel(int op, const std::uint16_t* __restrict__ a,
                                                              const std::uint16_t* __restrict__ b, std::uint16_t* __restrict__ out,
                                                              long nvec, long brow, double alpha) {
    const long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= nvec) return;
    const bool unit = alpha == 1.0;
    const u32x4 av = load16_nt(a + i * 8);
    u32x4 bv;
    if (brow == 0) {
        const std::uint32_t w = b[0] | (static_cast<std::uint32_t>(b[0]) << 16);
        bv = u32x4{w, w, w, w};
    } else {
        bv = brow == nvec ? load16_nt(b + i * 8) : load16(b + (i % brow) * 8);
    }
    const std::uint16_t* ae = reinterpret_cast<const std::uint16_t*>(&av);
    const std::uint16_t* be = reinterpret_cast<const std::uint16_t*>(&bv);
    u32x4 o;
    std::uint16_t* oe = reinterpret_cast<std::uint16_t*>(&o);
#pragma unroll
    for (int j = 0; j < 8; ++j) oe[j] = binary_one<T>(op, ae[j], be[j], alpha, unit);
    store16_nt(out + i * 8, o);
}

// ---- index_select along one dim of a dense tensor seen as [outer, n_src, inner]:
// dst[o, i, :] = src[o, idx[i], :] (the reference's index_select, csrc/ops/indexing_ops.cpp:96-150;
// embedding lookups arrive here as dim 0).  `inner` is counted in W-byte units.  An index outside
// [0, n_src) is clamped into it: the reference does not check either, and a clamp cannot fault.
template <typename W>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(const W* __restrict__ src, const long* __restrict__ idx,
                                                             W* __restrict__ dst, long total, long n_src, long n_idx, long inner) {
    for (long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x; i < total; i += static_cast<long>(gridDim.x) * kBlock) {
        const long c = i % inner, r = i / inner;
        const long sel = r % n_idx, o = r / n_idx;
        long j = idx[sel];
        j = j < 0 ? 0 : (j >= n_src ? n_src - 1 : j);
        dst[i] = src[(o * n_src + j) * inner + c];
    }
}

unsigned grid_for(long n) {
    long g = (n + kBlock - 1) / kBlock;
    if (g > 65536) g = 65536;
    return static_cast<unsigned>(g < 1 ? 1 : g);
}

// Launches the register-resident kernel if the row shape allows it; false = use the general one.
template <typename T>
bool launch_rms_composed_vec(const void* x, const void* w, void* out, long rows, long H, double eps_narrowed, dim3 g,
                             hipStream_t st) {
    const bool aligned = H % 8 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                                         reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const long nvec = H / 8;
    if (!aligned || nvec > 4 * kBlock) return false;
    const auto* xs = static_cast<const std::uint16_t*>(x);
    const auto* ws = static_cast<const std::uint16_t*>(w);
    auto* os = static_cast<std::uint16_t*>(out);
    const dim3 b(kBlock);
    if (nvec <= kBlock)          hipLaunchKernelGGL((rms_norm_composed_vec<T, 1>), g, b, 0, st, xs, ws, os, rows, (int)H, eps_narrowed);
    else if (nvec <= 2 * kBlock) hipLaunchKernelGGL((rms_norm_composed_vec<T, 2>), g, b, 0, st, xs, ws, os, rows, (int)H, eps_narrowed);
    else                         hipLaunchKernelGGL((rms_norm_composed_vec<T, 4>), g, b, 0, st, xs, ws, os, rows, (int)H, eps_narrowed);
    return true;
}

// 16-byte vectors on the streaming kernel, the last n % 8 elements (or everything, if unaligned) on the scalar one.
template <typename T>
void launch_swiglu_composed16(const void* x, const void* gate, void* out, long n, hipStream_t st) {
    const auto* xs = static_cast<const std::uint16_t*>(x);
    const auto* gs = static_cast<const std::uint16_t*>(gate);
    auto* os = static_cast<std::uint16_t*>(out);
    long done = 0;
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 && n >= 8) {
        const long nvec = n / 8;
        long blocks = (nvec + kBlock * kComposedUnroll - 1) / (kBlock * kComposedUnroll);
        if (blocks > 0x7fffffffL) blocks = 0x7fffffffL;      // the kernel grid-strides beyond that
        hipLaunchKernelGGL((swiglu_composed_vec<T>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, st, xs, gs, os, nvec);
        done = nvec * 8;
    }
    if (done < n)
        hipLaunchKernelGGL((swiglu_composed_kernel<T>), dim3(grid_for(n - done)), dim3(kBlock), 0, st, xs + done, gs + done,
                           os + done, n - done);
}

int make_spec(int ndim, const int64_t* sizes, const int64_t* ss, const int64_t* ds, Strided* s, long* n) {
    PARAS_REQUIRE(ndim >= 0 && ndim <= kMaxDims, "paras: tensor rank %d exceeds kernel limit of %d", ndim, kMaxDims);
    // Size-1 dimensions are dropped and a dimension whose stride on both sides
    // equals the extent of the next one is merged into it, so a contiguous tensor
    // of any rank arrives at the kernels as one dimension of stride 1.
    long total = 1;
    int m = 0;
    for (int d = 0; d < ndim; ++d) {
        PARAS_REQUIRE(sizes[d] >= 0, "paras: negative size");
        total *= sizes[d];
        if (sizes[d] == 1) continue;
        s->sizes[m] = sizes[d];
        s->src_strides[m] = ss ? ss[d] : 0;
        s->dst_strides[m] = ds ? ds[d] : 0;
        ++m;
    }
    for (int d = m - 2; d >= 0 && total > 0; --d) {
        if (s->src_strides[d] == s->src_strides[d + 1] * s->sizes[d + 1] &&
            s->dst_strides[d] == s->dst_strides[d + 1] * s->sizes[d + 1]) {
            s->sizes[d] *= s->sizes[d + 1];
            s->src_strides[d] = s->src_strides[d + 1];
            s->dst_strides[d] = s->dst_strides[d + 1];
            for (int e = d + 1; e + 1 < m; ++e) {
                s->sizes[e] = s->sizes[e + 1];
                s->src_strides[e] = s->src_strides[e + 1];
                s->dst_strides[e] = s->dst_strides[e + 1];
            }
            --m;
        }
    }
    s->ndim = m;
    *n = total;
    return PARAS_OK;
}

// Both sides dense: a plain stream of 16-byte vectors, one per thread, past the cache.
__global__ __launch_bounds__(kBlock) void copy_dense_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, long nvec) {
    const long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < nvec) store16_nt(dst + i, load16_nt(src + i));
}

// Both sides dense and suitably aligned: eight elements per thread, one wide load and one wide store.
template <typename TS, typename TD>
__global__ __launch_bounds__(kBlock) void convert_dense_kernel(const typename Elem<TS>::store_t* __restrict__ src,
                                                              typename Elem<TD>::store_t* __restrict__ dst, long n8) {
    using SS = typename Elem<TS>::store_t;
    using SD = typename Elem<TD>::store_t;
    struct alignas(sizeof(SS) * 8 > 16 ? 16 : sizeof(SS) * 8) PackS { SS v[8]; };
    struct alignas(sizeof(SD) * 8 > 16 ? 16 : sizeof(SD) * 8) PackD { SD v[8]; };
    const long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n8) return;
    const PackS in = reinterpret_cast<const PackS*>(src)[i];
    PackD o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if constexpr (sizeof(SS) == 8) o.v[j] = Elem<TD>::from_f64(Elem<TS>::to_f64(in.v[j]));
        else                           o.v[j] = Elem<TD>::from_f32(Elem<TS>::to_f32(in.v[j]));
    }
    reinterpret_cast<PackD*>(dst)[i] = o;
}

template <typename TS, typename TD>
void launch_convert(const typename Elem<TS>::store_t* sp, void* dst, long n, const Strided& s, hipStream_t st) {
    using SD = typename Elem<TD>::store_t;
    auto* dp = static_cast<SD*>(dst);
    const bool dense = s.ndim == 0 || (s.ndim == 1 && s.src_strides[0] == 1 && s.dst_strides[0] == 1);
    long done = 0;
    if (dense && n >= 8 && ((reinterpret_cast<uintptr_t>(sp) | reinterpret_cast<uintptr_t>(dp)) & 15) == 0) {
        const long n8 = n / 8;
        hipLaunchKernelGGL((convert_dense_kernel<TS, TD>), dim3(static_cast<unsigned>((n8 + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, sp, dp, n8);
        done = n8 * 8;
        if (done == n) return;
        Strided t = s;
        t.ndim = 1; t.sizes[0] = n - done; t.src_strides[0] = 1; t.dst_strides[0] = 1;
        hipLaunchKernelGGL((copy_convert_kernel<TS, TD>), dim3(grid_for(n - done)), dim3(kBlock), 0, st, sp + done, dp + done, n - done, t);
        return;
    }
    hipLaunchKernelGGL((copy_convert_kernel<TS, TD>), dim3(grid_for(n)), dim3(kBlock), 0, st, sp, dp, n, s);
}

template <typename TS>
int convert_from(const void* src, void* dst, long n, const Strided& s, int dst_dtype, hipStream_t st) {
    using SS = typename Elem<TS>::store_t;
    const auto* sp = static_cast<const SS*>(src);
    switch (dst_dtype) {
        case PARAS_F32:  launch_convert<TS, float>(sp, dst, n, s, st); break;
        case PARAS_F64:  launch_convert<TS, double>(sp, dst, n, s, st); break;
        case PARAS_BF16: launch_convert<TS, bf16_t>(sp, dst, n, s, st); break;
        case PARAS_F16:  launch_convert<TS, f16_t>(sp, dst, n, s, st); break;
        default: return fail(PARAS_ERR_INVALID, "paras_copy_strided: unknown dtype %d", dst_dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_copy_strided(const void* src, void* dst, int ndim, const int64_t* sizes, const int64_t* src_strides,
                       const int64_t* dst_strides, int elem_size, int src_dtype, int dst_dtype, void* stream) {
    using namespace paras;
    Strided s;
    long n = 0;
    int rc = make_spec(ndim, sizes, src_strides, dst_strides, &s, &n);
    if (rc != PARAS_OK) return rc;
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(src && dst, "paras_copy_strided: null pointer");
    hipStream_t st = nullptr;
    rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const dim3 g(grid_for(n)), b(kBlock);
    if (src_dtype == dst_dtype) {
        const bool dense = s.ndim == 0 || (s.ndim == 1 && s.src_strides[0] == 1 && s.dst_strides[0] == 1);
        const long bytes = n * elem_size;
        if (dense && bytes >= 16 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0) {
            const long nvec = bytes / 16;
            hipLaunchKernelGGL(copy_dense_kernel, dim3(static_cast<unsigned>((nvec + kBlock - 1) / kBlock)), b, 0, st,
                               static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), nvec);
            PARAS_HIP_TRY(hipGetLastError());
            const long done = nvec * 16 / elem_size;
            if (done == n) return PARAS_OK;
            // tail of fewer than 16 bytes: the element kernel on what is left
            src = static_cast<const char*>(src) + nvec * 16;
            dst = static_cast<char*>(dst) + nvec * 16;
            n -= done;
            s.ndim = 1; s.sizes[0] = n; s.src_strides[0] = 1; s.dst_strides[0] = 1;
        }
        // Rows contiguous on both sides (innermost strides 1) whose length, strides and bases are
        // multiples of 16 bytes: the same copy with 16-byte elements (head transposes, slices of a fused
        // projection): an eighth of the index arithmetic for 16-bit tensors, and wide accesses.
        if (s.ndim >= 2 && elem_size < 16 && s.src_strides[s.ndim - 1] == 1 && s.dst_strides[s.ndim - 1] == 1 &&
            ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0) {
            const long per = 16 / elem_size;
            bool ok = s.sizes[s.ndim - 1] % per == 0;
            for (int d = 0; d + 1 < s.ndim; ++d) ok = ok && s.src_strides[d] % per == 0 && s.dst_strides[d] % per == 0;
            if (ok) {
                Strided w = s;
                w.sizes[s.ndim - 1] /= per;
                for (int d = 0; d + 1 < s.ndim; ++d) { w.src_strides[d] /= per; w.dst_strides[d] /= per; }
                const long nw = n / per;
                hipLaunchKernelGGL((copy_same_kernel<u32x4>), dim3(grid_for(nw)), b, 0, st, static_cast<const u32x4*>(src),
                                   static_cast<u32x4*>(dst), nw, w);
                PARAS_HIP_TRY(hipGetLastError());
                return PARAS_OK;
            }
        }
        const dim3 g(grid_for(n));
        switch (elem_size) {
            case 1: hipLaunchKernelGGL((copy_same_kernel<uint8_t>), g, b, 0, st, static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), n, s); break;
            case 2: hipLaunchKernelGGL((copy_same_kernel<uint16_t>), g, b, 0, st, static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), n, s); break;
            case 4: hipLaunchKernelGGL((copy_same_kernel<uint32_t>), g, b, 0, st, static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst), n, s); break;
            case 8: hipLaunchKernelGGL((copy_same_kernel<uint64_t>), g, b, 0, st, static_cast<const uint64_t*>(src), static_cast<uint64_t*>(dst), n, s); break;
            default: return fail(PARAS_ERR_UNSUPPORTED, "paras_copy_strided: element size %d", elem_size);
        }
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    switch (src_dtype) {
        case PARAS_F32:  return convert_from<float>(src, dst, n, s, dst_dtype, st);
        case PARAS_F64:  return convert_from<double>(src, dst, n, s, dst_dtype, st);
        case PARAS_BF16: return convert_from<bf16_t>(src, dst, n, s, dst_dtype, st);
        case PARAS_F16:  return convert_from<f16_t>(src, dst, n, s, dst_dtype, st);
        default: return fail(PARAS_ERR_UNSUPPORTED, "paras_copy_strided: conversion from dtype %d", src_dtype);
    }
}

int paras_fill_strided(void* dst, int ndim, const int64_t* sizes, const int64_t* strides, int elem_size,
                       uint64_t value_bits, void* stream) {
    using namespace paras;
    Strided s;
    long n = 0;
    int rc = make_spec(ndim, sizes, nullptr, strides, &s, &n);
    if (rc != PARAS_OK) return rc;
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(dst != nullptr, "paras_fill_strided: null pointer");
    hipStream_t st = nullptr;
    rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const dim3 g(grid_for(n)), b(kBlock);
    switch (elem_size) {
        case 1: hipLaunchKernelGGL((fill_kernel<uint8_t>), g, b, 0, st, static_cast<uint8_t*>(dst), n, s, static_cast<uint8_t>(value_bits)); break;
        case 2: hipLaunchKernelGGL((fill_kernel<uint16_t>), g, b, 0, st, static_cast<uint16_t*>(dst), n, s, static_cast<uint16_t>(value_bits)); break;
        case 4: hipLaunchKernelGGL((fill_kernel<uint32_t>), g, b, 0, st, static_cast<uint32_t*>(dst), n, s, static_cast<uint32_t>(value_bits)); break;
        case 8: hipLaunchKernelGGL((fill_kernel<uint64_t>), g, b, 0, st, static_cast<uint64_t*>(dst), n, s, value_bits); break;
        default: return fail(PARAS_ERR_UNSUPPORTED, "paras_fill_strided: element size %d", elem_size);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

int paras_index_select(const void* src, const int64_t* index, void* dst, int64_t outer, int64_t n_src, int64_t n_index,
                       int64_t inner_bytes, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(outer >= 0 && n_src >= 0 && n_index >= 0 && inner_bytes >= 0, "paras_index_select: negative shape");
    if (outer == 0 || n_index == 0 || inner_bytes == 0) return PARAS_OK;
    PARAS_REQUIRE(n_src > 0, "paras_index_select: cannot select from an empty dimension");
    PARAS_REQUIRE(src && index && dst, "paras_index_select: null pointer");
    hipStream_t st = nullptr;
    int rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const long* idx = reinterpret_cast<const long*>(index);
    const uintptr_t bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | static_cast<uintptr_t>(inner_bytes);
    const int w = (bits % 16 == 0) ? 16 : (bits % 8 == 0) ? 8 : (bits % 4 == 0) ? 4 : (bits % 2 == 0) ? 2 : 1;
    const long inner = inner_bytes / w, total = outer * n_index * inner;
    const dim3 g(grid_for(total)), b(kBlock);
    switch (w) {
        case 16: hipLaunchKernelGGL((gather_rows_kernel<u32x4>), g, b, 0, st, static_cast<const u32x4*>(src), idx, static_cast<u32x4*>(dst), total, (long)n_src, (long)n_index, inner); break;
        case 8:  hipLaunchKernelGGL((gather_rows_kernel<uint64_t>), g, b, 0, st, static_cast<const uint64_t*>(src), idx, static_cast<uint64_t*>(dst), total, (long)n_src, (long)n_index, inner); break;
        case 4:  hipLaunchKernelGGL((gather_rows_kernel<uint32_t>), g, b, 0, st, static_cast<const uint32_t*>(src), idx, static_cast<uint32_t*>(dst), total, (long)n_src, (long)n_index, inner); break;
        case 2:  hipLaunchKernelGGL((gather_rows_kernel<uint16_t>), g, b, 0, st, static_cast<const uint16_t*>(src), idx, static_cast<uint16_t*>(dst), total, (long)n_src, (long)n_index, inner); break;
        default: hipLaunchKernelGGL((gather_rows_kernel<uint8_t>), g, b, 0, st, static_cast<const uint8_t*>(src), idx, static_cast<uint8_t*>(dst), total, (long)n_src, (long)n_index, inner); break;
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

int paras_binary_strided(int op, const void* a, const void* b, void* out, int ndim, const int64_t* sizes,
                         const int64_t* a_strides, const int64_t* b_strides, double alpha, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(op >= kOpAdd && op <= kOpDiv, "paras_binary_strided: unknown op %d", op);
    Strided s;
    long n = 0;
    int rc = make_spec(ndim, sizes, a_strides, b_strides, &s, &n);
    if (rc != PARAS_OK) return rc;
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(a && b && out, "paras_binary_strided: null pointer");
    hipStream_t st = nullptr;
    rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const dim3 g(grid_for(n)), blk(kBlock);
    if (dtype == PARAS_BF16 || dtype == PARAS_F16) {
        // a dense; b dense, a single value, or a trailing block repeated over the leading dims
        long brow = -1;
        if (s.ndim <= 1 && (s.ndim == 0 || s.src_strides[0] == 1)) {
            if (s.ndim == 0 || s.dst_strides[0] == 1) brow = n;
            else if (s.dst_strides[0] == 0) brow = 0;
        } else if (s.ndim == 2 && s.src_strides[1] == 1 && s.src_strides[0] == s.sizes[1] && s.dst_strides[1] == 1 &&
                   s.dst_strides[0] == 0) {
            brow = s.sizes[1];
        }
        const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
        if (brow >= 0 && aligned && n % 8 == 0 && brow % 8 == 0) {
            const long nvec = n / 8;
            const dim3 gv(static_cast<unsigned>((nvec + kBlock - 1) / kBlock));
            if (dtype == PARAS_BF16)
                hipLaunchKernelGGL((binary_vec16_kernel<bf16_t>), gv, blk, 0, st, op, static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b), static_cast<uint16_t*>(out), nvec, brow / 8, alpha);
            else
                hipLaunchKernelGGL((binary_vec16_kernel<f16_t>), gv, blk, 0, st, op, static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b), static_cast<uint16_t*>(out), nvec, brow / 8, alpha);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
    }
    switch (dtype) {
        case PARAS_F32:  hipLaunchKernelGGL((binary_strided_kernel<float>), g, blk, 0, st, op, static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(out), n, s, alpha); break;
        case PARAS_F64:  hipLaunchKernelGGL((binary_strided_kernel<double>), g, blk, 0, st, op, static_cast<const double*>(a), static_cast<const double*>(b), static_cast<double*>(out), n, s, alpha); break;
        case PARAS_BF16: hipLaunchKernelGGL((binary_strided_kernel<bf16_t>), g, blk, 0, st, op, static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b), static_cast<uint16_t*>(out), n, s, alpha); break;
        case PARAS_F16:  hipLaunchKernelGGL((binary_strided_kernel<f16_t>), g, blk, 0, st, op, static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b), static_cast<uint16_t*>(out), n, s, alpha); break;
        default: return fail(PARAS_ERR_INVALID, "paras_binary_strided: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

int paras_rms_norm_composed_fwd(const void* x, const void* w, void* out, int64_t rows, int64_t H, double eps,
                                int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(rows >= 0 && H >= 0, "paras_rms_norm_composed_fwd: negative shape");
    if (rows == 0 || H == 0) return PARAS_OK;
    PARAS_REQUIRE(x && out, "paras_rms_norm_composed_fwd: null pointer");
    hipStream_t st = nullptr;
    int rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const dim3 g(static_cast<unsigned>(rows < 65536 ? rows : 65536)), b(kBlock);
    switch (dtype) {
        case PARAS_F32:
            hipLaunchKernelGGL((rms_norm_composed_kernel<float>), g, b, 0, st, static_cast<const float*>(x), static_cast<const float*>(w),
                               static_cast<float*>(out), (long)rows, (long)H, static_cast<double>(static_cast<float>(eps)));
            break;
        case PARAS_F64:
            hipLaunchKernelGGL((rms_norm_composed_kernel<double>), g, b, 0, st, static_cast<const double*>(x), static_cast<const double*>(w),
                               static_cast<double*>(out), (long)rows, (long)H, eps);
            break;
        case PARAS_BF16: {
            // eps narrowed to bf16 on the host exactly as c10::BFloat16(float(eps)) would
            const float ef = static_cast<float>(eps);
            uint32_t u;
            __builtin_memcpy(&u, &ef, 4);
            u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
            float en;
            __builtin_memcpy(&en, &u, 4);
            if (!launch_rms_composed_vec<bf16_t>(x, w, out, rows, H, static_cast<double>(en), g, st))
                hipLaunchKernelGGL((rms_norm_composed_kernel<bf16_t>), g, b, 0, st, static_cast<const uint16_t*>(x),
                                   static_cast<const uint16_t*>(w), static_cast<uint16_t*>(out), (long)rows, (long)H,
                                   static_cast<double>(en));
            break;
        }
        case PARAS_F16: {
            const double en = static_cast<double>(static_cast<float>(static_cast<_Float16>(static_cast<float>(eps))));
            if (!launch_rms_composed_vec<f16_t>(x, w, out, rows, H, en, g, st))
                hipLaunchKernelGGL((rms_norm_composed_kernel<f16_t>), g, b, 0, st, static_cast<const uint16_t*>(x),
                                   static_cast<const uint16_t*>(w), static_cast<uint16_t*>(out), (long)rows, (long)H, en);
            break;
        }
        default: return fail(PARAS_ERR_INVALID, "paras_rms_norm_composed_fwd: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

int paras_swiglu_composed_fwd(const void* x, const void* gate, void* out, int64_t n, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(n >= 0, "paras_swiglu_composed_fwd: negative size");
    if (n == 0) return PARAS_OK;
    PARAS_REQUIRE(x && gate && out, "paras_swiglu_composed_fwd: null pointer");
    hipStream_t st = nullptr;
    int rc = resolve_stream(stream, &st);
    if (rc != PARAS_OK) return rc;
    const dim3 g(grid_for(n)), b(kBlock);
    switch (dtype) {
        case PARAS_F32:  hipLaunchKernelGGL((swiglu_composed_kernel<float>), g, b, 0, st, static_cast<const float*>(x), static_cast<const float*>(gate), static_cast<float*>(out), (long)n); break;
        case PARAS_F64:  hipLaunchKernelGGL((swiglu_composed_kernel<double>), g, b, 0, st, static_cast<const double*>(x), static_cast<const double*>(gate), static_cast<double*>(out), (long)n); break;
        case PARAS_BF16: launch_swiglu_composed16<bf16_t>(x, gate, out, n, st); break;
        case PARAS_F16:  launch_swiglu_composed16<f16_t>(x, gate, out, n, st); break;
        default: return fail(PARAS_ERR_INVALID, "paras_swiglu_composed_fwd: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // extern "C"
