// Scaled-dot-product attention as the reference composes it
// (csrc/ops/attention_ops.cpp:101-135), step by step on the device, for the
// problems no fused kernel takes and the general one-row-per-workgroup kernel
// would crawl through (fp32 / fp64 tensors, unusual head sizes or layouts at
// sequence lengths in the thousands):
//   s = T(q k^T)                     the batched product (paras_gemm_nt: fp32 accumulation,
//                                    fp64 for fp64 tensors, one rounding to T)
//   s = T(s * scale); -inf where masked / T(s + bias); p = T(softmax(s))   one row kernel, fp64
//   o = T(p v)                       the batched product again, against v transposed once
// The scores live in the caller's weights tensor when it asks for one, else in
// the workspace, a bounded piece at a time (a few heads, or a block of query
// rows of one head).  Each step narrows to T exactly where the reference's
// ops do, so results differ from the general kernel (which sums the products
// in fp64) only through the products' summation order.
#include <hip/hip_runtime.h>
#include <type_traits>

#include <algorithm>
#include <cmath>
#include <cstdlib>

#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_internal.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr long kScoreCapBytes = 1L << 30;        // scores held at a time: 1 GiB whatever the element type
size_t up256(size_t n) { return (n + 255) / 256 * 256; }
int elem_size(int dtype) { return dtype == PARAS_F64 ? 8 : dtype == PARAS_F32 ? 4 : 2; }
// The bound in elements.  PARAS_SDPA_SCORE_CAP (elements) lowers it, so that tests reach the
// piecewise forms at small sizes (looked up per call: the tests switch it between calls; a caller
// that changes it between paras_sdpa_workspace and paras_sdpa_fwd gets the workspace check's error).
long score_cap(int dtype) {
    const long cap = kScoreCapBytes / elem_size(dtype);
    const char* v = getenv("PARAS_SDPA_SCORE_CAP");
    const long n = v ? atol(v) : 0;
    return n > 0 && n < cap ? n : cap;
}

// vt[(b*Hkv + h)][d][j] = v[b][h][j][d]
template <typename S>
__global__ __launch_bounds__(kBlock) void transpose_v_kernel(const S* __restrict__ v, S* __restrict__ vt, long Hkv, long Lk, long Dv,
                                                            long vs0, long vs1, long vs2) {
    __shared__ S tile[32][33];
    const long bh = blockIdx.z;
    const long b = bh / Hkv, h = bh % Hkv;
    const S* src = v + b * vs0 + h * vs1;
    S* dst = vt + bh * Dv * Lk;
    const long j0 = static_cast<long>(blockIdx.x) * 32, d0 = static_cast<long>(blockIdx.y) * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;          // 32 x 8
    for (int r = ty; r < 32; r += 8) {
        const long j = j0 + r, d = d0 + tx;
        if (j < Lk && d < Dv) tile[r][tx] = src[j * vs2 + d];
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const long d = d0 + r, j = j0 + tx;
        if (d < Dv && j < Lk) dst[d * Lk + j] = tile[tx][r];
    }
}

struct RowsParams {
    void* scores;             // [heads][rows][Lk], a head every head_stride elements
    const void* mask;
    float* lse;               // [B, Hq, Lq] or null
    long heads, rows, Lk, Lq, Hq;
    long b, h0, i0;           // batch, first head and first query row of this piece
    long head_stride;
    long ms[4];
    int mask_kind, is_causal;
    double scale;
};

__device__ __forceinline__ double block_reduce(double v, double* slots, bool is_max) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const double o = __shfl_xor(v, off, kWave);
        v = is_max ? fmax(v, o) : v + o;
    }
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) slots[threadIdx.x / kWave] = v;
    __syncthreads();
    double t = slots[0];
#pragma unroll
    for (int i = 1; i < kWaves; ++i) t = is_max ? fmax(t, slots[i]) : t + slots[i];
    return t;
}

// One workgroup per score row, in place: scale, mask, softmax in fp64, every step narrowed to T
// as the reference's mul / masked_fill / add / _softmax do.
template <typename T>
__global__ __launch_bounds__(kBlock) void scale_mask_softmax_rows_kernel(const RowsParams p) {
    using E = Elem<T>;
    using S = typename E::store_t;
    __shared__ double slots[kWaves];
    for (long r = blockIdx.x; r < p.heads * p.rows; r += gridDim.x) {
        const long hh = r / p.rows, ri = r % p.rows;
        const long hg = p.h0 + hh, i = p.i0 + ri;                    // hg counts on through the batches when they are taken together
        const long b = p.b + hg / p.Hq, h = hg % p.Hq;
        S* row = static_cast<S*>(p.scores) + hh * p.head_stride + ri * p.Lk;
        const long mrow = b * p.ms[0] + h * p.ms[1] + i * p.ms[2];
        auto value = [&](long j) -> double {
            double s = E::to_f64(E::from_f64(E::to_f64(row[j]) * p.scale));
            if (p.is_causal) {
                if (j > i) s = -INFINITY;
            } else if (p.mask_kind == 1) {
                if (static_cast<const unsigned char*>(p.mask)[mrow + j * p.ms[3]] == 0) s = -INFINITY;
            } else if (p.mask_kind == 2) {
                s = E::to_f64(E::from_f64(s + E::to_f64(static_cast<const S*>(p.mask)[mrow + j * p.ms[3]])));
            }
            return s;
        };
        double m = -INFINITY;
        for (long j = threadIdx.x; j < p.Lk; j += kBlock) m = fmax(m, value(j));
        m = block_reduce(m, slots, true);
        double sum = 0.0;
        for (long j = threadIdx.x; j < p.Lk; j += kBlock) sum += exp(value(j) - m);
        sum = block_reduce(sum, slots, false);
        for (long j = threadIdx.x; j < p.Lk; j += kBlock) row[j] = E::from_f64(exp(value(j) - m) / sum);
        if (p.lse && threadIdx.x == 0) p.lse[(b * p.Hq + h) * p.Lq + i] = static_cast<float>(m + log(sum));
        __syncthreads();     // slots are reused by the next row
    }
}

// The same for rows of up to kBlock * EPT keys, with each thread's scores held in registers: the scaled,
// masked and narrowed score is formed once instead of three times, there is one exponential per
// score instead of two, and none at all for the keys a causal row cannot see (their weights are
// 0 / sum, as exp(-inf - m) / sum is).  Same sums in the same order as the kernel above.
template <typename T, int EPT>
__global__ __launch_bounds__(kBlock) void scale_mask_softmax_rows_reg_kernel(const RowsParams p) {
    using E = Elem<T>;
    using S = typename E::store_t;
    __shared__ double slots[kWaves];
    for (long r = blockIdx.x; r < p.heads * p.rows; r += gridDim.x) {
        const long hh = r / p.rows, ri = r % p.rows;
        const long hg = p.h0 + hh, i = p.i0 + ri;
        const long b = p.b + hg / p.Hq, h = hg % p.Hq;
        S* row = static_cast<S*>(p.scores) + hh * p.head_stride + ri * p.Lk;
        const long mrow = b * p.ms[0] + h * p.ms[1] + i * p.ms[2];
        const long seen = p.is_causal ? (i + 1 < p.Lk ? i + 1 : p.Lk) : p.Lk;      // keys past it are masked
        double v[EPT];
        double m = -INFINITY;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const long j = threadIdx.x + static_cast<long>(e) * kBlock;
            double s = -INFINITY;
            if (j < seen) {
                s = E::to_f64(E::from_f64(E::to_f64(row[j]) * p.scale));
                if (p.mask_kind == 1 && !p.is_causal) {
                    if (static_cast<const unsigned char*>(p.mask)[mrow + j * p.ms[3]] == 0) s = -INFINITY;
                } else if (p.mask_kind == 2 && !p.is_causal) {
                    s = E::to_f64(E::from_f64(s + E::to_f64(static_cast<const S*>(p.mask)[mrow + j * p.ms[3]])));
                }
            }
            v[e] = s;
            m = fmax(m, s);
        }
        m = block_reduce(m, slots, true);
        double sum = 0.0;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const long j = threadIdx.x + static_cast<long>(e) * kBlock;
            v[e] = j < seen ? exp(v[e] - m) : 0.0;
            sum += v[e];
        }
        sum = block_reduce(sum, slots, false);
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const long j = threadIdx.x + static_cast<long>(e) * kBlock;
            if (j < p.Lk) row[j] = E::from_f64(v[e] / sum);
        }
        if (p.lse && threadIdx.x == 0) p.lse[(b * p.Hq + h) * p.Lq + i] = static_cast<float>(m + log(sum));
        __syncthreads();     // slots are reused by the next row
    }
}

// fp32 score rows without a mask tensor (causal or not), a multiple of four keys long and 16-byte aligned:
// the same arithmetic with 16-byte loads and stores, four scores a piece and NV pieces a thread, BLK threads
// a row (the fewest that cover it).  The maximum is taken on the scaled floats (v_max_f32 passes a NaN
// by, as fmax does), the pieces a causal row cannot see cost no exponential, and nothing is tested
// per element but the diagonal.
template <int NV, int BLK>
__global__ __launch_bounds__(BLK) void scale_softmax_rows_f32_vec_kernel(const RowsParams p) {
    constexpr int kNW = BLK / kWave;
    __shared__ float m_slots[kNW];
    __shared__ double s_slots[kNW];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int pieces = static_cast<int>(p.Lk >> 2);
    for (long r = blockIdx.x; r < p.heads * p.rows; r += gridDim.x) {
        const long hh = r / p.rows, ri = r % p.rows;
        const long hg = p.h0 + hh, i = p.i0 + ri;
        const long b = p.b + hg / p.Hq, h = hg % p.Hq;
        float* row = static_cast<float*>(p.scores) + hh * p.head_stride + ri * p.Lk;
        const long seen = p.is_causal ? (i + 1 < p.Lk ? i + 1 : p.Lk) : p.Lk;      // keys past it are masked
        float f[NV][4];
        float m = -INFINITY;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int pc = threadIdx.x + v * BLK;
            const long j0 = 4L * pc;
            u32x4 w = {0u, 0u, 0u, 0u};
            if (pc < pieces && j0 < seen) w = *reinterpret_cast<const u32x4*>(row + j0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const std::uint32_t bits = w[e];
                const float sc = static_cast<float>(static_cast<double>(__builtin_bit_cast(float, bits)) * p.scale);
                f[v][e] = j0 + e < seen ? sc : -INFINITY;
                m = __builtin_fmaxf(m, f[v][e]);
            }
        }
        m = wave_max(m);
        __syncthreads();                 // (the slots of the row before have been read)
        if (lane == 0) m_slots[wave] = m;
        __syncthreads();
        m = m_slots[0];
#pragma unroll
        for (int k = 1; k < kNW; ++k) m = __builtin_fmaxf(m, m_slots[k]);
        const double md = static_cast<double>(m);
        double ex[NV][4], sum = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const long j0 = 4L * (threadIdx.x + v * BLK);
            if (j0 < seen) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ex[v][e] = j0 + e < seen ? exp(static_cast<double>(f[v][e]) - md) : 0.0;
                    sum += ex[v][e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) ex[v][e] = 0.0;
            }
        }
        sum = wave_sum(sum);
        if (lane == 0) s_slots[wave] = sum;
        __syncthreads();
        sum = 0.0;
#pragma unroll
        for (int k = 0; k < kNW; ++k) sum += s_slots[k];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int pc = threadIdx.x + v * BLK;
            if (pc < pieces) {
                u32x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float q = static_cast<float>(ex[v][e] / sum);
                    w[e] = __builtin_bit_cast(std::uint32_t, q);
                }
                *reinterpret_cast<u32x4*>(row + 4L * pc) = w;
            }
        }
        if (p.lse && threadIdx.x == 0) p.lse[(b * p.Hq + h) * p.Lq + i] = static_cast<float>(md + log(sum));
    }
}

bool launch_rows_f32_vec(const RowsParams& rp, unsigned grid, hipStream_t s) {
    if (rp.mask_kind != 0 && !rp.is_causal) return false;
    if (rp.Lk % 4 != 0 || rp.Lk > 32 * 1024 || rp.head_stride % 4 != 0 || (reinterpret_cast<uintptr_t>(rp.scores) & 15) != 0) return false;
    const long pieces = rp.Lk / 4;
    const dim3 g(grid);
    if (pieces <= 64)        hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<1, 64>), g, dim3(64), 0, s, rp);
    else if (pieces <= 128)  hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<1, 128>), g, dim3(128), 0, s, rp);
    else if (pieces <= 256)  hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<1, 256>), g, dim3(256), 0, s, rp);
    else if (pieces <= 512)  hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<2, 256>), g, dim3(256), 0, s, rp);
    else if (pieces <= 1024) hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<4, 256>), g, dim3(256), 0, s, rp);
    else if (pieces <= 2048) hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<8, 256>), g, dim3(256), 0, s, rp);
    else                     hipLaunchKernelGGL((scale_softmax_rows_f32_vec_kernel<8, 1024>), g, dim3(1024), 0, s, rp);
    return true;
}

template <typename T>
void launch_rows(const RowsParams& rp, unsigned grid, hipStream_t s) {
    if constexpr (std::is_same<T, float>::value) {
        if (launch_rows_f32_vec(rp, grid, s)) return;
    }
    if (rp.Lk <= 4 * kBlock)       hipLaunchKernelGGL((scale_mask_softmax_rows_reg_kernel<T, 4>), dim3(grid), dim3(kBlock), 0, s, rp);
    else if (rp.Lk <= 16 * kBlock) hipLaunchKernelGGL((scale_mask_softmax_rows_reg_kernel<T, 16>), dim3(grid), dim3(kBlock), 0, s, rp);
    else                           hipLaunchKernelGGL((scale_mask_softmax_rows_kernel<T>), dim3(grid), dim3(kBlock), 0, s, rp);
}

struct Plan {
    long heads;        // q heads per piece (a multiple of rep, or rep itself)
    long rows;         // query rows per piece
    size_t vt_bytes, score_bytes;
};

// One q head per kv head and batches that sit a whole number of heads apart: batch and head form
// one run of heads, and a piece may span batches (fewer, larger library calls).
bool heads_run_on(const paras_sdpa_args& a) {
    return a.Hq == a.Hkv && a.q_strides[0] == a.Hq * a.q_strides[1] && a.k_strides[0] == a.Hkv * a.k_strides[1];
}

Plan make_plan(const paras_sdpa_args& a) {
    const long rep = a.Hq / a.Hkv;
    const long per_head = a.Lq * a.Lk;
    const long head_run = heads_run_on(a) ? a.B * a.Hq : a.Hq;
    Plan pl{};
    if (per_head * rep <= score_cap(a.dtype)) {
        pl.rows = a.Lq;
        pl.heads = rep == 1 ? std::min<long>(head_run, std::max<long>(1, score_cap(a.dtype) / per_head)) : rep;
    } else {
        pl.heads = rep;
        pl.rows = std::max<long>(1, score_cap(a.dtype) / (a.Lk * rep));
    }
    const size_t es = static_cast<size_t>(elem_size(a.dtype));
    pl.vt_bytes = up256(static_cast<size_t>(a.B * a.Hkv * a.Dv * a.Lk) * es);
    pl.score_bytes = a.attn ? 0 : up256(static_cast<size_t>(pl.heads * pl.rows * a.Lk) * es);
    return pl;
}

}  // namespace

// Large enough that a handful of library calls cost less than the general kernel's scalar fp64 dot
// products (which it forms three times per score), and addressable by the products (32-bit element
// offsets inside one operand).
bool composed_supported(const paras_sdpa_args& a) {
    if (a.Lq < 64 || a.Lk < 64 || a.D < 1 || a.Dv < 1) return false;
    const double macs = static_cast<double>(a.B) * a.Hq * a.Lq * a.Lk * (a.D + a.Dv);
    if (macs < static_cast<double>(1L << 25)) return false;          // measured: level with the general kernel at 1.7e7, 2.6x faster at 6.7e7
    const long rep = a.Hq / a.Hkv;
    if (a.Lk * rep > score_cap(a.dtype)) return false;                        // not even one row block fits
    if (a.Lq * a.Lk >= (1L << 31) || a.Lk * a.Dv >= (1L << 31)) return false;
    if (a.q_strides[2] < a.D || a.k_strides[2] < a.D) return false;   // rows the products cannot take (expanded or overlapping views)
    if (a.B * a.Hkv > 65535 || (a.Dv + 31) / 32 > 65535 || a.B * a.Hq > 65535) return false;   // grid limits of the transpose and the batched products
    return true;
}

size_t composed_workspace(const paras_sdpa_args& a) {
    const Plan pl = make_plan(a);
    return pl.vt_bytes + pl.score_bytes;
}

int launch_composed(const paras_sdpa_args& a, void* workspace, void* stream, hipStream_t s) {
    PARAS_REQUIRE(workspace != nullptr, "paras sdpa: workspace is null");
    PARAS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "paras sdpa: the workspace must be 256-byte aligned");
    const Plan pl = make_plan(a);
    const int es = elem_size(a.dtype);
    char* vt = static_cast<char*>(workspace);
    char* score_ws = vt + pl.vt_bytes;
    const long rep = a.Hq / a.Hkv;

    // v transposed once: the second product reads it along the keys
    {
        const dim3 grid(static_cast<unsigned>((a.Lk + 31) / 32), static_cast<unsigned>((a.Dv + 31) / 32), static_cast<unsigned>(a.B * a.Hkv));
#define PARAS_TRANSPOSE_V(S_)                                                                                                   \
    hipLaunchKernelGGL((transpose_v_kernel<S_>), grid, dim3(kBlock), 0, s, static_cast<const S_*>(a.v), reinterpret_cast<S_*>(vt), \
                       (long)a.Hkv, (long)a.Lk, (long)a.Dv, (long)a.v_strides[0], (long)a.v_strides[1], (long)a.v_strides[2])
        if (es == 8)      PARAS_TRANSPOSE_V(double);
        else if (es == 4) PARAS_TRANSPOSE_V(float);
        else              PARAS_TRANSPOSE_V(std::uint16_t);
#undef PARAS_TRANSPOSE_V
        PARAS_HIP_TRY(hipGetLastError());
    }

    const bool run_on = heads_run_on(a);
    const long n_batches = run_on ? 1 : a.B, n_heads = run_on ? a.B * a.Hq : a.Hq;
    for (long b = 0; b < n_batches; ++b)
        for (long h0 = 0; h0 < n_heads; h0 += pl.heads) {
            const long nh = std::min<long>(pl.heads, n_heads - h0);
            const long hkv0 = h0 / rep;
            for (long i0 = 0; i0 < a.Lq; i0 += pl.rows) {
                const long nr = std::min<long>(pl.rows, a.Lq - i0);
                // where this piece's scores live and how far apart its heads are
                char* sc;
                long head_stride;
                if (a.attn) {
                    sc = static_cast<char*>(a.attn) + (((b * a.Hq + h0) * a.Lq + i0) * a.Lk) * es;
                    head_stride = a.Lq * a.Lk;
                } else {
                    sc = score_ws;
                    head_stride = nr * a.Lk;
                }
                const char* qp = static_cast<const char*>(a.q) + (b * a.q_strides[0] + h0 * a.q_strides[1] + i0 * a.q_strides[2]) * es;
                const char* kp = static_cast<const char*>(a.k) + (b * a.k_strides[0] + hkv0 * a.k_strides[1]) * es;
                // q heads of one kv head share its keys (stride 0); with one q head per kv head the heads step together
                const long k_step = rep == 1 ? a.k_strides[1] : 0;
                // (causal: the score tiles wholly past the diagonal are neither formed nor, below, multiplied -- the row
                // kernels read a row only as far as its query sees and write all of it)
                int rc = gemm_nt_causal(qp, kp, nullptr, sc, nr, a.Lk, a.D, a.q_strides[2], a.k_strides[2], a.Lk, 0, nh, a.q_strides[1],
                                        k_step, head_stride, 0, 1.0, 0.0, a.dtype, nullptr, 0, stream, a.is_causal ? 1 : 0, i0);
                if (rc != PARAS_OK) return rc;

                RowsParams rp{};
                rp.scores = sc; rp.mask = a.mask; rp.lse = a.lse;
                rp.heads = nh; rp.rows = nr; rp.Lk = a.Lk; rp.Lq = a.Lq; rp.Hq = a.Hq;
                rp.b = b; rp.h0 = h0; rp.i0 = i0; rp.head_stride = head_stride;
                for (int i = 0; i < 4; ++i) rp.ms[i] = a.mask_strides[i];
                rp.mask_kind = a.mask_kind; rp.is_causal = a.is_causal; rp.scale = a.scale;
                const long nrows = nh * nr;
                const unsigned grid = static_cast<unsigned>(nrows < 256L * 64 ? nrows : 256L * 64);
                switch (a.dtype) {
                    case PARAS_F32:  launch_rows<float>(rp, grid, s); break;
                    case PARAS_F64:  launch_rows<double>(rp, grid, s); break;
                    case PARAS_BF16: launch_rows<bf16_t>(rp, grid, s); break;
                    default:         launch_rows<f16_t>(rp, grid, s); break;
                }
                PARAS_HIP_TRY(hipGetLastError());

                const char* vp = vt + ((b * a.Hkv + hkv0) * a.Dv * a.Lk) * es;
                char* op = static_cast<char*>(a.out) + (((b * a.Hq + h0) * a.Lq + i0) * a.Dv) * es;
                rc = gemm_nt_causal(sc, vp, nullptr, op, nr, a.Dv, a.Lk, a.Lk, a.Lk, a.Dv, 0, nh, head_stride,
                                    rep == 1 ? a.Dv * a.Lk : 0, a.Lq * a.Dv, 0, 1.0, 0.0, a.dtype, nullptr, 0, stream, a.is_causal ? 2 : 0, i0);
                if (rc != PARAS_OK) return rc;
            }
        }
    return PARAS_OK;
}

}  // namespace paras
