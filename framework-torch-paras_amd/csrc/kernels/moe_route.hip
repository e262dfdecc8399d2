// MoE routing for gfx950: top-k expert selection, gate weights, and the stable
// expert-major permutation of the routed (token, slot) pairs.
//
// The reference has no MoE op; each step is the reference primitive a user
// would compose, with the same tie rules, so every integer output is equal to
// that composition bit for bit:
//   topk     k selection scans over the E logits, each bounded by the previous
//            (value, index); ties go to the lower index
//            (csrc/ops/pointwise_ops.cpp:1325-1378)
//   softmax  over the k kept logits: fp32 in, fp64 inside, fp32 out
//            (csrc/ops/pointwise_ops.cpp:954-977)
//   argsort(stable) of the flattened expert ids (csrc/ops/sort_ops.cpp:129-166)
//            == counting sort: histogram, exclusive scan, stable scatter
//
// Three launches over 256-token workgroups:
//   route_topk     one lane per token (E <= 64 logits are one or two cache
//                  lines); LDS histogram of the workgroup's expert ids
//   route_scan     one 64-lane workgroup turns the per-workgroup histograms
//                  into per-workgroup start positions, counts and offsets
//   route_scatter  rank inside the workgroup from wavefront ballots (a token
//                  hits an expert at most once), plus the start position
#include <hip/hip_runtime.h>

#include <cmath>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "paras_hip.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxExperts = 64;

template <typename T>
__global__ __launch_bounds__(kBlock) void route_topk_kernel(
    const typename Elem<T>::store_t* __restrict__ logits, long T_, int E, int k,
    long* __restrict__ topi, float* __restrict__ topw, int* __restrict__ block_hist) {
    using El = Elem<T>;
    __shared__ int hist[kMaxExperts];
    if (threadIdx.x < kMaxExperts) hist[threadIdx.x] = 0;
    __syncthreads();
    const long t = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (t < T_) {
        const auto* row = logits + t * E;
        double prev_val = 0.0;
        int prev_idx = -1;
        bool has_prev = false;
        double vmax = -INFINITY;
        for (int s = 0; s < k; ++s) {
            double best_val = 0.0;
            int best_idx = -1;
            bool has_best = false;
            for (int j = 0; j < E; ++j) {
                const double v = El::to_f64(row[j]);
                const bool within = !has_prev || (v < prev_val) || (v == prev_val && j > prev_idx);
                if (!within) continue;
                const bool better = !has_best || (v > best_val) || (v == best_val && j < best_idx);
                if (better) {
                    best_val = v;
                    best_idx = j;
                    has_best = true;
                }
            }
            topi[t * k + s] = best_idx;
            prev_val = best_val;
            prev_idx = best_idx;
            has_prev = true;
            if (best_idx >= 0) atomicAdd(&hist[best_idx], 1);
            // softmax input is the kept value as fp32 (topv.float())
            const double vf = static_cast<double>(static_cast<float>(best_val));
            if (vf > vmax) vmax = vf;
        }
        // gate weights: exp(v - max) / sum, fp64, narrowed to fp32
        double sum = 0.0;
        for (int s = 0; s < k; ++s) {
            const long idx = topi[t * k + s];
            const double vf = static_cast<double>(El::to_f32(row[idx >= 0 ? idx : 0]));
            sum += exp(vf - vmax);
        }
        for (int s = 0; s < k; ++s) {
            const long idx = topi[t * k + s];
            const double vf = static_cast<double>(El::to_f32(row[idx >= 0 ? idx : 0]));
            topw[t * k + s] = static_cast<float>(exp(vf - vmax) / sum);
        }
    }
    __syncthreads();
    if (threadIdx.x < E) block_hist[static_cast<long>(blockIdx.x) * E + threadIdx.x] = hist[threadIdx.x];
}

// block_hist[blk][e] -> start position of expert e's entries coming from blk.
__global__ __launch_bounds__(kMaxExperts) void route_scan_kernel(int* __restrict__ block_hist, long nblk,
                                                                  int E, long total, long* __restrict__ counts,
                                                                  long* __restrict__ offsets) {
    __shared__ long cnt[kMaxExperts];
    __shared__ long off[kMaxExperts + 1];
    const int e = threadIdx.x;
    long c = 0;
    if (e < E)
        for (long b = 0; b < nblk; ++b) c += block_hist[b * E + e];
    cnt[e] = e < E ? c : 0;
    __syncthreads();
    if (e == 0) {
        long run = 0;
        for (int i = 0; i < E; ++i) {
            off[i] = run;
            run += cnt[i];
        }
        off[E] = run;  // == total
    }
    __syncthreads();
    if (e < E) {
        counts[e] = cnt[e];
        offsets[e] = off[e];
        long run = off[e];
        for (long b = 0; b < nblk; ++b) {
            const int h = block_hist[b * E + e];
            block_hist[b * E + e] = static_cast<int>(run);
            run += h;
        }
    }
    if (e == 0) offsets[E] = off[E];
    (void)total;
}

__global__ __launch_bounds__(kBlock) void route_scatter_kernel(const long* __restrict__ topi, long T_, int E, int k,
                                                               const int* __restrict__ block_start,
                                                               long* __restrict__ order, long* __restrict__ inv_order) {
    __shared__ int wave_cnt[kWavesPerBlock][kMaxExperts];
    const long t = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const bool live = t < T_;
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (kWave - lane));
    for (int e = 0; e < E; ++e) {
        bool has = false;
        if (live)
            for (int s = 0; s < k; ++s) has |= (topi[t * k + s] == e);
        const unsigned long long mask = __ballot(has);
        if (lane == 0) wave_cnt[wave][e] = __popcll(mask);
    }
    __syncthreads();
    for (int e = 0; e < E; ++e) {
        int mine = -1;
        if (live)
            for (int s = 0; s < k; ++s)
                if (topi[t * k + s] == e) mine = s;
        const unsigned long long mask = __ballot(mine >= 0);
        if (mine >= 0) {
            long pos = block_start[static_cast<long>(blockIdx.x) * E + e] + __popcll(mask & below);
            for (int w = 0; w < wave; ++w) pos += wave_cnt[w][e];
            order[pos] = t * k + mine;
            if (inv_order) inv_order[t * k + mine] = pos;
        }
    }
}

}  // namespace
}  // namespace paras

extern "C" {

size_t paras_moe_route_workspace(int64_t T, int64_t E, int64_t k) {
    (void)k;
    if (T <= 0 || E <= 0) return 0;
    const int64_t nblk = (T + paras::kBlock - 1) / paras::kBlock;
    return static_cast<size_t>(nblk * E) * sizeof(int);
}

int paras_moe_route(const void* logits, int64_t T, int64_t E, int64_t k, int dtype, int64_t* topi,
                    float* topw, int64_t* order, int64_t* inv_order, int64_t* counts, int64_t* offsets,
                    void* workspace, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(T >= 0, "paras_moe_route: negative token count");
    PARAS_REQUIRE(E >= 1 && E <= kMaxExperts, "paras_moe_route: expert count must be in [1, %d]", kMaxExperts);
    PARAS_REQUIRE(k >= 1 && k <= E, "paras topk: k out of range");
    PARAS_REQUIRE(counts && offsets, "paras_moe_route: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    if (T == 0) {
        // fill kernels rather than hipMemsetAsync: the caller may be capturing this stream into a graph
        const int64_t one = 1, ne = E, ne1 = E + 1;
        rc = paras_fill_strided(counts, 1, &ne, &one, 8, 0, stream);
        if (rc != PARAS_OK) return rc;
        return paras_fill_strided(offsets, 1, &ne1, &one, 8, 0, stream);
    }
    PARAS_REQUIRE(logits && topi && topw && order && workspace, "paras_moe_route: null pointer");
    static_assert(sizeof(long) == sizeof(int64_t), "LP64 expected");
    const long nblk = (T + kBlock - 1) / kBlock;
    PARAS_REQUIRE(nblk <= 0x7fffffffL && T * k <= 0x7fffffffL, "paras_moe_route: too many routed rows");
    int* hist = static_cast<int*>(workspace);
    long* ti = reinterpret_cast<long*>(topi);
    const dim3 grid(static_cast<unsigned>(nblk)), block(kBlock);
    switch (dtype) {
        case PARAS_F32:
            hipLaunchKernelGGL((route_topk_kernel<float>), grid, block, 0, s, static_cast<const float*>(logits), (long)T, (int)E, (int)k, ti, topw, hist);
            break;
        case PARAS_F64:
            hipLaunchKernelGGL((route_topk_kernel<double>), grid, block, 0, s, static_cast<const double*>(logits), (long)T, (int)E, (int)k, ti, topw, hist);
            break;
        case PARAS_BF16:
            hipLaunchKernelGGL((route_topk_kernel<bf16_t>), grid, block, 0, s, static_cast<const uint16_t*>(logits), (long)T, (int)E, (int)k, ti, topw, hist);
            break;
        case PARAS_F16:
            hipLaunchKernelGGL((route_topk_kernel<f16_t>), grid, block, 0, s, static_cast<const uint16_t*>(logits), (long)T, (int)E, (int)k, ti, topw, hist);
            break;
        default: return fail(PARAS_ERR_INVALID, "paras_moe_route: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(kMaxExperts), 0, s, hist, nblk, (int)E, (long)(T * k),
                       reinterpret_cast<long*>(counts), reinterpret_cast<long*>(offsets));
    PARAS_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(route_scatter_kernel, grid, block, 0, s, ti, (long)T, (int)E, (int)k, hist,
                       reinterpret_cast<long*>(order), reinterpret_cast<long*>(inv_order));
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // extern "C"
