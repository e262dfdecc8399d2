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
// Up to 65536 tokens: ONE kernel over 256-token workgroups (route_fused_kernel), all of
// them resident at once.  A lane owns a token: its row of logits arrives as one 16-byte
// load (E = 8 of a 16-bit type) and stays in registers for the k selection scans; the
// workgroup counts its tokens per expert with wavefront ballots, publishes the counts,
// stamped with the launch's epoch, and polls the stamped counts of the other workgroups
// (a bounded wait; no counter, no clearing, nothing between the launches of two calls); then
// every workgroup adds up the counts of all workgroups (expert offsets) and of the
// workgroups before it (its own start positions) and scatters its (token, slot) pairs.
// A workgroup whose wait runs out (the others kept off the chip by unrelated work) does
// not depend on them any more: it counts every token's choices itself, from the logits.
//
// More tokens than that: three launches over 256-token workgroups,
//   route_topk     one lane per token; LDS histogram of the workgroup's expert ids
//   route_scan     one 64-lane workgroup turns the per-workgroup histograms
//                  into per-workgroup start positions, counts and offsets
//   route_scatter  rank inside the workgroup from wavefront ballots (a token
//                  hits an expert at most once), plus the start position
#include <hip/hip_runtime.h>

#include <type_traits>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <mutex>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "paras_hip.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxExperts = 256;          // one thread of a workgroup per expert
constexpr int kOwnScratchMaxExperts = 64; // what the library's own scratch areas and the allocation-free entry point are sized for

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


// ---------------------------------------------------------------------------------------
// One-launch routing.  Scratch layout (bytes): [0, kScratchHeader) unused by this path,
// [kScratchHeader ...] u64 words[nblk][E], word = (epoch << 16) | tokens of workgroup b that
// chose expert e.  A word is valid for a launch when its upper bits equal the launch's epoch,
// so the workgroups need no counter to meet at: each polls the words it needs.  Two ways to
// make stale words invalid: the library's own scratch is only ever written by this kernel and
// every launch on it gets an epoch no launch before it had (no clearing at all); scratch a
// caller hands in holds anything, so a fill kernel queued in front zeroes the words and the
// launch uses epoch 1 (this also is the form a graph can replay: the epoch is a kernel
// argument and would be the same on every replay).
constexpr int  kScratchHeader   = 256;
constexpr int  kFusedMaxBlocks  = 256;          // 256-thread workgroups: all resident on 256 CUs
constexpr long kFusedMaxTokens  = static_cast<long>(kFusedMaxBlocks) * kBlock;
// How long a workgroup waits for the others' counts before it counts for itself: by the clock
// (wall_clock64 ticks at 100 MHz), about what the recount costs, so that a grid kept off the chip
// by other work turns a 9 us call into a few hundred microseconds, not tens of milliseconds.
// PARAS_ROUTE_SPIN_LIMIT (a number of polls) is a test hook that forces the recount.
constexpr unsigned kWaitTicks   = 30000;        // 300 us
constexpr int  kSpinLimit       = 1 << 30;
constexpr int  kEpochShift      = 16;           // a workgroup's count is at most kBlock

// Workgroups that stopped waiting and counted for themselves, since the module was loaded
// (read through paras_moe_route_give_ups: a number that grows says the chip is oversubscribed).
static __device__ unsigned long long route_give_ups = 0;

__global__ __launch_bounds__(kBlock) void route_clear_kernel(unsigned long long* __restrict__ words, long n) {
    const long i = static_cast<long>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) words[i] = 0ull;
}

// NR > 0: E <= NR and k <= 8, the row and the selection live in registers -- 8: as doubles (any
// tensor type); 16, 32, 64: as floats, which hold 16-bit and fp32 logits exactly and compare like
// them (not for fp64 tensors).  NR = 0: the row is read from memory in every selection pass and
// the selection back from `topi` for every expert (E x k loads per token, three times over:
// T = 8192, E = 64, k = 8 took 228 us this way, 12 x the time of E = 8, k = 2).
template <typename T, int NR>
__global__ __launch_bounds__(kBlock) void route_fused_kernel(
    const typename Elem<T>::store_t* __restrict__ logits, long T_, int E, int k, long* __restrict__ topi,
    float* __restrict__ topw, long* __restrict__ order, long* __restrict__ inv_order, long* __restrict__ counts,
    long* __restrict__ offsets, unsigned char* __restrict__ scratch, unsigned long long epoch, int spin_limit, unsigned wait_ticks) {
    using El = Elem<T>;
    __shared__ int wave_cnt[kWavesPerBlock][kMaxExperts];
    __shared__ long tot[kMaxExperts + 1];     // after the meeting: exclusive expert offsets
    __shared__ int  all_cnt[kMaxExperts];     // tokens of expert e in all workgroups
    __shared__ int  pre[kMaxExperts];         // tokens of expert e in the workgroups before this one
    __shared__ int  gave_up;
    __shared__ int  recount[2][kMaxExperts];  // only used by a workgroup whose wait ran out
    unsigned long long* words = reinterpret_cast<unsigned long long*>(scratch + kScratchHeader);
    const int nblk = gridDim.x, bid = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const long t = static_cast<long>(bid) * kBlock + tid;
    const bool live = t < T_;
    if (tid == 0) gave_up = 0;
    if (tid < kMaxExperts) {
        all_cnt[tid] = 0;
        pre[tid] = 0;
    }

    // ---- top-k of this lane's token ---------------------------------
    constexpr bool kSmall = NR > 0;
    using V = typename std::conditional<(NR > 8), float, double>::type;     // what the row is held and compared as
    static_assert(NR <= 8 || sizeof(typename El::store_t) <= 4, "fp64 logits do not fit floats");
    int sel[kSmall ? 8 : 1];                  // chosen expert per slot (small path)
    double kept[kSmall ? 8 : 1];              // the kept values as fp32 (the softmax input is topv.float())
    double vmax = -INFINITY;
    if (live) {
        const auto* row = logits + t * E;
        V val[kSmall ? NR : 1];
        if constexpr (NR == 8) {
            if (sizeof(typename El::store_t) == 2 && E == 8 && (reinterpret_cast<std::uintptr_t>(logits) & 15) == 0) {     // the row is one aligned 16-byte load
                const u32x4 w = load16(row);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    val[j] = El::to_f64(static_cast<typename El::store_t>(w[j >> 1] >> (16 * (j & 1))));
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) val[j] = j < E ? El::to_f64(row[j]) : 0.0;
            }
        } else if constexpr (NR > 8) {
            if (sizeof(typename El::store_t) == 2 && E % 8 == 0 && (reinterpret_cast<std::uintptr_t>(logits) & 15) == 0) {  // rows of aligned 16-byte pieces
#pragma unroll
                for (int c = 0; c < NR / 8; ++c) {
                    if (c * 8 < E) {
                        const u32x4 w = load16(row + c * 8);
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            val[c * 8 + j] = static_cast<float>(El::to_f32(static_cast<typename El::store_t>(w[j >> 1] >> (16 * (j & 1)))));
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; ++j) val[c * 8 + j] = 0.f;
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < NR; ++j) val[j] = j < E ? static_cast<float>(El::to_f32(row[j])) : 0.f;
            }
        }
        V prev_val = 0;
        int prev_idx = -1;
        bool has_prev = false;
        for (int s = 0; s < k; ++s) {
            V best_val = 0;
            int best_idx = -1;
            bool has_best = false;
            auto consider = [&](int j, V v) {
                const bool within = !has_prev || (v < prev_val) || (v == prev_val && j > prev_idx);
                const bool better = !has_best || (v > best_val) || (v == best_val && j < best_idx);
                if (within && better) {
                    best_val = v;
                    best_idx = j;
                    has_best = true;
                }
            };
            if constexpr (kSmall) {
#pragma unroll
                for (int j = 0; j < NR; ++j)
                    if (j < E) consider(j, val[j]);
            } else {
                for (int j = 0; j < E; ++j) consider(j, El::to_f64(row[j]));
            }
            topi[t * k + s] = best_idx;
            prev_val = best_val;
            prev_idx = best_idx;
            has_prev = true;
            const double vf = static_cast<double>(static_cast<float>(best_val));
            if (vf > vmax) vmax = vf;
            if constexpr (kSmall) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (i == s) {
                        sel[i] = best_idx;
                        kept[i] = vf;
                    }
            }
        }
    }
    // gate weights: exp(v - max) / sum in fp64, narrowed to fp32 (evaluated after the counts are
    // published, while they travel)
    auto write_gate_weights = [&]() {
        if (!live) return;
        const auto* row = logits + t * E;
        (void)row;
        if constexpr (kSmall) {
            double ex[8], sum = 0.0;
#pragma unroll
            for (int s = 0; s < 8; ++s)
                if (s < k) {
                    ex[s] = exp(kept[s] - vmax);
                    sum += ex[s];
                }
#pragma unroll
            for (int s = 0; s < 8; ++s)
                if (s < k) topw[t * k + s] = static_cast<float>(ex[s] / sum);
        } else {
            double sum = 0.0;
            for (int s = 0; s < k; ++s) {
                const long idx = topi[t * k + s];
                sum += exp(static_cast<double>(El::to_f32(row[idx >= 0 ? idx : 0])) - vmax);
            }
            for (int s = 0; s < k; ++s) {
                const long idx = topi[t * k + s];
                topw[t * k + s] = static_cast<float>(exp(static_cast<double>(El::to_f32(row[idx >= 0 ? idx : 0])) - vmax) / sum);
            }
        }
        };
    // slot in which this lane's token chose expert e, or -1 (a token chooses an expert at most once)
    auto slot_of = [&](int e) -> int {
        int mine = -1;
        if (live) {
            if constexpr (kSmall) {
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    if (s < k && sel[s] == e) mine = s;
            } else {
                for (int s = 0; s < k; ++s)
                    if (topi[t * k + s] == e) mine = s;
            }
        }
        return mine;
    };

    // ---- counts of this workgroup, published for the others ---------------------------
    for (int e = 0; e < E; ++e) {
        const unsigned long long mask = __ballot(slot_of(e) >= 0);
        if (lane == 0) wave_cnt[wave][e] = __popcll(mask);
    }
    __syncthreads();
    if (tid < E) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) c += wave_cnt[w][tid];
        __hip_atomic_store(&words[static_cast<long>(bid) * E + tid], (epoch << kEpochShift) | static_cast<unsigned long long>(c),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    write_gate_weights();

    // ---- meet: a lane polls a word until it carries this launch's epoch -------------------
    {
        bool ran_out = false;
        const long n_words = static_cast<long>(nblk) * E;
        const unsigned long long t_start = wall_clock64();
        for (long i = tid; i < n_words; i += kBlock) {
            const unsigned long long* wp = &words[i];
            unsigned long long w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            int polls = 1;
            while ((w >> kEpochShift) != epoch) {
                if (polls >= spin_limit || wall_clock64() - t_start > wait_ticks) {
                    ran_out = true;
                    break;
                }
                ++polls;
                __builtin_amdgcn_s_sleep(1);
                w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (ran_out) break;
            const int c = static_cast<int>(w & ((1ull << kEpochShift) - 1));
            const int j = static_cast<int>(i / E), e = static_cast<int>(i % E);
            atomicAdd(&all_cnt[e], c);
            if (j < bid) atomicAdd(&pre[e], c);
        }
        if (ran_out) gave_up = 1;
    }
    __syncthreads();
    if (gave_up && tid == 0) atomicAdd(&route_give_ups, 1ull);

    // ---- totals (expert offsets) and the share of the workgroups before this one ---------
    if (gave_up) {
        // The others did not all arrive in time (workgroups of this grid kept off the chip by other
        // work): this workgroup counts every token's choices itself, from the logits, with the same
        // selection rule.  Slow, and independent of anybody else, so the result never depends on
        // which workgroups were resident together.
        for (int e = tid; e < E; e += kBlock) {
            recount[0][e] = 0;
            recount[1][e] = 0;
        }
        __syncthreads();
        for (long j = tid; j < T_; j += kBlock) {
            const auto* rowj = logits + j * E;
            const bool earlier = j / kBlock < bid;
            double prev_val = 0.0;
            int prev_idx = -1;
            bool has_prev = false;
            for (int s = 0; s < k; ++s) {
                double best_val = 0.0;
                int best_idx = -1;
                bool has_best = false;
                for (int i = 0; i < E; ++i) {
                    const double v = El::to_f64(rowj[i]);
                    const bool within = !has_prev || (v < prev_val) || (v == prev_val && i > prev_idx);
                    const bool better = !has_best || (v > best_val) || (v == best_val && i < best_idx);
                    if (within && better) {
                        best_val = v;
                        best_idx = i;
                        has_best = true;
                    }
                }
                if (best_idx >= 0) {
                    atomicAdd(&recount[0][best_idx], 1);
                    if (earlier) atomicAdd(&recount[1][best_idx], 1);
                }
                prev_val = best_val;
                prev_idx = best_idx;
                has_prev = true;
            }
        }
        __syncthreads();
        for (int e = tid; e < E; e += kBlock) {
            all_cnt[e] = recount[0][e];
            pre[e] = recount[1][e];
        }
        __syncthreads();
    }
    // exclusive scan over the experts by the first wave: a lane takes kMaxExperts / 64 consecutive
    // experts (totals below 2^31)
    if (wave == 0) {
        constexpr int kPerLane = kMaxExperts / kWave;
        int c[kPerLane], mine = 0;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const int e = lane * kPerLane + i;
            c[i] = e < E ? all_cnt[e] : 0;
            mine += c[i];
        }
        int incl = mine;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const int up = __shfl_up(incl, d, kWave);
            if (lane >= d) incl += up;
        }
        int run = incl - mine;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const int e = lane * kPerLane + i;
            if (e < E) {
                tot[e] = run;
                if (bid == 0) {
                    counts[e] = c[i];
                    offsets[e] = run;
                    if (e == E - 1) offsets[E] = run + c[i];
                }
            }
            run += c[i];
        }
    }
    __syncthreads();

    // ---- stable scatter: expert offset + earlier workgroups + earlier waves + earlier lanes
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (kWave - lane));
    for (int e = 0; e < E; ++e) {
        const int mine = slot_of(e);
        const unsigned long long mask = __ballot(mine >= 0);
        if (mine >= 0) {
            long pos = tot[e] + pre[e] + __popcll(mask & below);
            for (int w = 0; w < wave; ++w) pos += wave_cnt[w][e];
            order[pos] = t * k + mine;
            if (inv_order) inv_order[t * k + mine] = pos;
        }
    }
}

// epoch 0: `scratch` may hold anything -- its words are zeroed by a fill kernel queued in front and
// the launch runs as epoch 1.  Otherwise `scratch` is the library's own and `epoch` is new to it.
template <typename T>
void launch_fused(const void* logits, long T_, int E, int k, long* topi, float* topw, long* order, long* inv_order,
                  long* counts, long* offsets, unsigned char* scratch, unsigned long long epoch, hipStream_t s) {
    using store_t = typename Elem<T>::store_t;
    const long nblk = (T_ + kBlock - 1) / kBlock;
    const dim3 grid(static_cast<unsigned>(nblk)), block(kBlock);
    // PARAS_ROUTE_SPIN_LIMIT: polls before a workgroup stops waiting for the others (tests set 1 to
    // drive the workgroups through the path that counts for itself)
    const char* env = std::getenv("PARAS_ROUTE_SPIN_LIMIT");   // (looked up per call: the tests switch it between calls)
    const int spin = env != nullptr && std::atoi(env) > 0 ? std::atoi(env) : kSpinLimit;
    if (epoch == 0) {
        const long n_words = nblk * E;
        hipLaunchKernelGGL(route_clear_kernel, dim3(static_cast<unsigned>((n_words + kBlock - 1) / kBlock)), block, 0, s,
                           reinterpret_cast<unsigned long long*>(scratch + kScratchHeader), n_words);
        epoch = 1;
    }
#define PARAS_ROUTE_FUSED(NR_)                                                                                          \
    hipLaunchKernelGGL((route_fused_kernel<T, NR_>), grid, block, 0, s, static_cast<const store_t*>(logits), T_, E, k, topi, \
                       topw, order, inv_order, counts, offsets, scratch, epoch, spin, kWaitTicks)
    constexpr bool kFloats = sizeof(store_t) <= 4;       // 16-bit and fp32 logits: a row of up to 64 fits registers as floats
    if (E <= 8 && k <= 8) PARAS_ROUTE_FUSED(8);
    else if (kFloats && k <= 8 && E <= 16) PARAS_ROUTE_FUSED((kFloats ? 16 : 0));
    else if (kFloats && k <= 8 && E <= 32) PARAS_ROUTE_FUSED((kFloats ? 32 : 0));
    else if (kFloats && k <= 8 && E <= 64) PARAS_ROUTE_FUSED((kFloats ? 64 : 0));
    else PARAS_ROUTE_FUSED(0);
#undef PARAS_ROUTE_FUSED
}

// Shared by the entry points: routes on `scratch` (device memory of route_scratch_bytes(T, E)).
int route_on(const void* logits, long T_, int E, int k, int dtype, long* topi, float* topw, long* order, long* inv_order,
             long* counts, long* offsets, unsigned char* scratch, unsigned long long epoch, hipStream_t s) {
    switch (dtype) {
        case PARAS_F32:  launch_fused<float>(logits, T_, E, k, topi, topw, order, inv_order, counts, offsets, scratch, epoch, s); break;
        case PARAS_F64:  launch_fused<double>(logits, T_, E, k, topi, topw, order, inv_order, counts, offsets, scratch, epoch, s); break;
        case PARAS_BF16: launch_fused<bf16_t>(logits, T_, E, k, topi, topw, order, inv_order, counts, offsets, scratch, epoch, s); break;
        case PARAS_F16:  launch_fused<f16_t>(logits, T_, E, k, topi, topw, order, inv_order, counts, offsets, scratch, epoch, s); break;
        default: return fail(PARAS_ERR_INVALID, "paras_moe_route: unknown dtype %d", dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

// Bytes a caller's workspace must hold: the words of the one-launch path (8 bytes each), which also
// covers the int histograms of the three-launch path.
size_t route_scratch_bytes(long T_, long E) {
    const long nblk = (T_ + kBlock - 1) / kBlock;
    return static_cast<size_t>(kScratchHeader) + static_cast<size_t>(nblk * E) * sizeof(unsigned long long);
}


// ---------------------------------------------------------------------------------------
// Scratch of the allocation-free entry point: one copy per GPU, held until the process ends.
// Its name is a host-side stand-in, not a device address: host code only ever uses the
// per-device address hipGetSymbolAddress returns (static_scratch_for below).
constexpr size_t kStaticScratchBytes = static_cast<size_t>(kScratchHeader) + static_cast<size_t>(kFusedMaxBlocks) * kOwnScratchMaxExperts * sizeof(unsigned long long);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxGpus = 64;
std::mutex g_scratch_mutex;
unsigned char* g_scratch_ptr[kMaxGpus] = {};

// Address of `scratch` on the calling thread's current device, resolved once per device.
int static_scratch_for(unsigned char** out) {
    int dev = -1;
    PARAS_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxGpus) return fail(PARAS_ERR_UNSUPPORTED, "paras_moe_route_noalloc: device index %d beyond %d", dev, kMaxGpus);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        PARAS_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return fail(PARAS_ERR_HIP, "paras_moe_route_noalloc: no device address for the scratch array");
        g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return PARAS_OK;
}

// ---------------------------------------------------------------------------------------
// The library's own scratch for paras_moe_route: kEpochSlots areas per GPU that only
// route_fused_kernel ever writes (zero when the module is loaded), one per stream by a hash of the
// stream handle: calls on one stream run one after the other anyway, calls on different streams
// rarely share an area.  If two launches do share one, each sees the other's epoch in some words,
// waits its time out and counts for itself: slower, never wrong.  As for `scratch`, host code
// uses the per-device address only.
constexpr int kEpochSlots = 8;
static __device__ __align__(256) unsigned char epoch_scratch[kEpochSlots * kStaticScratchBytes];
unsigned char* g_epoch_scratch_ptr[kMaxGpus] = {};
std::atomic<unsigned long long> g_epoch{2};        // 0: "clear first", 1: the epoch of a cleared area

int epoch_scratch_for(hipStream_t s, unsigned char** out) {
    int dev = -1;
    // the device the launch goes to: the stream's, or the current one for the null stream
    if (s == nullptr || hipStreamGetDevice(s, &dev) != hipSuccess) {
        (void)hipGetLastError();
        PARAS_HIP_TRY(hipGetDevice(&dev));
    }
    if (dev < 0 || dev >= kMaxGpus) {
        *out = nullptr;          // beyond the table: the caller's workspace serves
        return PARAS_OK;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_epoch_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        PARAS_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(epoch_scratch)));
        if (ptr == nullptr) return fail(PARAS_ERR_HIP, "paras_moe_route: no device address for the routing scratch");
        g_epoch_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
    }
    const uintptr_t h = reinterpret_cast<uintptr_t>(s);
    const size_t slot = static_cast<size_t>(((h >> 4) * 0x9E3779B97F4A7C15ull) >> 61);   // top three bits: kEpochSlots == 8
    static_assert(kEpochSlots == 8, "the hash above yields three bits");
    *out = g_epoch_scratch_ptr[dev] + slot * kStaticScratchBytes;
    return PARAS_OK;
}

// True when work queued on `s` now is being recorded into a graph (or that cannot be told).
bool stream_is_capturing(hipStream_t s) {
    if (s == nullptr) return false;   // the null stream cannot be captured, and asking would disturb a capture elsewhere
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &status) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return status != hipStreamCaptureStatusNone;
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_moe_route_give_ups(uint64_t* count) {
    using namespace paras;
    PARAS_REQUIRE(count != nullptr, "paras_moe_route_give_ups: null pointer");
    unsigned long long n = 0;
    PARAS_HIP_TRY(hipMemcpyFromSymbol(&n, HIP_SYMBOL(route_give_ups), sizeof(n)));
    *count = n;
    return PARAS_OK;
}

size_t paras_moe_route_workspace(int64_t T, int64_t E, int64_t k) {
    (void)k;
    if (T <= 0 || E <= 0) return 0;
    return paras::route_scratch_bytes(T, E);
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
    long* ti = reinterpret_cast<long*>(topi);
    if (T <= kFusedMaxTokens) {
        // One launch on the library's own scratch with a fresh epoch.  A stream that is being captured
        // into a graph gets the replayable form instead (the workspace's words zeroed by a fill kernel
        // in front, epoch 1); PARAS_ROUTE_OWN_SCRATCH=0 asks for that form everywhere.
        unsigned char* area = static_cast<unsigned char*>(workspace);
        unsigned long long epoch = 0;
        const char* own = std::getenv("PARAS_ROUTE_OWN_SCRATCH");
        if ((own == nullptr || std::atoi(own) != 0) && E <= kOwnScratchMaxExperts && !stream_is_capturing(s)) {
            unsigned char* base = nullptr;
            rc = epoch_scratch_for(s, &base);
            if (rc != PARAS_OK) return rc;
            if (base != nullptr) {
                area = base;
                epoch = g_epoch.fetch_add(1, std::memory_order_relaxed);
            }
        }
        return route_on(logits, T, (int)E, (int)k, dtype, ti, topw, reinterpret_cast<long*>(order), reinterpret_cast<long*>(inv_order),
                        reinterpret_cast<long*>(counts), reinterpret_cast<long*>(offsets), area, epoch, s);
    }
    int* hist = reinterpret_cast<int*>(static_cast<unsigned char*>(workspace) + kScratchHeader);
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

int paras_moe_route_noalloc(const void* logits, int64_t T, int64_t E, int64_t k, int dtype, int64_t* topi,
                            float* topw, int64_t* order, int64_t* inv_order, int64_t* counts, int64_t* offsets,
                            void* stream) {
    using namespace paras;
    PARAS_REQUIRE(T >= 1, "paras_moe_route_noalloc: at least one token is required");
    PARAS_REQUIRE(T <= kFusedMaxTokens, "paras_moe_route_noalloc: %lld tokens exceed the static scratch (at most %ld tokens)",
                  static_cast<long long>(T), kFusedMaxTokens);
    PARAS_REQUIRE(E >= 1 && E <= kOwnScratchMaxExperts, "paras_moe_route_noalloc: expert count must be in [1, %d] (the static scratch is sized for that)", kOwnScratchMaxExperts);
    PARAS_REQUIRE(k >= 1 && k <= E, "paras topk: k out of range");
    PARAS_REQUIRE(T * k <= 0x7fffffffL, "paras_moe_route_noalloc: too many routed rows");
    PARAS_REQUIRE(logits && topi && topw && order && counts && offsets, "paras_moe_route_noalloc: null pointer");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    unsigned char* ptr = nullptr;
    rc = static_scratch_for(&ptr);
    if (rc != PARAS_OK) return rc;
    // Epoch 0: the words of the scratch that this call uses are zeroed by the fill kernel route_on
    // queues first (the form a graph can replay).
    return route_on(logits, T, (int)E, (int)k, dtype, reinterpret_cast<long*>(topi), topw, reinterpret_cast<long*>(order),
                    reinterpret_cast<long*>(inv_order), reinterpret_cast<long*>(counts), reinterpret_cast<long*>(offsets), ptr, 0ull, s);
}

}  // extern "C"
