// MoE grouped expert FFN for gfx950: two grouped GEMMs on bf16/fp16 MFMA with
// fp32 accumulation, and the weighted combine.
//
//   GEMM 1   h[p, :] = T( silu(T(xp W_gate[e]^T)) * T(xp W_up[e]^T) )
//            xp = x[order[p] / k] is gathered inside the A-tile load (no
//            permuted copy of x is ever written); gate and up columns of the
//            same tile are accumulated side by side and the SwiGLU runs in
//            the epilogue on the values already rounded to T, as the composed
//            reference would see them (mm -> T, paras::swiglu -> T).
//   GEMM 2   y[p, :] = T( h[p, :] W_down[e]^T )
//   combine  out[t] = T( sum_slot T( y[inv_order[t*k+slot]] * T(topw[t][slot]) ) )
//
// Both products are "NT": A rows and weight rows are contiguous along the
// contraction dim, which is exactly the 8-element-per-lane operand layout of
// v_mfma_f32_32x32x16, so neither operand needs a transpose.
//
// Tiling (gemm_tile.h): a workgroup computes 128 or 256 routed rows x two
// 128-column groups (gate and up columns n0..n0+127 for GEMM 1; columns
// n0..n0+255 for GEMM 2), k-tile 64.  128 rows: waves arranged 2x2 with 64x64
// per column group each (128 fp32 accumulators per lane).  256 rows, when the
// experts hold enough rows for them: four waves with 128 x 128 each on
// v_mfma_f32_16x16x32 (256 accumulators per lane; grouped_gemm_quad16_kernel).
// Global -> registers -> LDS with the next
// k-tile's loads in flight during the MFMAs.  Rows of one expert are contiguous
// in the routed order; m-tiles never straddle experts (the grid is sized for the
// worst case and surplus workgroups exit).  The block index is unscrambled so
// that the workgroups resident on one XCD cover all m-tiles of a few column
// tiles: weight tiles are then shared through that XCD's L2.
#include <hip/hip_runtime.h>
#include <cstdlib>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/gemm_tile.h"
#include "kernels/swiglu_math.h"

namespace paras {
namespace {

using namespace gemm;

struct FfnGemmParams {
    const std::uint16_t* a;     // x [T, K] (gathered) or h [R, K]
    const std::uint16_t* b;     // weights of column group 0, [E, Nw, K]
    const std::uint16_t* b2;    // weights of column group 1 (same layout)
    std::uint16_t* c;           // [R, N]
    const long* order;          // gather index (routed row -> flat (token, slot)); null = direct rows
    const long* offsets;        // [E+1]
    long K, N, Nw, R;           // contraction, output columns, weight rows per expert, routed rows
    int E, k;
    int mt_total;               // upper bound on m-tiles
    int n_units;                // column units (128 output columns for GEMM 1, 256 for GEMM 2)
    int ngt;                    // column units an XCD sweeps together
    unsigned div_m;             // flat (token, slot) index / k as a multiplication: (x * div_m) >> div_s
    int div_s;                  // for every x < 2^30 (a 64-bit division per gathered row is ~150 instructions)
};

// Multiplier and shift with floor(x / d) == (x * m) >> s for all 0 <= x < 2^30, 1 <= d < 2^30:
// s = 30 + ceil(log2 d), m = ceil(2^s / d) < 2^31; the error x * (m d - 2^s) stays below 2^s.
inline void division_by(unsigned d, unsigned* m, int* s) {
    int lg = 0;
    while ((1ull << lg) < d) ++lg;
    *s = 30 + lg;
    *m = static_cast<unsigned>(((1ull << *s) + d - 1) / d);
}

template <typename T, bool kSwiglu, typename S>
__global__ __launch_bounds__(S::kThreads, 2) void grouped_gemm_kernel(const FfnGemmParams p) {
    using El = Elem<T>;
    constexpr int kBM = S::kBM;
    __shared__ __attribute__((aligned(16))) typename S::Lds lds;

    // ---- tile coordinates.  Linear id L: xcd = L % 8 (hardware round-robin);
    // within an XCD walk (column group, m-tile, column-in-group).
    int mt, nu;
    {
        const long L = blockIdx.x;
        const int xcd = static_cast<int>(L & 7);
        const long j = L >> 3;
        const long per_group = static_cast<long>(p.mt_total) * p.ngt;
        const long g = j / per_group, rem = j % per_group;
        mt = static_cast<int>(rem / p.ngt);
        nu = static_cast<int>((g * 8 + xcd) * p.ngt + rem % p.ngt);
        if (nu >= p.n_units) return;
    }
    // m-tile -> (expert, first row)
    int e = 0;
    long row0 = 0, row_end = 0;
    {
        int tiles_before = 0;
        bool found = false;
        for (int i = 0; i < p.E; ++i) {
            const long lo = p.offsets[i], hi = p.offsets[i + 1];
            const int tiles = static_cast<int>((hi - lo + kBM - 1) / kBM);
            if (!found && mt < tiles_before + tiles) {
                e = i;
                row0 = lo + static_cast<long>(mt - tiles_before) * kBM;
                row_end = hi;
                found = true;
            }
            tiles_before += tiles;
        }
        if (!found) return;
    }
    const long n0 = static_cast<long>(nu) * (kSwiglu ? kBN : 2 * kBN);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> register staging: 16-byte chunks, 8 per row of a k-tile
    unsigned a_off[4], b_off[2][S::kBChunks];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * S::kThreads;
        long prow = row0 + (c >> 3);
        if (prow >= row_end) prow = row_end - 1;  // clamp: result rows beyond the expert are not stored
        const long src = p.order ? static_cast<long>((static_cast<unsigned long long>(static_cast<unsigned>(p.order[prow])) * p.div_m) >> p.div_s) : prow;
        a_off[i] = static_cast<unsigned>(src * p.K + (c & 7) * 8);
    }
    // weights of this expert: a uniform base per column group, rows as 32-bit offsets
    const std::uint16_t* const b_base[2] = {p.b + static_cast<long>(e) * p.Nw * p.K, p.b2 + static_cast<long>(e) * p.Nw * p.K};
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < S::kBChunks; ++i) {
            const int c = tid + i * S::kThreads;
            long wrow = (kSwiglu ? n0 : n0 + g * kBN) + (c >> 3);
            if (wrow >= p.Nw) wrow = p.Nw - 1;
            b_off[g][i] = static_cast<unsigned>(wrow * p.K + (c & 7) * 8);
        }
    // An expert's last tile with few rows: the waves share those rows (same sums, a fraction of
    // the time) instead of most of them idling through the contraction.
    if constexpr (S::kShortRows > 0) {
        if (row_end - row0 <= S::kShortRows) {
            float16_t sacc[2];
            S::template short_mainloop<T>(p.a, a_off[0], b_base, b_off, p.K, lds, sacc);
            const long col = n0 + (wave & 3) * 32 + lr;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const long prow = row0 + (wave >> 2) * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
                if (prow >= row_end) continue;
                if (kSwiglu) {
                    if (col < p.N) p.c[prow * p.N + col] = swiglu_from_acc<T>(sacc[0][r], sacc[1][r]);
                } else {
                    if (col < p.N) p.c[prow * p.N + col] = El::from_f32(sacc[0][r]);
                    if (col + kBN < p.N) p.c[prow * p.N + col + kBN] = El::from_f32(sacc[1][r]);
                }
            }
            return;
        }
    }
    float16_t acc[2][2][2];
    S::template mainloop<T>(p.a, a_off, b_base, b_off, p.K, lds, acc);

    // ---- epilogue.  Accumulator lane (column lr, half lh) holds rows (r/4)*8 + 4*lh + r%4.
    // One uniform base, a 32-bit byte offset per lane (the launcher sends output rows of 2^22
    // elements or more elsewhere), rows and columns checked against counts in 32-bit registers,
    // narrowing by the conversion instruction; a 32 x 32 block of the plain product in which a NaN
    // turns up is narrowed again in software, which writes NaNs as the host's types do.
    {
        char* cb = reinterpret_cast<char*>(p.c + row0 * p.N + n0);       // uniform
        const long rows_left = row_end - row0, cols_left = p.N - n0;
        const int nrows = static_cast<int>(rows_left < kBM ? rows_left : kBM) - (wm * 64 + 4 * lh);
        const int ncols = static_cast<int>(cols_left < 2 * kBN ? cols_left : 2 * kBN) - (wn * 64 + lr);
        const unsigned ld2 = static_cast<unsigned>(p.N) * 2u;
        unsigned lane_b = static_cast<unsigned>(wm * 64 + 4 * lh) * ld2 + static_cast<unsigned>(wn * 64 + lr) * 2u;
        asm volatile("" : "+v"(lane_b));       // one add per store from here on
        const bool full = rows_left >= kBM && cols_left >= (kSwiglu ? kBN : 2 * kBN);    // uniform
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                if (kSwiglu) {
                    if (ni * 32 >= ncols) continue;
                    std::uint16_t o[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[r] = swiglu_from_acc<T>(acc[0][mi][ni][r], acc[1][mi][ni][r]);
                    if (full) store_block<true>(cb + ni * 64, lane_b, ld2, mi, nrows, o);
                    else      store_block<false>(cb + ni * 64, lane_b, ld2, mi, nrows, o);
                } else {
#pragma unroll
                    for (int g = 0; g < 2; ++g) {
                        if (g * kBN + ni * 32 >= ncols) continue;
                        std::uint16_t o[16];
                        narrow_block<T>(acc[g][mi][ni], o);
                        char* blk = cb + (g * kBN + ni * 32) * 2;
                        if (full) store_block<true>(blk, lane_b, ld2, mi, nrows, o);
                        else      store_block<false>(blk, lane_b, ld2, mi, nrows, o);
                    }
                }
            }
    }
}

// f(integral_constant<int, I>) for I = 0 .. N-1
template <int... I, typename F>
__device__ __forceinline__ void quad16_static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void quad16_static_for(F&& f) {
    quad16_static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// A wave's queue of SwiGLU values that left the common tier (four of one lane per entry): laid over the
// tile stages once the contraction is done.
struct SwigluQueue {
    static constexpr unsigned kEntries = 1024;
    unsigned where[kEntries];       // (row in the tile) << 16 | column in the column unit
    quad16::float4v gate[kEntries], up[kEntries];
};
static_assert(4 * sizeof(SwigluQueue) <= sizeof(quad16::TileLds), "four queues in the tile stages");

// The same on the four-wave tile of v_mfma_f32_16x16x32 (gemm_tile.h, namespace quad16): what the layer
// runs on when the experts are big enough for 256-row tiles.  Tile coordinates, the search for the
// m-tile's expert and the staging offsets as above (a thread stages eight chunks of A and four per
// column group of B); a lane of accumulator block (i, j) holds row i*16 + lane%16 and columns
// 4*(lane/16) .. + 3 of column block j (group j / 4, columns wn*64 + (j % 4)*16 of it), so gate and
// up of one output sit in blocks j and j + 4 of the same lane and an output row gets 8-byte stores.
template <typename T, bool kSwiglu>
__global__ __launch_bounds__(quad16::kThreads, 1) void grouped_gemm_quad16_kernel(const FfnGemmParams p) {
    using El = Elem<T>;
    constexpr int kBM = quad16::kBM;
    __shared__ __attribute__((aligned(16))) quad16::TileLds lds;
    int mt, nu;
    {
        const long L = blockIdx.x;
        const int xcd = static_cast<int>(L & 7);
        const long j = L >> 3;
        const long per_group = static_cast<long>(p.mt_total) * p.ngt;
        const long g = j / per_group, rem = j % per_group;
        mt = static_cast<int>(rem / p.ngt);
        nu = static_cast<int>((g * 8 + xcd) * p.ngt + rem % p.ngt);
        if (nu >= p.n_units) return;
    }
    int e = 0;
    long row0 = 0, row_end = 0;
    {
        int tiles_before = 0;
        bool found = false;
        for (int i = 0; i < p.E; ++i) {
            const long lo = p.offsets[i], hi = p.offsets[i + 1];
            const int tiles = static_cast<int>((hi - lo + kBM - 1) / kBM);
            if (!found && mt < tiles_before + tiles) {
                e = i;
                row0 = lo + static_cast<long>(mt - tiles_before) * kBM;
                row_end = hi;
                found = true;
            }
            tiles_before += tiles;
        }
        if (!found) return;
    }
    const long n0 = static_cast<long>(nu) * (kSwiglu ? kBN : 2 * kBN);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, kq = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;

    unsigned a_off[8], b_off[2][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = tid + i * quad16::kThreads;
        long prow = row0 + (c >> 3);
        if (prow >= row_end) prow = row_end - 1;  // clamp: result rows beyond the expert are not stored
        const long src = p.order ? static_cast<long>((static_cast<unsigned long long>(static_cast<unsigned>(p.order[prow])) * p.div_m) >> p.div_s) : prow;
        a_off[i] = static_cast<unsigned>(src * p.K + (c & 7) * 8);
    }
    const std::uint16_t* const b_base[2] = {p.b + static_cast<long>(e) * p.Nw * p.K, p.b2 + static_cast<long>(e) * p.Nw * p.K};
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * quad16::kThreads;
            long wrow = (kSwiglu ? n0 : n0 + g * kBN) + (c >> 3);
            if (wrow >= p.Nw) wrow = p.Nw - 1;
            b_off[g][i] = static_cast<unsigned>(wrow * p.K + (c & 7) * 8);
        }
    // four values of one output row: SwiGLU of the gate / up pairs, or the narrowed product
    auto put4 = [&](long prow, long col, const quad16::float4v a0, const quad16::float4v a1, bool nan_here) __attribute__((always_inline)) {
        if (prow >= row_end || col >= p.N) return;
        std::uint16_t o[4];
        if constexpr (kSwiglu) {
            swiglu4_from_acc<T>(a0, a1, o);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = __builtin_expect(nan_here, 0) ? El::from_f32(a0[r]) : El::from_f32_finite(a0[r]);
        }
        if (col + 3 < p.N) {        // (N is a multiple of 64 here and the rows are 16-byte aligned)
            u32x2 w2;
            w2[0] = o[0] | (static_cast<std::uint32_t>(o[1]) << 16);
            w2[1] = o[2] | (static_cast<std::uint32_t>(o[3]) << 16);
            *reinterpret_cast<u32x2*>(p.c + prow * p.N + col) = w2;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (col + r < p.N) p.c[prow * p.N + col + r] = o[r];
        }
    };
    auto any_nan = [&](float probe) { return __builtin_amdgcn_ballot_w64(probe != probe) != 0; };

    if (row_end - row0 <= 64) {     // an expert's last tile with few rows: the waves share them
        quad16::float4v sacc[4][4];
        quad16::short_tile_mainloop<T>(p.a, a_off, b_base, b_off, p.K, lds, sacc);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const long prow = row0 + i * 16 + l16;
            bool nan_here = false;
            if (!kSwiglu) {
                float probe = 0.f;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj)
#pragma unroll
                    for (int r = 0; r < 4; ++r) probe += sacc[i][jj][r];
                nan_here = any_nan(probe);
            }
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const long col = n0 + wave * 32 + cb * 16 + 4 * kq;
                if (kSwiglu) {
                    put4(prow, col, sacc[i][cb], sacc[i][2 + cb], false);
                } else {
                    put4(prow, col, sacc[i][cb], sacc[i][cb], nan_here);
                    put4(prow, col + kBN, sacc[i][2 + cb], sacc[i][2 + cb], nan_here);
                }
            }
        }
        return;
    }
    quad16::float4v acc[8][8];
    quad16::tile_mainloop<T>(p.a, a_off, b_base, b_off, p.K, lds, acc);
    if constexpr (kSwiglu) {
        // About one value in a thousand leaves the common tier of SwiGLU, and where one lane of the 64 does,
        // the whole wave walks through the fp64 formula: at 128 values a lane that happened eight times a tile
        // and cost 4 % of the kernel.  A lane whose four values do not all pass queues them (the accumulators
        // and where they go) in the wave's share of the tile stages, which nobody reads any more; after
        // the last row block (or when the next one might not fit) the wave works its queue off, one value per lane.
        __syncthreads();
        // (the lane's coordinates derived again, from a value the compiler cannot trace: none of this is to
        // occupy a register during the contraction, which has none to spare)
        int t = threadIdx.x;
        asm volatile("" : "+v"(t));
        const int lane = t & 63, wave = t >> 6, l16 = t & 15, kq = (t >> 4) & 3, wm = t >> 7, wn = (t >> 6) & 1;
        SwigluQueue& q = reinterpret_cast<SwigluQueue*>(&lds)[wave];
        const unsigned long long lanes_below = (1ull << lane) - 1ull;
        unsigned queued = 0;      // uniform
        auto work_off = [&]() __attribute__((always_inline)) {
            for (unsigned idx = lane; idx < 4 * queued; idx += 64) {
                const unsigned e = idx >> 2, r = idx & 3, where = q.where[e];
                const float a0 = reinterpret_cast<const float*>(&q.gate[e])[r];
                const float a1 = reinterpret_cast<const float*>(&q.up[e])[r];
                const long qcol = n0 + (where & 0xFFFFu) + r;
                const std::uint16_t v = swiglu_from_acc<T>(a0, a1);
                if (qcol < p.N) p.c[(row0 + (where >> 16)) * p.N + qcol] = v;
            }
            queued = 0;
        };
        quad16_static_for<8>([&](auto I) __attribute__((always_inline)) {
            constexpr int i = decltype(I)::value;
            const int trow = wm * 128 + i * 16 + l16;
            const long prow = row0 + trow;
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                const int tcol = wn * 64 + jb * 16 + 4 * kq;
                const long col = n0 + tcol;
                const bool live = prow < row_end && col < p.N;
                std::uint16_t o[4];
                const bool ok = swiglu4_common_tier<T>(acc[i][jb], acc[i][4 + jb], o);
                if (live && ok) {
                    if (col + 3 < p.N) {
                        u32x2 w2;
                        w2[0] = o[0] | (static_cast<std::uint32_t>(o[1]) << 16);
                        w2[1] = o[2] | (static_cast<std::uint32_t>(o[3]) << 16);
                        *reinterpret_cast<u32x2*>(p.c + prow * p.N + col) = w2;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (col + r < p.N) p.c[prow * p.N + col + r] = o[r];
                    }
                }
                const unsigned long long left = __builtin_amdgcn_ballot_w64(live && !ok);
                if (left != 0) {
                    if (live && !ok) {
                        const unsigned slot = queued + static_cast<unsigned>(__builtin_popcountll(left & lanes_below));
                        q.where[slot] = (static_cast<unsigned>(trow) << 16) | static_cast<unsigned>(tcol);
                        q.gate[slot] = acc[i][jb];
                        q.up[slot] = acc[i][4 + jb];
                    }
                    queued += static_cast<unsigned>(__builtin_popcountll(left));
                }
            }
            // a row block queues 4 x 64 entries at most
            if (i == 7 || queued > SwigluQueue::kEntries - 256) work_off();
        });
        return;
    }
    // (row blocks as constants of the front end: the optimiser's unroller gives up on a loop of 128
    // SwiGLU values with their exact tier, and the accumulators would move to scratch memory)
    quad16_static_for<8>([&](auto I) __attribute__((always_inline)) {
        constexpr int i = decltype(I)::value;
        const long prow = row0 + wm * 128 + i * 16 + l16;
        bool nan_here = false;
        if (!kSwiglu) {
            float probe = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) probe += acc[i][j][r];
            nan_here = any_nan(probe);
        }
#pragma unroll
        for (int jb = 0; jb < 4; ++jb) {
            const long col = n0 + wn * 64 + jb * 16 + 4 * kq;
            if (kSwiglu) {
                put4(prow, col, acc[i][jb], acc[i][4 + jb], false);
            } else {
                put4(prow, col, acc[i][jb], acc[i][jb], nan_here);
                put4(prow, col + kBN, acc[i][4 + jb], acc[i][4 + jb], nan_here);
            }
        }
    });
}

// ---- few rows per expert (decode-time batches): the layer is bound by streaming every active
// expert's weights once, which 128-row tiles with a handful of live rows do at half the memory
// rate (and a single token, two active experts, at a fifth of it: its down-projection is 32
// workgroups).  Here, as in the dense few-row kernel: a workgroup owns 16 weight rows of one expert
// (for the gate-up GEMM the 16 gate rows and the 16 up rows of the same columns), its eight waves
// split the contraction in pieces of 64 and feed v_mfma_f32_16x16x32 straight from global memory
// (weights as the row operand; the expert's few routed rows, from L2, as the other), the eight
// partial results meet in LDS in wave order.  An expert's rows are taken MB x 16 at a time, so any
// count works (the weights of a second pass come from L2); experts without rows return at once.
template <typename T> struct Mma16x16;
template <> struct Mma16x16<bf16_t> {
    __device__ static __forceinline__ float4_t run(u32x4 a, u32x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma16x16<f16_t> {
    __device__ static __forceinline__ float4_t run(u32x4 a, u32x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

constexpr int kFewWaves = 8;

template <typename T, bool kSwiglu, int MB>
__global__ __launch_bounds__(kFewWaves * 64) void grouped_few_rows_kernel(const FfnGemmParams p) {
    using El = Elem<T>;
    constexpr int NB = kSwiglu ? 2 : 1;                 // weight blocks: gate and up, or one
    __shared__ float4_t part[kFewWaves][NB * MB][64];
    const int e = blockIdx.y;
    const long row_lo = p.offsets[e], row_hi = p.offsets[e + 1];
    if (row_lo >= row_hi) return;                        // (uniform)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kg = lane >> 4;
    const long n0 = static_cast<long>(blockIdx.x) * 16;
    long wrow = n0 + r16;
    if (wrow >= p.Nw) wrow = p.Nw - 1;                   // clamped rows are computed but never stored
    const std::uint16_t* wp[NB];
    wp[0] = p.b + (static_cast<long>(e) * p.Nw + wrow) * p.K + kg * 16;
    if constexpr (kSwiglu) wp[1] = p.b2 + (static_cast<long>(e) * p.Nw + wrow) * p.K + kg * 16;
    const long pieces = p.K / 64;
    // this wave's pieces of the contraction: wave, wave + 8, ...
    const long mine = pieces > wave ? (pieces - wave + kFewWaves - 1) / kFewWaves : 0;

    for (long chunk = row_lo; chunk < row_hi; chunk += MB * 16) {
        const std::uint16_t* xp[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            long prow = chunk + mb * 16 + r16;
            if (prow >= row_hi) prow = row_hi - 1;
            const long src = p.order ? static_cast<long>((static_cast<unsigned long long>(static_cast<unsigned>(p.order[prow])) * p.div_m) >> p.div_s) : prow;
            xp[mb] = p.a + src * p.K + kg * 16;
        }
        float4_t acc[NB][MB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};
        // two pieces per trip, every load of the trip requested before its first MFMA; lane group kg
        // supplies elements 16 kg .. + 7 of a piece to the first MFMA and the next eight to the
        // second (any assignment works as long as both operands use the same one)
        long t = 0;
        for (; t + 2 <= mine; t += 2) {
            u32x4 wv[2][2][NB], xv[2][2][MB];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const long kk = (wave + (t + u) * kFewWaves) * 64 + h * 8;
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) wv[u][h][nb] = load16(wp[nb] + kk);
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) xv[u][h][mb] = load16(xp[mb] + kk);
                }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = Mma16x16<T>::run(wv[u][h][nb], xv[u][h][mb], acc[nb][mb]);
        }
        for (; t < mine; ++t) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const long kk = (wave + t * kFewWaves) * 64 + h * 8;
                u32x4 wv[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) wv[nb] = load16(wp[nb] + kk);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 xv = load16(xp[mb] + kk);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = Mma16x16<T>::run(wv[nb], xv, acc[nb][mb]);
                }
            }
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) part[wave][nb * MB + mb][lane] = acc[nb][mb];
        __syncthreads();
        // wave w finishes row block w, w + 8, ...: lane l holds routed row l % 16 of the block and the
        // four weight rows (output columns) 4 (l / 16) .. + 3
        for (int mb = wave; mb < MB; mb += kFewWaves) {
            float4_t g = part[0][mb][lane], u = float4_t{0.f, 0.f, 0.f, 0.f};
            if constexpr (kSwiglu) u = part[0][MB + mb][lane];
#pragma unroll
            for (int w = 1; w < kFewWaves; ++w) {
                const float4_t o = part[w][mb][lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) g[r] += o[r];
                if constexpr (kSwiglu) {
                    const float4_t o2 = part[w][MB + mb][lane];
#pragma unroll
                    for (int r = 0; r < 4; ++r) u[r] += o2[r];
                }
            }
            const long prow = chunk + mb * 16 + r16;
            const long col = n0 + 4 * kg;
            if (prow < row_hi) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (col + r >= p.N) continue;
                    if constexpr (kSwiglu) p.c[prow * p.N + col + r] = swiglu_from_acc<T>(g[r], u[r]);
                    else                   p.c[prow * p.N + col + r] = El::from_f32(g[r]);
                }
            }
        }
        __syncthreads();                                 // `part` is free for the next rows
    }
}

// out[t, :] = T( sum_slot T( y[inv[t*k+slot], :] * T(w[t, slot]) ) ), 8 columns per lane.
template <typename T>
__global__ __launch_bounds__(kThreads) void moe_combine_kernel(const std::uint16_t* __restrict__ y,
                                                              const float* __restrict__ topw,
                                                              const long* __restrict__ inv_order,
                                                              std::uint16_t* __restrict__ out, long T_, int k, long H) {
    using El = Elem<T>;
    const long hv = H / 8;
    const long total = T_ * hv;
    for (long i = static_cast<long>(blockIdx.x) * kThreads + threadIdx.x; i < total;
         i += static_cast<long>(gridDim.x) * kThreads) {
        const long t = i / hv, c = (i % hv) * 8;
        double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int s = 0; s < k; ++s) {
            const long prow = inv_order[t * k + s];
            const double w = El::to_f64(El::from_f32(topw[t * k + s]));  // w.to(T)
            const u32x4 v = load16(y + prow * H + c);
            const std::uint16_t* ve = reinterpret_cast<const std::uint16_t*>(&v);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += El::to_f64(El::from_f64(El::to_f64(ve[j]) * w));
        }
        u32x4 o;
        std::uint16_t* oe = reinterpret_cast<std::uint16_t*>(&o);
#pragma unroll
        for (int j = 0; j < 8; ++j) oe[j] = El::from_f64(acc[j]);
        store16(out + t * H + c, o);
    }
}

// ---- sizes the MFMA tiles do not take (hidden or intermediate size not a multiple of 64) -------
// One thread per output element: the routed row's expert is looked up in `offsets`, the dot
// products over the contraction dim accumulate in fp32 (one rounding to T, like the tile kernels),
// the SwiGLU of GEMM 1 is applied to the narrowed gate and up values.  No alignment or size
// requirement; two orders of magnitude slower than the tiles, so it only serves odd shapes.
template <typename T, bool kSwiglu>
__global__ __launch_bounds__(kThreads) void grouped_any_kernel(const FfnGemmParams p) {
    using El = Elem<T>;
    const long prow = blockIdx.y;
    const long col = static_cast<long>(blockIdx.x) * kThreads + threadIdx.x;
    if (col >= p.N) return;
    int e = 0;
    while (e + 1 < p.E && prow >= p.offsets[e + 1]) ++e;
    const long src = p.order ? p.order[prow] / p.k : prow;
    const std::uint16_t* a = p.a + src * p.K;
    const std::uint16_t* w0 = p.b + (static_cast<long>(e) * p.Nw + col) * p.K;
    float acc0 = 0.f, acc1 = 0.f;
    if (kSwiglu) {
        const std::uint16_t* w1 = p.b2 + (static_cast<long>(e) * p.Nw + col) * p.K;
        for (long kk = 0; kk < p.K; ++kk) {
            const float av = El::to_f32(a[kk]);
            acc0 = fmaf(av, El::to_f32(w0[kk]), acc0);
            acc1 = fmaf(av, El::to_f32(w1[kk]), acc1);
        }
        p.c[prow * p.N + col] = swiglu_one<T>(El::from_f32(acc0), El::from_f32(acc1));
    } else {
        for (long kk = 0; kk < p.K; ++kk) acc0 = fmaf(El::to_f32(a[kk]), El::to_f32(w0[kk]), acc0);
        p.c[prow * p.N + col] = El::from_f32(acc0);
    }
}

// The combine for any H: one element per thread.
template <typename T>
__global__ __launch_bounds__(kThreads) void moe_combine_any_kernel(const std::uint16_t* __restrict__ y, const float* __restrict__ topw,
                                                                  const long* __restrict__ inv_order, std::uint16_t* __restrict__ out,
                                                                  long T_, int k, long H) {
    using El = Elem<T>;
    const long total = T_ * H;
    for (long i = static_cast<long>(blockIdx.x) * kThreads + threadIdx.x; i < total; i += static_cast<long>(gridDim.x) * kThreads) {
        const long t = i / H, c = i % H;
        double acc = 0.0;
        for (int s = 0; s < k; ++s) {
            const double w = El::to_f64(El::from_f32(topw[t * k + s]));
            acc += El::to_f64(El::from_f64(El::to_f64(y[inv_order[t * k + s] * H + c]) * w));
        }
        out[t * H + c] = El::from_f64(acc);
    }
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

template <typename T>
int run_ffn_any(const void* x, const void* w_gate, const void* w_up, const void* w_down, const float* topw, const long* order,
                const long* inv_order, const long* offsets, void* out, void* workspace, long T_, int E, int k, long H, long I,
                hipStream_t s) {
    const long R = T_ * k;
    auto* h = static_cast<std::uint16_t*>(workspace);
    auto* y = reinterpret_cast<std::uint16_t*>(static_cast<char*>(workspace) + align_up(static_cast<size_t>(R) * I * 2, 256));
    PARAS_REQUIRE(R <= 65535, "paras_moe_ffn: at most 65535 routed rows when the hidden or intermediate size is not a multiple of %d", kBK);
    FfnGemmParams g1{};
    g1.a = static_cast<const std::uint16_t*>(x);
    g1.b = static_cast<const std::uint16_t*>(w_gate);
    g1.b2 = static_cast<const std::uint16_t*>(w_up);
    g1.c = h;
    g1.order = order;
    g1.offsets = offsets;
    g1.K = H; g1.N = I; g1.Nw = I; g1.R = R; g1.E = E; g1.k = k;
    hipLaunchKernelGGL((grouped_any_kernel<T, true>), dim3(static_cast<unsigned>((I + kThreads - 1) / kThreads), static_cast<unsigned>(R)),
                       dim3(kThreads), 0, s, g1);
    PARAS_HIP_TRY(hipGetLastError());
    FfnGemmParams g2{};
    g2.a = h;
    g2.b = static_cast<const std::uint16_t*>(w_down);
    g2.b2 = g2.b;
    g2.c = y;
    g2.order = nullptr;
    g2.offsets = offsets;
    g2.K = I; g2.N = H; g2.Nw = H; g2.R = R; g2.E = E; g2.k = k;
    hipLaunchKernelGGL((grouped_any_kernel<T, false>), dim3(static_cast<unsigned>((H + kThreads - 1) / kThreads), static_cast<unsigned>(R)),
                       dim3(kThreads), 0, s, g2);
    PARAS_HIP_TRY(hipGetLastError());
    long blocks = (T_ * H + kThreads - 1) / kThreads;
    if (blocks > 256L * 16) blocks = 256L * 16;
    hipLaunchKernelGGL((moe_combine_any_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, y, topw, inv_order,
                       static_cast<std::uint16_t*>(out), T_, k, H);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

template <typename T, typename S>
int run_ffn_shape(const void* x, const void* w_gate, const void* w_up, const void* w_down, const float* topw,
            const long* order, const long* inv_order, const long* offsets, void* out, void* workspace, long T_,
            int E, int k, long H, long I, hipStream_t s) {
    const long R = T_ * k;
    auto* h = static_cast<std::uint16_t*>(workspace);
    auto* y = reinterpret_cast<std::uint16_t*>(static_cast<char*>(workspace) + align_up(static_cast<size_t>(R) * I * 2, 256));
    const int mt_total = static_cast<int>((R + S::kBM - 1) / S::kBM) + E;

    FfnGemmParams g1{};
    g1.a = static_cast<const std::uint16_t*>(x);
    g1.b = static_cast<const std::uint16_t*>(w_gate);
    g1.b2 = static_cast<const std::uint16_t*>(w_up);
    g1.c = h;
    g1.order = order;
    g1.offsets = offsets;
    g1.K = H; g1.N = I; g1.Nw = I; g1.R = R; g1.E = E; g1.k = k;
    g1.mt_total = mt_total;
    division_by(static_cast<unsigned>(k), &g1.div_m, &g1.div_s);
    g1.n_units = static_cast<int>((I + kBN - 1) / kBN);
    // Column units an XCD sweeps together: up to 2 (one expert's weight panel for them is
    // 4 MB at K = 4096, the size of an XCD's L2; 4 units measured 8 % slower), fewer when
    // there are not enough units to keep all 8 XCDs busy.
    auto plan = [](FfnGemmParams& g) {
        int ngt = g.n_units / 8;
        g.ngt = ngt < 1 ? 1 : (ngt > 2 ? 2 : ngt);
    };
    auto grid_of = [&](const FfnGemmParams& g) {
        const long groups = (g.n_units + 8 * g.ngt - 1) / (8 * g.ngt);
        return static_cast<unsigned>(groups * 8 * g.ngt * g.mt_total);
    };
    plan(g1);
    // 256-row tiles: the four-wave tile of 16 x 16 x 32 MFMAs (PARAS_GEMM_EIGHT_WAVES: the eight-wave tile of
    // 32 x 32 x 16 ones, for measurements)
    static const bool eight_waves = std::getenv("PARAS_GEMM_EIGHT_WAVES") != nullptr;
    constexpr bool kBig = S::kBM == 256;
    if (kBig && !eight_waves)
        hipLaunchKernelGGL((grouped_gemm_quad16_kernel<T, true>), dim3(grid_of(g1)), dim3(quad16::kThreads), 0, s, g1);
    else
        hipLaunchKernelGGL((grouped_gemm_kernel<T, true, S>), dim3(grid_of(g1)), dim3(S::kThreads), 0, s, g1);
    PARAS_HIP_TRY(hipGetLastError());

    FfnGemmParams g2{};
    g2.a = h;
    g2.b = static_cast<const std::uint16_t*>(w_down);
    g2.b2 = g2.b;  // column group 1 = the next 128 weight rows, selected through the row index
    g2.c = y;
    g2.order = nullptr;
    g2.offsets = offsets;
    g2.K = I; g2.N = H; g2.Nw = H; g2.R = R; g2.E = E; g2.k = k;
    g2.mt_total = mt_total;
    g2.n_units = static_cast<int>((H + 2 * kBN - 1) / (2 * kBN));
    plan(g2);
    if (kBig && !eight_waves)
        hipLaunchKernelGGL((grouped_gemm_quad16_kernel<T, false>), dim3(grid_of(g2)), dim3(quad16::kThreads), 0, s, g2);
    else
        hipLaunchKernelGGL((grouped_gemm_kernel<T, false, S>), dim3(grid_of(g2)), dim3(S::kThreads), 0, s, g2);
    PARAS_HIP_TRY(hipGetLastError());

    const long total = T_ * (H / 8);
    long blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 256L * 16) blocks = 256L * 16;
    hipLaunchKernelGGL((moe_combine_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, y, topw,
                       inv_order, static_cast<std::uint16_t*>(out), T_, k, H);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

template <typename T>
int run_ffn_few_rows(const void* x, const void* w_gate, const void* w_up, const void* w_down, const float* topw,
                     const long* order, const long* inv_order, const long* offsets, void* out, void* workspace, long T_,
                     int E, int k, long H, long I, hipStream_t s) {
    const long R = T_ * k;
    auto* h = static_cast<std::uint16_t*>(workspace);
    auto* y = reinterpret_cast<std::uint16_t*>(static_cast<char*>(workspace) + align_up(static_cast<size_t>(R) * I * 2, 256));
    FfnGemmParams g1{};
    g1.a = static_cast<const std::uint16_t*>(x);
    g1.b = static_cast<const std::uint16_t*>(w_gate);
    g1.b2 = static_cast<const std::uint16_t*>(w_up);
    g1.c = h;
    g1.order = order;
    g1.offsets = offsets;
    g1.K = H; g1.N = I; g1.Nw = I; g1.R = R; g1.E = E; g1.k = k;
    division_by(static_cast<unsigned>(k), &g1.div_m, &g1.div_s);
    hipLaunchKernelGGL((grouped_few_rows_kernel<T, true, 2>), dim3(static_cast<unsigned>((I + 15) / 16), static_cast<unsigned>(E)),
                       dim3(kFewWaves * 64), 0, s, g1);
    PARAS_HIP_TRY(hipGetLastError());
    FfnGemmParams g2{};
    g2.a = h;
    g2.b = static_cast<const std::uint16_t*>(w_down);
    g2.b2 = g2.b;
    g2.c = y;
    g2.order = nullptr;
    g2.offsets = offsets;
    g2.K = I; g2.N = H; g2.Nw = H; g2.R = R; g2.E = E; g2.k = k;
    hipLaunchKernelGGL((grouped_few_rows_kernel<T, false, 2>), dim3(static_cast<unsigned>((H + 15) / 16), static_cast<unsigned>(E)),
                       dim3(kFewWaves * 64), 0, s, g2);
    PARAS_HIP_TRY(hipGetLastError());
    const long total = T_ * (H / 8);
    long blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 256L * 16) blocks = 256L * 16;
    hipLaunchKernelGGL((moe_combine_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, y, topw,
                       inv_order, static_cast<std::uint16_t*>(out), T_, k, H);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

// 256-row tiles when the experts are big enough for them: an expert's last tile is half empty on
// average, so the rows per expert should be many times the tile, and there must be tiles for at
// least half the CUs.
template <typename T>
int run_ffn(const void* x, const void* w_gate, const void* w_up, const void* w_down, const float* topw,
            const long* order, const long* inv_order, const long* offsets, void* out, void* workspace, long T_,
            int E, int k, long H, long I, hipStream_t s) {
    const long R = T_ * k;
    // Up to 16 routed rows per expert on average the few-row kernels (an expert with more than 32 rows
    // takes them 32 at a time).  8 experts, top-2, H = 4096, I = 14336, tiles against few-row kernels:
    // 1 token 421 / 168 us, 8 tokens 615 / 397, 32 tokens 659 / 574, 64 tokens 663 / 667, 128 tokens
    // 672 / 1124.  PARAS_MOE_FEW_ROWS = n moves the limit (0: never).
    static const char* few_env = std::getenv("PARAS_MOE_FEW_ROWS");
    const long few_limit = few_env != nullptr ? std::atol(few_env) : 16;
    if (R <= few_limit * E && E <= 65535 && (I + 15) / 16 <= 0x7fffffffL)
        return run_ffn_few_rows<T>(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, out, workspace, T_, E, k, H, I, s);
    const long wide_tiles = (R / Tile256::kBM) * ((H + 2 * kBN - 1) / (2 * kBN));
    if (R / E >= 4 * Tile256::kBM && wide_tiles >= 128)
        return run_ffn_shape<T, Tile256>(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, out, workspace, T_, E, k, H, I, s);
    return run_ffn_shape<T, Tile128>(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, out, workspace, T_, E, k, H, I, s);
}

}  // namespace
}  // namespace paras

extern "C" {

size_t paras_moe_ffn_workspace(int64_t T, int64_t k, int64_t H, int64_t I, int dtype) {
    (void)dtype;
    if (T <= 0 || k <= 0 || H <= 0 || I <= 0) return 0;
    const size_t R = static_cast<size_t>(T) * k;
    return paras::align_up(R * I * 2, 256) + paras::align_up(R * H * 2, 256);
}

int paras_moe_ffn(const void* x, const void* w_gate, const void* w_up, const void* w_down, const float* topw,
                  const int64_t* order, const int64_t* inv_order, const int64_t* offsets, void* out,
                  void* workspace, int64_t T, int64_t E, int64_t k, int64_t H, int64_t I, int dtype, void* stream) {
    using namespace paras;
    PARAS_REQUIRE(T >= 0 && E >= 1 && k >= 1 && H >= 1 && I >= 1, "paras_moe_ffn: bad shape");
    if (T == 0) return PARAS_OK;
    PARAS_REQUIRE(dtype == PARAS_BF16 || dtype == PARAS_F16, "paras_moe_ffn: dtype must be bf16 or f16");
    PARAS_REQUIRE(x && w_gate && w_up && w_down && topw && order && inv_order && offsets && out && workspace,
                  "paras_moe_ffn: null pointer");
    // The MFMA tiles take hidden and intermediate sizes that are multiples of 64 and 16-byte aligned
    // tensors; anything else goes to the general kernels (any size, any alignment).
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w_gate) | reinterpret_cast<uintptr_t>(w_up) |
                           reinterpret_cast<uintptr_t>(w_down) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(workspace)) & 15) == 0;
    const bool tiles = H % kBK == 0 && I % kBK == 0 && aligned && H < (1LL << 22) && I < (1LL << 22);   // (the tiles' stores use 32-bit byte offsets within a tile)
    PARAS_REQUIRE(T * k <= 0x3fffffffLL, "paras_moe_ffn: too many routed rows");
    if (T * H >= (1LL << 32) || T * k * I >= (1LL << 32) || I * H >= (1LL << 32))
        return fail(PARAS_ERR_UNSUPPORTED, "paras_moe_ffn: an operand (x, the routed intermediate, or one expert's weight matrix) spans 2^32 elements or more");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    const long* ord = reinterpret_cast<const long*>(order);
    const long* inv = reinterpret_cast<const long*>(inv_order);
    const long* off = reinterpret_cast<const long*>(offsets);
    if (!tiles) {
        if (dtype == PARAS_BF16)
            return run_ffn_any<bf16_t>(x, w_gate, w_up, w_down, topw, ord, inv, off, out, workspace, T, (int)E, (int)k, H, I, s);
        return run_ffn_any<f16_t>(x, w_gate, w_up, w_down, topw, ord, inv, off, out, workspace, T, (int)E, (int)k, H, I, s);
    }
    if (dtype == PARAS_BF16)
        return run_ffn<bf16_t>(x, w_gate, w_up, w_down, topw, ord, inv, off, out, workspace, T, (int)E, (int)k, H, I, s);
    return run_ffn<f16_t>(x, w_gate, w_up, w_down, topw, ord, inv, off, out, workspace, T, (int)E, (int)k, H, I, s);
}

}  // extern "C"
