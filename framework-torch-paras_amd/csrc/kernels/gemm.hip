// Dense (optionally batched) NT GEMM for gfx950 on bf16/fp16 MFMA, fp32 accumulate:
//
//   C[b] = T( alpha * A[b] B[b]^T + beta * addend[b] )      A [M, K], B [N, K], C [M, N]
//
// The reference bounces mm / bmm / addmm / linear to ATen on the host
// (csrc/ops/vision_ops.cpp:248-309,388-423: copy to CPU, at::mm / at::bmm /
// at::addmm / at::linear with fp32 accumulation and one rounding, copy back).
// "NT" is the layout of every nn.Linear (x W^T) and of q k^T: both operands are
// contiguous along the contraction dim, which is what the MFMA operand layout
// wants; the tile mainloop is the one the expert GEMMs use (gemm_tile.h).
// `addend` is a matrix with row stride ld_add; ld_add = 0 broadcasts one row
// (a bias) over all rows.
#include <hip/hip_runtime.h>
#include <cstdlib>

#include <type_traits>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/gemm_tile.h"
#include "paras_hip.h"

namespace paras {
namespace {

using namespace gemm;

struct DenseParams {
    const std::uint16_t* a;
    const std::uint16_t* b;
    const std::uint16_t* add;   // may be null
    std::uint16_t* c;
    long M, N, K;
    long lda, ldb, ldc, ld_add;
    long sa, sb, sc, sadd;      // batch strides (elements)
    int  m_tiles, n_units;      // row tiles (128 or 256 rows), column units (128 or 256 columns)
    float alpha, beta;
    double alpha64, beta64;     // the same, for fp64 tensors
    int  splits;                // kPartial kernels: parts of the contraction, one workgroup each per tile
    long k_per_split;           // contraction elements per part (a multiple of 64)
    float* partial;             // [batch][split][M][N] fp32
    int  swapped;               // few-row kernels only: a and b have changed places (few output COLUMNS, many rows), so a
                                // result (row of a, row of b) belongs at c[row of b][row of a], and the addend likewise
    int  xcd_blocks, xcd_blocks_n;   // XCD-blocked tile order: blocks of kXcdBlockM x kXcdBlockN tiles per batch (0: plain order), blocks along n
    int  causal_kind;           // fp32 MFMA kernel, for causal attention: 1 = the product is a score matrix of which row r only needs
                                // columns <= r + causal_first (tiles wholly beyond are left unwritten); 2 = a is such a matrix after
                                // its softmax (zeros beyond), so row tile r0 contracts over k < r0 + 128 + causal_first only; 0 = neither
    long causal_first;          // index of row 0 among the queries
};

// Workgroup w runs on XCD w % 8, each with an L2 of its own.  In the plain order (column units
// innermost) the 32 workgroups an XCD runs at a time are 16 row tiles x 2 column units: 18 operand
// panels pass through its L2.  Dealing the tiles in blocks of 4 x 8, one block per XCD at a time,
// makes that 12 panels: a third fewer L2 misses.  The grid is padded to whole blocks and to a
// multiple of 8 blocks; a workgroup whose tile does not exist returns at once.
constexpr int kXcdBlockM = 4, kXcdBlockN = 8, kXcdBlockTiles = kXcdBlockM * kXcdBlockN, kXcds = 8;
__host__ __device__ inline long xcd_order_workgroups(int blocks) { return static_cast<long>((blocks + kXcds - 1) / kXcds) * kXcds * kXcdBlockTiles; }
// false: no tile for this workgroup
__device__ __forceinline__ bool tile_of_workgroup(const DenseParams& p, long wg, long& bidx, int& mt, int& nu) {
    if (p.xcd_blocks == 0) {
        const long per_batch = static_cast<long>(p.m_tiles) * p.n_units;
        bidx = wg / per_batch;
        const long rem = wg % per_batch;
        mt = static_cast<int>(rem / p.n_units);
        nu = static_cast<int>(rem % p.n_units);
        return true;
    }
    const long per_batch = xcd_order_workgroups(p.xcd_blocks);
    bidx = wg / per_batch;
    const int w = static_cast<int>(wg % per_batch);
    const int xcd = w % kXcds, j = w / kXcds;
    const int block = (j / kXcdBlockTiles) * kXcds + xcd, t = j % kXcdBlockTiles;
    mt = (block / p.xcd_blocks_n) * kXcdBlockM + t / kXcdBlockN;
    nu = (block % p.xcd_blocks_n) * kXcdBlockN + t % kXcdBlockN;
    return block < p.xcd_blocks && mt < p.m_tiles && nu < p.n_units;
}

// S = Tile256 (8 waves, 256 x 256 on 32 x 32 x 16 MFMAs: launched only when PARAS_GEMM_EIGHT_WAVES is set,
// the problems of at least 144 such tiles run on dense_gemm_nt_quad16_kernel below), Tile128 (4 waves,
// 128 x 256) or Tile128x128 (4 waves, one column group; when there would be fewer than 512 tiles of 128 x 256).
// kPartial: the contraction is split over p.splits workgroups per tile (the few-tile problems of 33 to
// 128 rows: a projection at decode batch sizes has 32 to 112 tiles for 256 CUs); each writes its
// fp32 partial tile, and skinny_splitk_finish_kernel adds them in split order and applies the epilogue.
template <typename T, typename S, bool kPartial = false>
__global__ __launch_bounds__(S::kThreads, (S::kGroups == 1 ? 3 : 2)) void dense_gemm_nt_kernel(const DenseParams p) {
    using El = Elem<T>;
    __shared__ __attribute__((aligned(16))) typename S::Lds lds;

    // Column units innermost: the workgroups running together share the A row panel
    // (and, across m-tiles, stream the same B panels through L2).
    const long tile_id = kPartial ? blockIdx.x / p.splits : blockIdx.x;
    const long split = kPartial ? blockIdx.x % p.splits : 0;
    const long k_first = kPartial ? split * p.k_per_split : 0;
    const long k_count = kPartial ? (k_first + p.k_per_split < p.K ? p.k_per_split : p.K - k_first) : p.K;
    long bidx;
    int mt, nu;
    if (!tile_of_workgroup(p, tile_id, bidx, mt, nu)) return;      // (the whole workgroup: nobody is left at a barrier)
    const long row0 = static_cast<long>(mt) * S::kBM, n0 = static_cast<long>(nu) * S::kGroups * kBN;
    const std::uint16_t* A = p.a + bidx * p.sa + k_first;
    const std::uint16_t* B = p.b + bidx * p.sb + k_first;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    constexpr int G = S::kGroups;
    unsigned a_off[4], b_off[G][S::kBChunks];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * S::kThreads;
        long arow = row0 + (c >> 3);
        if (arow >= p.M) arow = p.M - 1;     // clamped rows are computed but never stored
        a_off[i] = static_cast<unsigned>(arow * p.lda + (c & 7) * 8);
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < S::kBChunks; ++i) {
            const int c = tid + i * S::kThreads;
            long brow = n0 + g * kBN + (c >> 3);
            if (brow >= p.N) brow = p.N - 1;
            b_off[g][i] = static_cast<unsigned>(brow * p.ldb + (c & 7) * 8);
        }
    const std::uint16_t* b_base[G];
#pragma unroll
    for (int g = 0; g < G; ++g) b_base[g] = B;
    float16_t acc[G][2][2];
    S::template mainloop<T>(A, a_off, b_base, b_off, k_count, lds, acc);

    if constexpr (kPartial) {
        float* dst = p.partial + (bidx * p.splits + split) * (p.M * p.N);
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    const long col = n0 + g * kBN + wn * 64 + ni * 32 + lr;
                    if (col >= p.N) continue;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const long row = row0 + wm * 64 + mi * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
                        if (row < p.M) dst[row * p.N + col] = acc[g][mi][ni][r];
                    }
                }
        return;
    }
    std::uint16_t* C = p.c + bidx * p.sc;
    const std::uint16_t* ADD = p.add ? p.add + bidx * p.sadd : nullptr;
    // The plain product (alpha = 1, nothing added) of a tile whose byte offsets fit 32 bits: one
    // uniform base, a 32-bit offset per lane, rows and columns checked against counts in 32-bit
    // registers, and the conversion instruction for the narrowing; a 32 x 32 block in which a NaN
    // turns up is narrowed again in software, which writes NaNs as the host's types do.
    if (p.alpha == 1.0f && ADD == nullptr && p.ldc < (1L << 22)) {
        std::uint16_t* cb = C + row0 * p.ldc + n0;                       // uniform
        const long rows_left = p.M - row0, cols_left = p.N - n0;
        const int nrows = static_cast<int>(rows_left < S::kBM ? rows_left : S::kBM) - (wm * 64 + 4 * lh);
        const int ncols = static_cast<int>(cols_left < G * kBN ? cols_left : G * kBN) - (wn * 64 + lr);
        const unsigned ldc2 = static_cast<unsigned>(p.ldc) * 2u;
        unsigned lane_b = static_cast<unsigned>(wm * 64 + 4 * lh) * ldc2 + static_cast<unsigned>(wn * 64 + lr) * 2u;
        asm volatile("" : "+v"(lane_b));       // one add per store from here on (not a 64-bit multiply-add per element)
        const bool full = rows_left >= S::kBM && cols_left >= G * kBN;    // uniform
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    if (g * kBN + ni * 32 >= ncols) continue;
                    std::uint16_t o[16];
                    narrow_block<T>(acc[g][mi][ni], o);
                    char* blk = reinterpret_cast<char*>(cb) + (g * kBN + ni * 32) * 2;
                    if (full) store_block<true>(blk, lane_b, ldc2, mi, nrows, o);
                    else      store_block<false>(blk, lane_b, ldc2, mi, nrows, o);
                }
        return;
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const long col = n0 + g * kBN + wn * 64 + ni * 32 + lr;
                if (col >= p.N) continue;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const long row = row0 + wm * 64 + mi * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
                    if (row >= p.M) continue;
                    float v = p.alpha * acc[g][mi][ni][r];
                    if (ADD) v = fmaf(p.beta, El::to_f32(ADD[row * p.ld_add + col]), v);
                    C[row * p.ldc + col] = El::from_f32(v);
                }
            }
}

// The 256 x 256 tile of four waves on v_mfma_f32_16x16x32 (gemm_tile.h, namespace quad16): what the
// dense product runs on from 144 tiles on.  Same-box timings against the eight-wave tile of
// 32 x 32 x 16 MFMAs, which it replaces here: 16384 x 4096 x 4096 414.6 against 424.6 us (bench.py,
// sustained: 415 against 427), 8192^3 806 against 836 us, N = 14336 1477 against 1500 us.
template <typename T>
__global__ __launch_bounds__(quad16::kThreads, 1) void dense_gemm_nt_quad16_kernel(const DenseParams p) {
    using El = Elem<T>;
    __shared__ __attribute__((aligned(16))) quad16::TileLds lds;
    long bidx;
    int mt, nu;
    if (!tile_of_workgroup(p, blockIdx.x, bidx, mt, nu)) return;      // (the whole workgroup: nobody is left at a barrier)
    const long row0 = static_cast<long>(mt) * quad16::kBM, n0 = static_cast<long>(nu) * 2 * kBN;
    const std::uint16_t* A = p.a + bidx * p.sa;
    const std::uint16_t* B = p.b + bidx * p.sb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    unsigned a_off[8], b_off[2][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = tid + i * quad16::kThreads;
        long arow = row0 + (c >> 3);
        if (arow >= p.M) arow = p.M - 1;     // clamped rows are computed but never stored
        a_off[i] = static_cast<unsigned>(arow * p.lda + (c & 7) * 8);
    }
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * quad16::kThreads;
            long brow = n0 + g * kBN + (c >> 3);
            if (brow >= p.N) brow = p.N - 1;
            b_off[g][i] = static_cast<unsigned>(brow * p.ldb + (c & 7) * 8);
        }
    const std::uint16_t* b_base[2] = {B, B};
    quad16::float4v acc[8][8];
    quad16::tile_mainloop<T>(A, a_off, b_base, b_off, p.K, lds, acc);

    // epilogue: lane (l16 = lane % 16, kq = lane / 16) of block (i, j) holds row i*16 + l16 and columns
    // 4 kq .. + 3 of column block j (group j / 4, columns wn*64 + (j % 4)*16 of it)
    const int l16 = lane & 15, kq = lane >> 4;
    std::uint16_t* C = p.c + bidx * p.sc;
    const std::uint16_t* ADD = p.add ? p.add + bidx * p.sadd : nullptr;
    // the plain product into rows of 8-byte aligned pieces: the conversion instruction, four columns per store;
    // a row block in which a NaN turns up takes the software narrowing (which writes NaNs as the host's types do)
    const bool plain = p.alpha == 1.0f && ADD == nullptr && p.ldc % 4 == 0 && p.sc % 4 == 0 && (reinterpret_cast<uintptr_t>(p.c) & 7) == 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const long row = row0 + wm * 128 + i * 16 + l16;
        bool nan_here = false;
        if (plain) {
            float probe = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) probe += acc[i][j][r];
            nan_here = __builtin_amdgcn_ballot_w64(probe != probe) != 0;      // (an infinity minus an infinity counts as well)
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const long col = n0 + (j >> 2) * kBN + wn * 64 + (j & 3) * 16 + 4 * kq;
            if (row >= p.M || col >= p.N) continue;
            if (plain && col + 3 < p.N) {
                std::uint16_t o[4];
                if (__builtin_expect(nan_here, 0)) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] = El::from_f32(acc[i][j][r]);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] = El::from_f32_finite(acc[i][j][r]);
                }
                u32x2 w2;
                w2[0] = o[0] | (static_cast<std::uint32_t>(o[1]) << 16);
                w2[1] = o[2] | (static_cast<std::uint32_t>(o[3]) << 16);
                *reinterpret_cast<u32x2*>(C + row * p.ldc + col) = w2;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (col + r >= p.N) continue;
                    float v = p.alpha * acc[i][j][r];
                    if (ADD) v = fmaf(p.beta, El::to_f32(ADD[row * p.ld_add + col + r]), v);
                    C[row * p.ldc + col + r] = El::from_f32(v);
                }
            }
        }
    }
}

// ---- few rows (M <= 128): the decode-time projections.  The product is bound by streaming the
// weights once, so there is no tile and no LDS staging: a workgroup owns 16 weight rows, its eight
// waves split the contraction (pieces of 64 dealt round-robin, so the eight read adjacent 128-byte
// lines of each row), every wave feeds v_mfma_f32_16x16x32 straight from global memory (weights
// as the row operand, with plain loads: non-temporal ones measured 5-18 % slower here, each
// 128-byte line being touched by two instructions; the few activation rows from L2), and the eight partial
// results meet in LDS in wave order.  Lane l of a 16x16 result holds activation row l%16 and
// weight rows 4*(l/16) .. +3: four adjacent outputs, stored as one 8-byte piece when aligned.
template <typename T> struct Mma16;
template <> struct Mma16<bf16_t> {
    __device__ static __forceinline__ float4_t run(u32x4 a, u32x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma16<f16_t> {
    __device__ static __forceinline__ float4_t run(u32x4 a, u32x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

constexpr int kSkinnyWaves = 8;
constexpr int kSkinnyMaxM = 128;

template <typename T, int MB, int NB>   // MB = 16-row blocks of activations, NB = 16-row blocks of weights per workgroup
__global__ __launch_bounds__(kSkinnyWaves * 64) void skinny_gemm_nt_kernel(const DenseParams p) {
    using El = Elem<T>;
    __shared__ float4_t part[kSkinnyWaves][NB * MB][64];
    const long bidx = blockIdx.y;
    const std::uint16_t* A = p.a + bidx * p.sa;
    const std::uint16_t* B = p.b + bidx * p.sb;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kg = lane >> 4;
    const long n0 = static_cast<long>(blockIdx.x) * (16 * NB);
    const std::uint16_t* wp[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        long wrow = n0 + nb * 16 + r16;
        if (wrow >= p.N) wrow = p.N - 1;                    // clamped rows are computed but never stored
        wp[nb] = B + wrow * p.ldb + kg * 16;
    }
    const std::uint16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        long xrow = mb * 16 + r16;
        if (xrow >= p.M) xrow = p.M - 1;
        xp[mb] = A + xrow * p.lda + kg * 16;
    }
    float4_t acc[NB][MB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};
    // The contraction is walked in pieces of 64 (two MFMAs): lane group kg supplies elements
    // 16 kg .. 16 kg + 7 of a piece to the first MFMA and the next eight to the second -- any
    // assignment works as long as both operands use the same one -- so that the four groups
    // together read whole 128-byte lines of a row.  A batch is kPieces pieces: every load of the
    // batch is requested before its first MFMA, so a wave pays the memory latency once per batch.
    const long pieces = p.K / 64;
    constexpr int kPieces = MB <= 4 ? 2 : 1;
    // this wave's pieces are wave, wave + W, ...; each workgroup starts at a different one of them and
    // wraps around, so that the workgroups do not all read the same part of every weight row at once
    const long mine = pieces > wave ? (pieces - wave + kSkinnyWaves - 1) / kSkinnyWaves : 0;
    const long first = mine > 0 ? (static_cast<long>(blockIdx.x) * 3) % mine : 0;
    auto piece_at = [&](long t) {
        long r = t + first;
        if (r >= mine) r -= mine;
        return (wave + r * kSkinnyWaves) * 64;
    };
    long t = 0;
    for (; t + kPieces <= mine; t += kPieces) {
        u32x4 wv[kPieces][2][NB], xv[kPieces][2][MB];
#pragma unroll
        for (int u = 0; u < kPieces; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const long k = piece_at(t + u) + h * 8;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) wv[u][h][nb] = load16(wp[nb] + k);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) xv[u][h][mb] = load16(xp[mb] + k);
            }
#pragma unroll
        for (int u = 0; u < kPieces; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = Mma16<T>::run(wv[u][h][nb], xv[u][h][mb], acc[nb][mb]);
    }
    for (; t < mine; ++t) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const long k = piece_at(t) + h * 8;
            u32x4 wv[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) wv[nb] = load16(wp[nb] + k);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const u32x4 xv = load16(xp[mb] + k);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = Mma16<T>::run(wv[nb], xv, acc[nb][mb]);
            }
        }
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) part[wave][nb * MB + mb][lane] = acc[nb][mb];
    __syncthreads();
    // wave w finishes result blocks w, w + 8, ...
    std::uint16_t* C = p.c + bidx * p.sc;
    const std::uint16_t* ADD = p.add ? p.add + bidx * p.sadd : nullptr;
    const bool vec_ok = (p.ldc % 4 == 0) && (p.sc % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0);
    for (int blk = wave; blk < NB * MB; blk += kSkinnyWaves) {
        const int nb = blk / MB, mb = blk % MB;
        float4_t t = part[0][blk][lane];
#pragma unroll
        for (int w = 1; w < kSkinnyWaves; ++w) {
            const float4_t o = part[w][blk][lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) t[r] += o[r];
        }
        const long row = mb * 16 + r16;
        const long col = n0 + nb * 16 + 4 * kg;
        if (row >= p.M) continue;
        if (p.swapped) {        // `row` is a column of the caller's result and `col + r` a row of it
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (col + r >= p.N) continue;
                float v = p.alpha * t[r];
                if (ADD) v = fmaf(p.beta, El::to_f32(ADD[(col + r) * p.ld_add + row]), v);
                C[(col + r) * p.ldc + row] = El::from_f32(v);
            }
            continue;
        }
        std::uint16_t o16[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = p.alpha * t[r];
            if (ADD && col + r < p.N) v = fmaf(p.beta, El::to_f32(ADD[row * p.ld_add + col + r]), v);
            o16[r] = El::from_f32(v);
        }
        if (vec_ok && col + 3 < p.N) {
            u32x2 w2;
            w2[0] = o16[0] | (static_cast<std::uint32_t>(o16[1]) << 16);
            w2[1] = o16[2] | (static_cast<std::uint32_t>(o16[3]) << 16);
            *reinterpret_cast<u32x2*>(C + row * p.ldc + col) = w2;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (col + r < p.N) C[row * p.ldc + col + r] = o16[r];
        }
    }
}

// Two blocks of weight rows per workgroup when that still leaves a workgroup for every CU: every
// activation fragment then feeds two MFMAs, which halves the reads of the activations from L2.
template <typename T>
void launch_skinny(const DenseParams& p, long batch, hipStream_t s) {
    const dim3 block(kSkinnyWaves * 64);
    const int mb = static_cast<int>((p.M + 15) / 16);
    const dim3 g1(static_cast<unsigned>((p.N + 15) / 16), static_cast<unsigned>(batch));
    const dim3 g2(static_cast<unsigned>((p.N + 31) / 32), static_cast<unsigned>(batch));
    const bool two = mb > 1 && static_cast<long>(g2.x) * batch >= 256;
    if (mb <= 1)      hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 1, 1>), g1, block, 0, s, p);
    else if (mb <= 2) { if (two) hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 2, 2>), g2, block, 0, s, p);
                        else     hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 2, 1>), g1, block, 0, s, p); }
    else if (mb <= 4) { if (two) hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 4, 2>), g2, block, 0, s, p);
                        else     hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 4, 1>), g1, block, 0, s, p); }
    else              { if (two) hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 8, 2>), g2, block, 0, s, p);
                        else     hipLaunchKernelGGL((skinny_gemm_nt_kernel<T, 8, 1>), g1, block, 0, s, p); }
}

// ---- few rows with a workspace: the same product with the activations read once per 128 weight
// rows instead of once per 16.  In the kernel above every workgroup re-reads all M x K activations
// from L2, which -- not the weights -- bounds it from M = 32 upwards.  Here the eight waves of a
// workgroup own eight blocks of 16 weight rows and walk the SAME part of the contraction, so a slab
// of activations (M rows x 256 elements) is brought into LDS once and shared; the contraction is
// split over workgroups instead (grid.x), each writes its fp32 partial result to the workspace, and
// a second kernel adds the partials in split order and applies the epilogue: deterministic, and
// 128 / 16 = 8 times fewer activation reads for a workspace of splits x M x N floats.
constexpr int kSlab = 256;                 // contraction elements per LDS slab (4 pieces of 64)
constexpr int kSlabLd = kSlab + 8;         // LDS row stride (elements): 16 consecutive rows hit distinct banks

template <typename T, int MB>
__global__ __launch_bounds__(512) void skinny_splitk_kernel(const DenseParams p, float* __restrict__ partial, int pieces_per_split) {
    __shared__ __attribute__((aligned(16))) std::uint16_t xs[2][MB * 16 * kSlabLd];
    const long bidx = blockIdx.z;
    const std::uint16_t* A = p.a + bidx * p.sa;
    const std::uint16_t* B = p.b + bidx * p.sb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kg = lane >> 4;
    // grid.x = split, grid.y = block of 128 weight rows: workgroups that run together read adjacent
    // parts of the same weight rows
    const long n0 = static_cast<long>(blockIdx.y) * 128 + wave * 16;
    long wrow = n0 + r16;
    if (wrow >= p.N) wrow = p.N - 1;                        // clamped rows are computed but never stored
    const std::uint16_t* wp = B + wrow * p.ldb + kg * 16;
    const long pieces = p.K / 64;
    const long pc0 = static_cast<long>(blockIdx.x) * pieces_per_split;
    const long pc1 = pc0 + pieces_per_split < pieces ? pc0 + pieces_per_split : pieces;
    // staging of a slab: MB*16 rows x 32 chunks of 16 bytes, 512 threads -> MB chunks per thread
    u32x4 stage[MB];
    auto load_slab = [&](long pc) {                         // pieces pc .. pc+3 (clamped to the split's end)
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int c = tid + i * 512;
            long row = c >> 5;
            const long k = pc * 64 + (c & 31) * 8;
            if (row >= p.M) row = p.M - 1;
            stage[i] = k < pc1 * 64 ? load16(A + row * p.lda + k) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_slab = [&](int buf) {
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int c = tid + i * 512;
            *reinterpret_cast<u32x4*>(&xs[buf][(c >> 5) * kSlabLd + (c & 31) * 8]) = stage[i];
        }
    };
    float4_t acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = float4_t{0.f, 0.f, 0.f, 0.f};
    // Weights and activations of slab s+1 are requested before the MFMAs of slab s, so that two
    // slabs' worth of loads are in flight per wave and a split of two slabs pays the memory latency
    // about once.
    u32x4 wv[4][2], wn[4][2];
    auto load_w = [&](long pc, u32x4 (&dst)[4][2]) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                dst[u][h] = pc + u < pc1 ? load16(wp + (pc + u) * 64 + h * 8) : u32x4{0, 0, 0, 0};
    };
    // The slabs of the split are walked from a different starting slab in every block of weight rows
    // (and wrap around), so that the workgroups of one split do not read the same part of their rows
    // at the same time.
    const long nslabs = pc1 > pc0 ? (pc1 - pc0 + 3) / 4 : 0;
    const long rot = nslabs > 0 ? static_cast<long>(blockIdx.y) % nslabs : 0;
    auto slab_pc = [&](long i) {
        long r = i + rot;
        if (r >= nslabs) r -= nslabs;
        return pc0 + 4 * r;
    };
    if (nslabs > 0) {
        load_slab(slab_pc(0));
        load_w(slab_pc(0), wv);
        store_slab(0);
    }
    __syncthreads();
    int buf = 0;
    for (long i = 0; i < nslabs; ++i, buf ^= 1) {
        const bool more = i + 1 < nslabs;
        if (more) {
            load_slab(slab_pc(i + 1));
            load_w(slab_pc(i + 1), wn);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 xv = *reinterpret_cast<const u32x4*>(&xs[buf][(mb * 16 + r16) * kSlabLd + u * 64 + kg * 16 + h * 8]);
                    acc[mb] = Mma16<T>::run(wv[u][h], xv, acc[mb]);
                }
        if (more) {
            store_slab(buf ^ 1);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int h = 0; h < 2; ++h) wv[u][h] = wn[u][h];
        }
        __syncthreads();
    }
    // partial[(batch, split)][row][col]: lane holds row mb*16 + r16, columns n0 + 4 kg .. + 3
    float* dst = partial + (bidx * gridDim.x + blockIdx.x) * (p.M * p.N);
    const long col = n0 + 4 * kg;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const long row = mb * 16 + r16;
        if (row >= p.M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (col + r < p.N) dst[row * p.N + col + r] = acc[mb][r];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void skinny_splitk_finish_kernel(const DenseParams p, const float* __restrict__ partial, int splits) {
    using El = Elem<T>;
    const long mn = p.M * p.N;
    const long i = static_cast<long>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= mn) return;
    const long bidx = blockIdx.y;
    const float* src = partial + bidx * splits * mn + i;
    float t = 0.f;
    for (int sp = 0; sp < splits; ++sp) t += src[sp * mn];
    const long row = i / p.N, col = i % p.N;
    float v = p.alpha * t;
    if (p.add) v = fmaf(p.beta, El::to_f32((p.add + bidx * p.sadd)[row * p.ld_add + col]), v);
    (p.c + bidx * p.sc)[row * p.ldc + col] = El::from_f32(v);
}

// Splits of the contraction for the workspace kernel (0 = it does not apply): enough workgroups to
// fill the chip twice, at least two slabs each.
// Few rows but many columns (a vocabulary projection, a fused gate-up projection at M = 64 ... 128):
// from about 200 tiles of 128 x 128 the tile kernel streams the weights faster than the few-row
// kernels do (M = 128, N = 128256, K = 4096: 267 against 649 us; N = 28672: 75 against 106 us; at
// N = 6144 the few-row kernels win, 47 against 67 us).  Up to 32 rows the few-row kernels stay.
bool few_rows_by_tiles(long M, long N, long batch) {
    return M > 32 && M <= kSkinnyMaxM && (N + gemm::kBN - 1) / gemm::kBN * batch >= 192;
}

// Few output columns and many rows: the few-row kernels with the operands in each other's place.  Up to
// 32 columns (every workgroup re-reads the short operand, and from 48 rows of it on the tile kernel with
// the contraction in parts is faster: M = 16384, N = 128, K = 4096 80 us this way).
bool swapped_route(long M, long N, long batch) {
    return N <= 32 && M > kSkinnyMaxM && batch <= 65535 && (M + 15) / 16 <= 0x7fffffffL;
}

// Parts of the contraction for the 128 x 128 tile kernel with a workspace (0 = it does not apply): 49 to
// 128 rows and too few tiles to fill the chip; about 384 workgroups in all (measured 128 ... 1024: fewer
// leave CUs idle, more only add partial tiles for the finishing kernel to read), at least four k-tiles each.
// More rows than that with at most one tile per CU (a projection over 256 ... 1024 tokens: 64 ... 256
// tiles, each walking the whole contraction alone on its CU): the same, two parts from 193 tiles on.
int tile_splitk_plan(long M, long N, long K, long batch, long* k_per_split) {
    if (M <= 48 || K % 64 != 0 || N < 128) return 0;
    if (M <= kSkinnyMaxM && few_rows_by_tiles(M, N, batch)) return 0;
    const long m_tiles = (M + gemm::kBM - 1) / gemm::kBM;
    const long tiles = m_tiles * ((N + gemm::kBN - 1) / gemm::kBN) * batch;
    if (m_tiles > 1 && tiles > 256) return 0;
    const long k_tiles = K / 64;
    long splits = (m_tiles > 1 && tiles > 192) ? 2 : (384 + tiles - 1) / tiles;
    if (splits > k_tiles / 4) splits = k_tiles / 4;
    if (splits < 2) return 0;
    const long per = (k_tiles + splits - 1) / splits;
    splits = (k_tiles + per - 1) / per;
    if (splits < 2 || tiles * splits > 0x7fffffffL) return 0;
    *k_per_split = per * 64;
    return static_cast<int>(splits);
}

int splitk_plan(long M, long N, long K, long batch, int* pieces_per_split) {
    if (M < 32 || M > kSkinnyMaxM || K % 64 != 0 || N < 512) return 0;   // up to 16 rows the activations are no load
    if (few_rows_by_tiles(M, N, batch)) return 0;
    const long pieces = K / 64;
    const long groups = (N + 127) / 128 * batch;
    long splits = (512 + groups - 1) / groups;
    if (splits > pieces / 8) splits = pieces / 8;
    if (splits < 2) return 0;
    long per = (pieces + splits - 1) / splits;
    per = (per + 3) / 4 * 4;                                  // whole slabs
    splits = (pieces + per - 1) / per;
    if (splits < 2 || (N + 127) / 128 > 65535) return 0;
    *pieces_per_split = static_cast<int>(per);
    return static_cast<int>(splits);
}

// ---- any float dtype, any contraction size, any alignment: the product for what the MFMA kernels
// do not take (fp32 / fp64 tensors, K not a multiple of 64, rows that are not 16-byte aligned), so
// that no GEMM leaves the device.  64 x 64 outputs per workgroup, 4 x 4 per thread, k-tiles of 16
// through LDS; fp32 accumulation (fp64 for fp64 tensors) and one rounding, as ATen-CPU does.
template <typename T>
__global__ __launch_bounds__(256) void gemm_nt_any_kernel(const typename Elem<T>::store_t* __restrict__ a,
                                                          const typename Elem<T>::store_t* __restrict__ b,
                                                          const typename Elem<T>::store_t* __restrict__ add,
                                                          typename Elem<T>::store_t* __restrict__ c, const DenseParams p) {
    using El = Elem<T>;
    using Acc = typename std::conditional<sizeof(typename El::store_t) == 8, double, float>::type;
    constexpr int BM = 64, BN = 64, BKK = 16;
    __shared__ Acc as[BKK][BM + 1], bs[BKK][BN + 1];
    const long bidx = blockIdx.z;
    const auto* A = a + bidx * p.sa;
    const auto* B = b + bidx * p.sb;
    const long row0 = static_cast<long>(blockIdx.y) * BM, col0 = static_cast<long>(blockIdx.x) * BN;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int lrow = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;     // staging: 64 rows x 16 k, 4 k per thread
    auto widen = [](typename El::store_t v) -> Acc {
        if constexpr (sizeof(typename El::store_t) == 8) return El::to_f64(v);
        else return El::to_f32(v);
    };
    Acc acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0;
    for (long k0 = 0; k0 < p.K; k0 += BKK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const long k = k0 + lk + e;
            const long ar = row0 + lrow, br = col0 + lrow;
            as[lk + e][lrow] = (ar < p.M && k < p.K) ? widen(A[ar * p.lda + k]) : Acc(0);
            bs[lk + e][lrow] = (br < p.N && k < p.K) ? widen(B[br * p.ldb + k]) : Acc(0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BKK; ++kk) {
            Acc av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
        }
        __syncthreads();
    }
    auto* C = c + bidx * p.sc;
    const auto* ADD = add ? add + bidx * p.sadd : nullptr;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long row = row0 + ty * 4 + i;
        if (row >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long col = col0 + tx * 4 + j;
            if (col >= p.N) continue;
            if constexpr (sizeof(typename El::store_t) == 8) {
                double v = static_cast<double>(p.alpha64) * acc[i][j];
                if (ADD) v += p.beta64 * El::to_f64(ADD[row * p.ld_add + col]);
                C[row * p.ldc + col] = El::from_f64(v);
            } else {
                float v = p.alpha * acc[i][j];
                if (ADD) v = fmaf(p.beta, El::to_f32(ADD[row * p.ld_add + col]), v);
                C[row * p.ldc + col] = El::from_f32(v);
            }
        }
    }
}

// ---- fp32 tensors on the matrix cores: v_mfma_f32_32x32x2_f32 multiplies and accumulates in full
// fp32 (no tf32-style truncation), 157 TFLOP/s at the published clock against the 10-30 the general
// kernel reaches with scalar FMAs.  128 x 128 outputs per workgroup, four waves 2 x 2 with 64 x 64
// each, k-tiles of 16: global -> registers (next k-tile in flight during the MFMAs) -> LDS laid out
// [k][row] so that a lane's operand (row lane % 32, k lane / 32 of a k-pair) is one 4-byte read and
// the 32 lanes of a half read consecutive words.  Any M, N, K and leading dimensions: rows and k
// beyond the end are staged as zeros; 16-byte loads when rows are 16-byte aligned, scalar ones else.
constexpr int kF32BM = 128, kF32BN = 128, kF32BK = 16, kF32LS = kF32BM + 4;
template <bool kVec>
__global__ __launch_bounds__(256, 2) void gemm_nt_f32_mfma_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                  const float* __restrict__ add, float* __restrict__ c, const DenseParams p) {
    __shared__ float as[2][kF32BK][kF32LS], bs[2][kF32BK][kF32LS];
    const long bidx = blockIdx.z;
    const float* A = a + bidx * p.sa;
    const float* B = b + bidx * p.sb;
    const long row0 = static_cast<long>(blockIdx.y) * kF32BM, col0 = static_cast<long>(blockIdx.x) * kF32BN;
    if (p.causal_kind == 1 && col0 > row0 + (kF32BM - 1) + p.causal_first) return;      // no query of this tile sees any of its keys
    long K = p.K;           // (the contraction as far as this tile needs it)
    if (p.causal_kind == 2) {
        const long upto = (row0 + kF32BM + p.causal_first + kF32BK - 1) / kF32BK * kF32BK;
        if (upto < K) K = upto;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    // staging: 128 rows x 4 quads of k per operand = 512 pieces of 4 floats, two per thread; the quad
    // varies fastest so that four lanes read one row's 64 contiguous bytes
    float4_t a_st[2], b_st[2];
    auto fetch = [&](const float* base, long ld, long limit, long r0, long k0, float4_t (&st)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + i * 256;
            const long row = r0 + (idx >> 2), k = k0 + (idx & 3) * 4;
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (row < limit) {
                const float* src = base + row * ld + k;
                if (kVec && k + 3 < K) {
                    v = *reinterpret_cast<const float4_t*>(src);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (k + e < K) v[e] = src[e];
                }
            }
            st[i] = v;
        }
    };
    auto stash = [&](float (&dst)[kF32BK][kF32LS], const float4_t (&st)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 2, kq = (idx & 3) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[kq + e][row] = st[i][e];
        }
    };
    float16_t acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
    const long k_tiles = (K + kF32BK - 1) / kF32BK;
    fetch(A, p.lda, p.M, row0, 0, a_st);
    fetch(B, p.ldb, p.N, col0, 0, b_st);
    stash(as[0], a_st);
    stash(bs[0], b_st);
    __syncthreads();
    for (long kt = 0; kt < k_tiles; ++kt) {
        const int cur = static_cast<int>(kt & 1);
        if (kt + 1 < k_tiles) {
            fetch(A, p.lda, p.M, row0, (kt + 1) * kF32BK, a_st);
            fetch(B, p.ldb, p.N, col0, (kt + 1) * kF32BK, b_st);
        }
#pragma unroll
        for (int kk = 0; kk < kF32BK; kk += 2) {
            float af[2], bf[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) af[mi] = as[cur][kk + lh][wm * 64 + mi * 32 + lr];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) bf[ni] = bs[cur][kk + lh][wn * 64 + ni * 32 + lr];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[mi], bf[ni], acc[mi][ni], 0, 0, 0);
        }
        if (kt + 1 < k_tiles) {
            stash(as[cur ^ 1], a_st);      // the other stage: last read before the previous barrier
            stash(bs[cur ^ 1], b_st);
        }
        __syncthreads();
    }
    // epilogue: lane (column lr, half lh) of block (mi, ni) holds rows (r/4)*8 + 4*lh + r%4
    float* C = c + bidx * p.sc;
    const float* ADD = add ? add + bidx * p.sadd : nullptr;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const long col = col0 + wn * 64 + ni * 32 + lr;
            if (col >= p.N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const long row = row0 + wm * 64 + mi * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
                if (row >= p.M) continue;
                float v = p.alpha * acc[mi][ni][r];
                if (ADD) v = fmaf(p.beta, ADD[row * p.ld_add + col], v);
                C[row * p.ldc + col] = v;
            }
        }
}

template <typename T>
int launch_any(const DenseParams& p, const void* a, const void* b, const void* add, void* c, long batch, hipStream_t s) {
    using S = typename Elem<T>::store_t;
    const long gx = (p.N + 63) / 64, gy = (p.M + 63) / 64;
    PARAS_REQUIRE(gx <= 0x7fffffffL && gy <= 65535 && batch <= 65535, "paras_gemm_nt: shape too large for the general kernel");
    hipLaunchKernelGGL((gemm_nt_any_kernel<T>), dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy), static_cast<unsigned>(batch)),
                       dim3(256), 0, s, static_cast<const S*>(a), static_cast<const S*>(b), static_cast<const S*>(add),
                       static_cast<S*>(c), p);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

template <typename T, typename S>
void launch_dense(const DenseParams& p, unsigned grid, hipStream_t s) {
    hipLaunchKernelGGL((dense_gemm_nt_kernel<T, S>), dim3(grid), dim3(S::kThreads), 0, s, p);
}

}  // namespace
}  // namespace paras

namespace paras {
// paras_gemm_nt_ws with the two hints for causal attention (DenseParams::causal_kind, ::causal_first); also declared in sdpa_internal.h
int gemm_nt_causal(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                   int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                   void* workspace, size_t workspace_bytes, void* stream, int causal_kind, long causal_first);
}  // namespace paras

extern "C" {

size_t paras_gemm_nt_workspace(int64_t M, int64_t N, int64_t K, int64_t batch, int dtype) {
    using namespace paras;
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || (dtype != PARAS_BF16 && dtype != PARAS_F16)) return 0;
    int per = 0;
    long kper = 0;
    if (K % gemm::kBK == 0 && swapped_route(M, N, batch)) return 0;
    int splits = tile_splitk_plan(M, N, K, batch, &kper);
    if (splits == 0) splits = splitk_plan(M, N, K, batch, &per);
    return static_cast<size_t>(splits) * static_cast<size_t>(batch) * static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(float);
}

int paras_gemm_nt(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                  int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                  int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                  void* stream) {
    return paras_gemm_nt_ws(a, b, addend, c, M, N, K, lda, ldb, ldc, ld_add, batch, stride_a, stride_b, stride_c, stride_add,
                            alpha, beta, dtype, nullptr, 0, stream);
}

int paras_gemm_nt_ws(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                     int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                     int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                     void* workspace, size_t workspace_bytes, void* stream) {
    return paras::gemm_nt_causal(a, b, addend, c, M, N, K, lda, ldb, ldc, ld_add, batch, stride_a, stride_b, stride_c, stride_add, alpha, beta,
                                 dtype, workspace, workspace_bytes, stream, 0, 0);
}

}  // extern "C"

// paras_gemm_nt_ws, and for the attention route that multiplies causal score matrices (DenseParams::causal_kind)
int paras::gemm_nt_causal(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                          int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                          void* workspace, size_t workspace_bytes, void* stream, int causal_kind, long causal_first) {
    using namespace paras;
    PARAS_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "paras_gemm_nt: negative shape");
    if (M == 0 || N == 0 || batch == 0) return PARAS_OK;
    PARAS_REQUIRE(dtype == PARAS_BF16 || dtype == PARAS_F16 || dtype == PARAS_F32 || dtype == PARAS_F64,
                  "paras_gemm_nt: unknown dtype");
    PARAS_REQUIRE(c && (K == 0 || (a && b)), "paras_gemm_nt: null pointer");   // an empty contraction has no operands to read
    PARAS_REQUIRE(lda >= K && ldb >= K && ldc >= N && (addend == nullptr || ld_add == 0 || ld_add >= N),
                  "paras_gemm_nt: a leading dimension is smaller than its row");
    hipStream_t s = nullptr;
    int rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    DenseParams p{};
    p.a = static_cast<const std::uint16_t*>(a);
    p.b = static_cast<const std::uint16_t*>(b);
    p.add = static_cast<const std::uint16_t*>(addend);
    p.c = static_cast<std::uint16_t*>(c);
    p.M = M; p.N = N; p.K = K;
    p.lda = lda; p.ldb = ldb; p.ldc = ldc; p.ld_add = ld_add;
    p.sa = stride_a; p.sb = stride_b; p.sc = stride_c; p.sadd = stride_add;
    p.alpha = static_cast<float>(alpha); p.beta = static_cast<float>(beta);
    p.alpha64 = alpha; p.beta64 = beta;
    p.causal_kind = causal_kind; p.causal_first = causal_first;
    // What the MFMA kernels take: 16-bit floats, K a positive multiple of 64, 16-byte aligned operand
    // rows, operands of fewer than 2^32 elements.  Everything else runs on the general kernel.
    const bool mfma_ok = (dtype == PARAS_BF16 || dtype == PARAS_F16) && K > 0 && K % gemm::kBK == 0 &&
                         ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0 && lda % 8 == 0 &&
                         ldb % 8 == 0 && stride_a % 8 == 0 && stride_b % 8 == 0 && M * lda < (1LL << 32) && N * ldb < (1LL << 32);
    if (!mfma_ok) {
        // fp32 products with enough work for 128 x 128 tiles: the fp32 MFMA kernel
        if (dtype == PARAS_F32 && K >= 16 && M >= 64 && N >= 64 && M * N * batch >= 128 * 128 * 32) {
            const long gx = (N + kF32BN - 1) / kF32BN, gy = (M + kF32BM - 1) / kF32BM;
            if (gx <= 0x7fffffffL && gy <= 65535 && batch <= 65535) {
                const bool vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0 && lda % 4 == 0 && ldb % 4 == 0 &&
                                 stride_a % 4 == 0 && stride_b % 4 == 0;
                const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy), static_cast<unsigned>(batch));
                if (vec)
                    hipLaunchKernelGGL((gemm_nt_f32_mfma_kernel<true>), grid, dim3(256), 0, s, static_cast<const float*>(a), static_cast<const float*>(b),
                                       static_cast<const float*>(addend), static_cast<float*>(c), p);
                else
                    hipLaunchKernelGGL((gemm_nt_f32_mfma_kernel<false>), grid, dim3(256), 0, s, static_cast<const float*>(a), static_cast<const float*>(b),
                                       static_cast<const float*>(addend), static_cast<float*>(c), p);
                PARAS_HIP_TRY(hipGetLastError());
                return PARAS_OK;
            }
        }
        switch (dtype) {
            case PARAS_F32:  return launch_any<float>(p, a, b, addend, c, batch, s);
            case PARAS_F64:  return launch_any<double>(p, a, b, addend, c, batch, s);
            case PARAS_BF16: return launch_any<bf16_t>(p, a, b, addend, c, batch, s);
            default:         return launch_any<f16_t>(p, a, b, addend, c, batch, s);
        }
    }
    // Few output columns and many rows (a router's logits: tokens x experts): the product is bound by
    // reading a once, which 128 x 128 tiles on N / 128 of the CUs do badly (M = 16384, K = 4096:
    // N = 8 in 78 us, N = 128 in 78 us).  The few-row kernels stream a long operand with every CU and
    // keep the short one in registers, so the operands change places and the results are stored
    // transposed.
    if (swapped_route(M, N, batch)) {
        DenseParams q = p;
        q.a = p.b; q.b = p.a;
        q.M = N; q.N = M;
        q.lda = ldb; q.ldb = lda;
        q.sa = stride_b; q.sb = stride_a;
        q.swapped = 1;
        if (dtype == PARAS_BF16) launch_skinny<bf16_t>(q, batch, s);
        else                     launch_skinny<f16_t>(q, batch, s);
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    int64_t n_units = (N + 2 * gemm::kBN - 1) / (2 * gemm::kBN);
    const int64_t wide_tiles = (M + gemm::wide::kBM - 1) / gemm::wide::kBM * n_units * batch;
    // measured: faster from a little over half a round of one workgroup per CU upwards (at exactly 128
    // tiles the 128 x 128 tiling below wins by 10-25 %, at 160 the 256-row tiles win by 20 %)
    const bool use_wide = wide_tiles >= 144 && M > gemm::kBM;
    const int64_t bm = use_wide ? gemm::wide::kBM : gemm::kBM;
    const int64_t m_tiles = (M + bm - 1) / bm;
    // fewer 128 x 256 tiles than the chip holds at once (two per CU): 128 x 128 tiles, twice as many
    const bool use_square = !use_wide && m_tiles * n_units * batch < 512 && N > gemm::kBN;
    if (use_square) n_units = (N + gemm::kBN - 1) / gemm::kBN;
    PARAS_REQUIRE(m_tiles * n_units * batch <= 0x7fffffffLL, "paras_gemm_nt: too many tiles");
    p.m_tiles = static_cast<int>(m_tiles); p.n_units = static_cast<int>(n_units);
    if (workspace != nullptr && batch <= 65535) {
        long kper = 0;
        const int tsplits = tile_splitk_plan(M, N, K, batch, &kper);
        const size_t tneed = static_cast<size_t>(tsplits) * static_cast<size_t>(batch) * static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(float);
        if (tsplits >= 2 && workspace_bytes >= tneed && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
            p.m_tiles = static_cast<int>((M + gemm::kBM - 1) / gemm::kBM);
            p.n_units = static_cast<int>((N + gemm::kBN - 1) / gemm::kBN);
            p.splits = tsplits;
            p.k_per_split = kper;
            p.partial = static_cast<float*>(workspace);
            const unsigned blocks = static_cast<unsigned>(static_cast<long>(p.m_tiles) * p.n_units * batch * tsplits);
            const bool bf = dtype == PARAS_BF16;
            if (bf) hipLaunchKernelGGL((dense_gemm_nt_kernel<bf16_t, gemm::Tile128x128, true>), dim3(blocks), dim3(gemm::Tile128x128::kThreads), 0, s, p);
            else    hipLaunchKernelGGL((dense_gemm_nt_kernel<f16_t, gemm::Tile128x128, true>), dim3(blocks), dim3(gemm::Tile128x128::kThreads), 0, s, p);
            PARAS_HIP_TRY(hipGetLastError());
            const dim3 fgrid(static_cast<unsigned>((M * N + 255) / 256), static_cast<unsigned>(batch));
            if (bf) hipLaunchKernelGGL((skinny_splitk_finish_kernel<bf16_t>), fgrid, dim3(256), 0, s, p, p.partial, tsplits);
            else    hipLaunchKernelGGL((skinny_splitk_finish_kernel<f16_t>), fgrid, dim3(256), 0, s, p, p.partial, tsplits);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
        int per = 0;
        const int splits = splitk_plan(M, N, K, batch, &per);
        const size_t need = static_cast<size_t>(splits) * static_cast<size_t>(batch) * static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(float);
        if (splits >= 2 && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
            const dim3 grid(static_cast<unsigned>(splits), static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>(batch));
            const int mb = static_cast<int>((M + 15) / 16);
            float* part = static_cast<float*>(workspace);
            const bool bf = dtype == PARAS_BF16;
            if (mb <= 2)      { if (bf) hipLaunchKernelGGL((skinny_splitk_kernel<bf16_t, 2>), grid, dim3(512), 0, s, p, part, per);
                                else    hipLaunchKernelGGL((skinny_splitk_kernel<f16_t, 2>), grid, dim3(512), 0, s, p, part, per); }
            else if (mb <= 4) { if (bf) hipLaunchKernelGGL((skinny_splitk_kernel<bf16_t, 4>), grid, dim3(512), 0, s, p, part, per);
                                else    hipLaunchKernelGGL((skinny_splitk_kernel<f16_t, 4>), grid, dim3(512), 0, s, p, part, per); }
            else              { if (bf) hipLaunchKernelGGL((skinny_splitk_kernel<bf16_t, 8>), grid, dim3(512), 0, s, p, part, per);
                                else    hipLaunchKernelGGL((skinny_splitk_kernel<f16_t, 8>), grid, dim3(512), 0, s, p, part, per); }
            PARAS_HIP_TRY(hipGetLastError());
            const dim3 fgrid(static_cast<unsigned>((M * N + 255) / 256), static_cast<unsigned>(batch));
            if (bf) hipLaunchKernelGGL((skinny_splitk_finish_kernel<bf16_t>), fgrid, dim3(256), 0, s, p, part, splits);
            else    hipLaunchKernelGGL((skinny_splitk_finish_kernel<f16_t>), fgrid, dim3(256), 0, s, p, part, splits);
            PARAS_HIP_TRY(hipGetLastError());
            return PARAS_OK;
        }
    }
    if (!few_rows_by_tiles(M, N, batch) && M <= kSkinnyMaxM && batch <= 65535 && (N + 15) / 16 <= 0x7fffffffLL) {
        if (dtype == PARAS_BF16) launch_skinny<bf16_t>(p, batch, s);
        else                     launch_skinny<f16_t>(p, batch, s);
        PARAS_HIP_TRY(hipGetLastError());
        return PARAS_OK;
    }
    unsigned blocks = static_cast<unsigned>(m_tiles * n_units * batch);
    if (use_wide && m_tiles >= kXcdBlockM && n_units >= kXcdBlockN) {
        const long xbm = (m_tiles + kXcdBlockM - 1) / kXcdBlockM, xbn = (n_units + kXcdBlockN - 1) / kXcdBlockN;
        const long wgs = xbm * xbn <= 0x7fffffLL ? xcd_order_workgroups(static_cast<int>(xbm * xbn)) * batch : -1;
        if (wgs > 0 && wgs <= 0x7fffffffLL) {
            p.xcd_blocks = static_cast<int>(xbm * xbn);
            p.xcd_blocks_n = static_cast<int>(xbn);
            blocks = static_cast<unsigned>(wgs);
        }
    }
    static const bool eight_waves = std::getenv("PARAS_GEMM_EIGHT_WAVES") != nullptr;     // the eight-wave tile of 32 x 32 x 16 MFMAs, for measurements
    if (use_wide && !eight_waves) {
        if (dtype == PARAS_BF16) hipLaunchKernelGGL((dense_gemm_nt_quad16_kernel<bf16_t>), dim3(blocks), dim3(quad16::kThreads), 0, s, p);
        else                     hipLaunchKernelGGL((dense_gemm_nt_quad16_kernel<f16_t>), dim3(blocks), dim3(quad16::kThreads), 0, s, p);
    } else if (use_wide) {
        if (dtype == PARAS_BF16) launch_dense<bf16_t, gemm::Tile256>(p, blocks, s);
        else                     launch_dense<f16_t, gemm::Tile256>(p, blocks, s);
    } else if (use_square) {
        if (dtype == PARAS_BF16) launch_dense<bf16_t, gemm::Tile128x128>(p, blocks, s);
        else                     launch_dense<f16_t, gemm::Tile128x128>(p, blocks, s);
    } else {
        if (dtype == PARAS_BF16) launch_dense<bf16_t, gemm::Tile128>(p, blocks, s);
        else                     launch_dense<f16_t, gemm::Tile128>(p, blocks, s);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}
