// Tile mainloops shared by the MFMA GEMM kernels (grouped expert GEMMs and the
// dense NT GEMM): C tile = A[rows x K] * B[256 x K]^T with bf16/fp16 operands and
// fp32 accumulation on v_mfma_f32_32x32x16.
//
// Both operands are read along their contiguous contraction dim, which is the
// 8-element-per-lane operand layout of the MFMA, so neither needs a transpose.
// The 256 B rows come as two groups of 128 (gate / up weights, or two adjacent
// column blocks) and each wave owns 64x64 of each group: 128 fp32 accumulators
// per lane.  k-tile 64, global -> registers -> LDS with the next k-tile's loads
// in flight during the MFMAs.  Two shapes: 128 rows with 4 waves arranged 2x2
// (two workgroups per CU, each with a single LDS stage), and 256 rows with 8
// waves arranged 4x2 (one workgroup per CU, two LDS stages, namespace wide).
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "core/device_math.h"

namespace paras {
namespace gemm {

constexpr int kThreads = 256;
constexpr int kBM = 128;
constexpr int kBN = 128;          // columns per group; a workgroup computes two groups
constexpr int kBK = 64;
constexpr int kLS = kBK + 8;      // LDS row stride (elements): 16 consecutive rows hit distinct banks.  (Unpadded rows
                                  // with an XOR swizzle of the chunks measured no faster.)

typedef short i16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct MmaT;
template <> struct MmaT<bf16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct MmaT<f16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};


template <int G>     // G column groups of 128
struct TileLdsG {
    std::uint16_t a[kBM * kLS];
    std::uint16_t b[G][kBN * kLS];
};
using TileLds = TileLdsG<2>;

// a_off[i] / b_off[g][i]: element offsets (from the uniform bases a_base / b_base[g]) of this
// thread's four 16-byte chunks per operand row set at k = 0 (chunk c = tid + i*256 -> tile row
// c/8, column (c%8)*8).  32-bit offsets against a scalar base keep the addressing out of the
// vector registers; callers check that every operand spans fewer than 2^32 elements.
// Accumulates into acc[g][mi][ni]; lane (column lr = lane%32, half lh = lane/32) of
// block (mi, ni) ends up holding rows (r/4)*8 + 4*lh + r%4, r = 0..15.
template <typename T, int G>
__device__ __forceinline__ void tile_mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[4],
                                              const std::uint16_t* const (&b_base)[G], const unsigned (&b_off)[G][4],
                                              long K, TileLdsG<G>& lds, float16_t (&acc)[G][2][2]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    std::uint16_t* a_lds = lds.a;
    std::uint16_t (*b_lds)[kBN * kLS] = lds.b;
    u32x4 a_st[4], b_st[G][4];
    auto load_tile = [&](long k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) a_st[i] = load16(a_base + k0 + a_off[i]);
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) b_st[g][i] = load16(b_base[g] + k0 + b_off[g][i]);
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * kThreads;
            const int off = (c >> 3) * kLS + (c & 7) * 8;
            *reinterpret_cast<u32x4*>(&a_lds[off]) = a_st[i];
#pragma unroll
            for (int g = 0; g < G; ++g) *reinterpret_cast<u32x4*>(&b_lds[g][off]) = b_st[g][i];
        }
    };

#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[g][mi][ni][r] = 0.f;

    const int a_off0 = (wm * 64 + lr) * kLS + lh * 8;
    const int b_off0 = (wn * 64 + lr) * kLS + lh * 8;
    const long k_tiles = K / kBK;
    load_tile(0);
    store_tile();
    __syncthreads();
    for (long kt = 0; kt < k_tiles; ++kt) {
        if (kt + 1 < k_tiles) load_tile((kt + 1) * kBK);
        // Fixed issue order, fenced slot by slot: one MFMA per slot, the fragments of the next
        // k-step requested while the current one computes (A into a second register pair right
        // away, each B fragment back into its own registers as soon as its two MFMAs have
        // issued), so an operand is asked for about six MFMAs before it is used.
        constexpr int Q = 2 * G;               // B fragments per k-step
        i16x8 af[2][2], bf[Q];
        auto read_a = [&](int buf, int ks) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
                af[buf][mi] = *reinterpret_cast<const i16x8*>(&a_lds[a_off0 + mi * 32 * kLS + ks * 16]);
        };
        auto read_b = [&](int q, int ks) {   // q = 2*g + ni
            bf[q] = *reinterpret_cast<const i16x8*>(&b_lds[q >> 1][b_off0 + (q & 1) * 32 * kLS + ks * 16]);
        };
        read_a(0, 0);
#pragma unroll
        for (int q = 0; q < Q; ++q) read_b(q, 0);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            const int cur = ks & 1;
            const bool more = ks + 1 < kBK / 16;
#pragma unroll
            for (int q = 0; q < Q; ++q)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) {
                    acc[q >> 1][mi][q & 1] = MmaT<T>::run(af[cur][mi], bf[q], acc[q >> 1][mi][q & 1]);
                    if (more && q == 0 && mi == 0) read_a(cur ^ 1, ks + 1);
                    if (more && mi == 1) read_b(q, ks + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
        __syncthreads();
        if (kt + 1 < k_tiles) {
            store_tile();
            __syncthreads();
        }
    }

}

// The same per-wave work (64 x 64 of each column group) with eight waves arranged 4 x 2 over a
// 256 x (2 x 128) tile: a third fewer global loads and LDS stores per flop than the 128-row tile.
// The eight waves move in step (one barrier per k-tile), so LDS is double buffered and a k-tile is
// in registers for a whole tile time before it is stored.
namespace wide {

constexpr int kThreads = 512;
constexpr int kBM = 256;

struct StageLds {
    std::uint16_t a[kBM * kLS];
    std::uint16_t b[2][kBN * kLS];
};
struct TileLds {
    StageLds st[2];
};

// a_off[i]: chunk c = tid + i*512 -> tile row c/8, column (c%8)*8 (i < 4); b_off[g][i]: the same
// for the 128 rows of column group g (i < 2).
template <typename T>
__device__ __forceinline__ void tile_mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[4],
                                              const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][2],
                                              long K, TileLds& lds, float16_t (&acc)[2][2][2]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    u32x4 a_st[4], b_st[2][2];
    auto load_one = [&](int idx, long k0) {              // idx 0..3: A chunks, 4..7: B chunks (g, i)
        if (idx < 4) a_st[idx] = load16(a_base + k0 + a_off[idx]);
        else         b_st[(idx - 4) >> 1][(idx - 4) & 1] = load16(b_base[(idx - 4) >> 1] + k0 + b_off[(idx - 4) >> 1][(idx - 4) & 1]);
    };
    auto load_tile = [&](long k0) {
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) load_one(idx, k0);
    };
    auto store_one = [&](StageLds& st, int idx) {
        const int i = idx < 4 ? idx : (idx - 4) & 1;
        const int c = tid + i * kThreads;
        const int off = (c >> 3) * kLS + (c & 7) * 8;
        if (idx < 4) *reinterpret_cast<u32x4*>(&st.a[off]) = a_st[idx];
        else         *reinterpret_cast<u32x4*>(&st.b[(idx - 4) >> 1][off]) = b_st[(idx - 4) >> 1][i];
    };

#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[g][mi][ni][r] = 0.f;

    const int a_off0 = (wm * 64 + lr) * kLS + lh * 8;
    const int b_off0 = (wn * 64 + lr) * kLS + lh * 8;
    const long k_tiles = K / kBK;
    // The k-steps form one continuous pipeline across k-tiles: the operand fragments of a k-step are
    // requested while the previous one computes, also across the tile boundary.  For that the
    // barrier of a tile sits before its LAST k-step: by then the next k-tile has been stored into
    // the other stage (one 16-byte store per MFMA pair of k-steps 1 and 2, each followed by the
    // global load of the same chunk of the tile after that; nobody reads that stage between the
    // previous barrier and this one), after it the last k-step's MFMAs run from registers while
    // the first fragments of the next tile are requested.
    i16x8 af[2][2], bf[4];
    auto read_a = [&](const StageLds& st, int buf, int ks) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
            af[buf][mi] = *reinterpret_cast<const i16x8*>(&st.a[a_off0 + mi * 32 * kLS + ks * 16]);
    };
    auto read_b = [&](const StageLds& st, int q, int ks) {   // q = 2*g + ni
        bf[q] = *reinterpret_cast<const i16x8*>(&st.b[q >> 1][b_off0 + (q & 1) * 32 * kLS + ks * 16]);
    };
    auto compute = [&](const StageLds& cur_st, StageLds& nxt_st, long k_after, auto next_tag) {
        constexpr bool kNext = decltype(next_tag)::value;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            const int cur = ks & 1;
            const bool last = ks + 1 == kBK / 16;
            if (kNext && last) __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) {
                    acc[q >> 1][mi][q & 1] = MmaT<T>::run(af[cur][mi], bf[q], acc[q >> 1][mi][q & 1]);
                    if (!last) {
                        if (q == 0 && mi == 0) read_a(cur_st, cur ^ 1, ks + 1);
                        if (mi == 1) read_b(cur_st, q, ks + 1);
                    } else if (kNext) {
                        if (q == 0 && mi == 0) read_a(nxt_st, cur ^ 1, 0);
                        if (mi == 1) read_b(nxt_st, q, 0);
                    }
                    if (kNext && (ks == 1 || ks == 2) && mi == 0) {
                        store_one(nxt_st, (ks - 1) * 4 + q);
                        load_one((ks - 1) * 4 + q, k_after);   // the register is free again: a whole tile of time to arrive
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    };
    load_tile(0);
#pragma unroll
    for (int idx = 0; idx < 8; ++idx) store_one(lds.st[0], idx);
    __syncthreads();
    if (k_tiles > 1) load_tile(kBK);
    read_a(lds.st[0], 0, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) read_b(lds.st[0], q, 0);
    for (long kt = 0; kt + 1 < k_tiles; ++kt) {
        const long after = kt + 2 < k_tiles ? kt + 2 : k_tiles - 1;   // the last tiles reload a tile nobody stores
        compute(lds.st[kt & 1], lds.st[(kt + 1) & 1], after * kBK, std::true_type{});
    }
    compute(lds.st[(k_tiles - 1) & 1], lds.st[k_tiles & 1], 0, std::false_type{});
}

// A 256-row tile of which at most 64 rows exist (the last tile of a group of rows): the eight
// waves share those 64 rows instead of six of them idling through the whole contraction.  Wave w
// takes row block w / 4 (32 rows) and the 32 columns w % 4 of BOTH column groups, so a gate / up
// pair still meets in one lane: 2 MFMAs per k-step and wave instead of 8, every product summed in
// the same order as in the full tile (bit-identical results).  Only the first 64 A rows are staged
// (a_off0: this thread's chunk of them); two LDS stages, one barrier per k-tile.
template <typename T>
__device__ __forceinline__ void short_tile_mainloop(const std::uint16_t* a_base, unsigned a_off0,
                                                    const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][2],
                                                    long K, TileLds& lds, float16_t (&acc)[2]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int rb = wave >> 2, cb = wave & 3;
    u32x4 a_st, b_st[2][2];
    auto load_tile = [&](long k0) {
        a_st = load16(a_base + k0 + a_off0);
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
            for (int i = 0; i < 2; ++i) b_st[g][i] = load16(b_base[g] + k0 + b_off[g][i]);
    };
    auto store_tile = [&](StageLds& st) {
        *reinterpret_cast<u32x4*>(&st.a[(tid >> 3) * kLS + (tid & 7) * 8]) = a_st;
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int c = tid + i * kThreads;
                *reinterpret_cast<u32x4*>(&st.b[g][(c >> 3) * kLS + (c & 7) * 8]) = b_st[g][i];
            }
    };
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[g][r] = 0.f;
    const int a_o = (rb * 32 + lr) * kLS + lh * 8;
    const int b_o = (cb * 32 + lr) * kLS + lh * 8;
    const long k_tiles = K / kBK;
    load_tile(0);
    store_tile(lds.st[0]);
    __syncthreads();
    for (long kt = 0; kt < k_tiles; ++kt) {
        const StageLds& cur = lds.st[kt & 1];
        if (kt + 1 < k_tiles) load_tile((kt + 1) * kBK);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            const i16x8 af = *reinterpret_cast<const i16x8*>(&cur.a[a_o + ks * 16]);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const i16x8 bf = *reinterpret_cast<const i16x8*>(&cur.b[g][b_o + ks * 16]);
                acc[g] = MmaT<T>::run(af, bf, acc[g]);
            }
        }
        if (kt + 1 < k_tiles) store_tile(lds.st[(kt + 1) & 1]);
        __syncthreads();
    }
}

}  // namespace wide

// The 256 x (2 x 128) tile once more, for the dense kernel: four waves arranged 2 x 2, one wave per
// SIMD, each with 128 x 128 as 8 x 8 blocks of v_mfma_f32_16x16x32 (four accumulator registers per
// block, 256 in all: the accumulation half of the register file).  Per flop that instruction
// moves half the accumulator data of the 32 x 32 x 16 one, and the part is power limited under
// MFMA load: a register-only loop of it sustains 2.19 PFLOP/s where the 32 x 32 x 16 loop sustains
// 1.90 - 1.94.  A k-step (32 elements of the contraction) is 64 MFMAs on 8 + 8 fragments: a
// quarter of an LDS read per MFMA, i.e. half a read per 32 x 32 x 16's worth of flops (0.75 in the
// eight-wave tile).  Staging, stages and the place of the barrier as in the eight-wave tile.  The
// B fragment is the instruction's first operand, so a lane ends up with four adjacent COLUMNS of
// one row (8-byte stores): acc[i][j][r] = row i*16 + lane%16, column block j, column 4*(lane/16) + r of it.
namespace quad16 {

constexpr int kThreads = 256;
constexpr int kBM = 256;
using wide::StageLds;
using wide::TileLds;
typedef float float4v __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ static __forceinline__ float4v run(i16x8 a, i16x8 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    __device__ static __forceinline__ float4v run(i16x8 a, i16x8 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

template <typename T>
__device__ __forceinline__ void tile_mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[8],
                                              const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][4],
                                              long K, TileLds& lds, float4v (&acc)[8][8]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, kq = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    u32x4 a_st[8], b_st[2][4];
    auto load_one = [&](int idx, long k0) {              // idx 0..7: A chunks, 8..15: B chunks (g, i)
        if (idx < 8) a_st[idx] = load16(a_base + k0 + a_off[idx]);
        else         b_st[(idx - 8) >> 2][(idx - 8) & 3] = load16(b_base[(idx - 8) >> 2] + k0 + b_off[(idx - 8) >> 2][(idx - 8) & 3]);
    };
    auto store_one = [&](StageLds& st, int idx) {
        const int i = idx < 8 ? idx : (idx - 8) & 3;
        const int c = tid + i * kThreads;
        const int off = (c >> 3) * kLS + (c & 7) * 8;
        if (idx < 8) *reinterpret_cast<u32x4*>(&st.a[off]) = a_st[idx];
        else         *reinterpret_cast<u32x4*>(&st.b[(idx - 8) >> 2][off]) = b_st[(idx - 8) >> 2][i];
    };
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    const int a_off0 = (wm * 128 + l16) * kLS + kq * 8;
    const int b_off0 = (wn * 64 + l16) * kLS + kq * 8;
    const long k_tiles = K / kBK;
    // fragments of a k-step (32 elements of the contraction): 8 of A (16 rows each), 8 of B (column
    // blocks j: group j / 4, columns wn*64 + (j % 4)*16 ..); two register sets
    i16x8 af[2][8], bf[2][8];
    auto read_frag = [&](const StageLds& st, int buf, int f, int ks) {     // f 0..7: A block, 8..15: B block
        if (f < 8) af[buf][f] = *reinterpret_cast<const i16x8*>(&st.a[a_off0 + f * 16 * kLS + ks * 32]);
        else       bf[buf][f - 8] = *reinterpret_cast<const i16x8*>(&st.b[(f - 8) >> 2][b_off0 + ((f - 8) & 3) * 16 * kLS + ks * 32]);
    };
    auto compute = [&](const StageLds& cur_st, StageLds& nxt_st, long k_after, auto next_tag) {
        constexpr bool kNext = decltype(next_tag)::value;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bool last = ks == 1;
            if (kNext && last) __syncthreads();
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int slot = j * 8 + i;
                    acc[i][j] = Mma<T>::run(bf[ks][j], af[ks][i], acc[i][j]);
                    if ((slot & 3) == 0) {          // one fragment of the next k-step every fourth MFMA
                        if (!last) read_frag(cur_st, 1, slot >> 2, 1);
                        else if (kNext) read_frag(nxt_st, 0, slot >> 2, 0);
                    }
                    // the next k-tile into the other stage during the first k-step, one chunk every fourth MFMA, each
                    // followed two MFMAs later by the global load of the same chunk of the tile after that
                    if (kNext && !last && (slot & 3) == 1) store_one(nxt_st, slot >> 2);
                    if (kNext && !last && (slot & 3) == 3) load_one(slot >> 2, k_after);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    };
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) load_one(idx, 0);
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) store_one(lds.st[0], idx);
    __syncthreads();
    if (k_tiles > 1) {
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) load_one(idx, kBK);
    }
#pragma unroll
    for (int f = 0; f < 16; ++f) read_frag(lds.st[0], 0, f, 0);
    for (long kt = 0; kt + 1 < k_tiles; ++kt) {
        const long after = kt + 2 < k_tiles ? kt + 2 : k_tiles - 1;   // the last tiles reload a tile nobody stores
        compute(lds.st[kt & 1], lds.st[(kt + 1) & 1], after * kBK, std::true_type{});
    }
    compute(lds.st[(k_tiles - 1) & 1], lds.st[k_tiles & 1], 0, std::false_type{});
}

// A tile of which at most 64 rows exist (the last tile of a group of rows): the four waves share those
// rows instead of three of them idling through the contraction.  Wave w takes all four row blocks and
// the 32 columns w of BOTH column groups (two blocks of 16 each), so a gate / up pair still meets in one
// lane: 16 MFMAs per k-step and wave instead of 64, every product summed in the same order as in the full
// tile (bit-identical results).  Only the first 64 A rows are staged (a_off[0], a_off[1]: this thread's two
// chunks of them); two LDS stages, one barrier per k-tile.  acc[i][jj]: row block i, column block
// jj = 2 g + cb: rows i*16 + lane%16, columns w*32 + cb*16 + 4*(lane/16) + r of group g.
template <typename T>
__device__ __forceinline__ void short_tile_mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[8],
                                                    const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][4],
                                                    long K, TileLds& lds, float4v (&acc)[4][4]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, kq = lane >> 4;
    u32x4 a_st[2], b_st[2][4];
    auto load_tile = [&](long k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) a_st[i] = load16(a_base + k0 + a_off[i]);
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) b_st[g][i] = load16(b_base[g] + k0 + b_off[g][i]);
    };
    auto store_tile = [&](StageLds& st) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * kThreads;
            const int off = (c >> 3) * kLS + (c & 7) * 8;
            if (i < 2) *reinterpret_cast<u32x4*>(&st.a[off]) = a_st[i];
#pragma unroll
            for (int g = 0; g < 2; ++g) *reinterpret_cast<u32x4*>(&st.b[g][off]) = b_st[g][i];
        }
    };
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) acc[i][jj] = float4v{0.f, 0.f, 0.f, 0.f};
    const int a_o = l16 * kLS + kq * 8;
    const int b_o = (wave * 32 + l16) * kLS + kq * 8;
    const long k_tiles = K / kBK;
    load_tile(0);
    store_tile(lds.st[0]);
    __syncthreads();
    for (long kt = 0; kt < k_tiles; ++kt) {
        const StageLds& cur = lds.st[kt & 1];
        if (kt + 1 < k_tiles) load_tile((kt + 1) * kBK);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            i16x8 af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const i16x8*>(&cur.a[a_o + i * 16 * kLS + ks * 32]);
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) bf[jj] = *reinterpret_cast<const i16x8*>(&cur.b[jj >> 1][b_o + (jj & 1) * 16 * kLS + ks * 32]);
#pragma unroll
            for (int jj = 0; jj < 4; ++jj)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i][jj] = Mma<T>::run(bf[jj], af[i], acc[i][jj]);
        }
        if (kt + 1 < k_tiles) store_tile(lds.st[(kt + 1) & 1]);
        __syncthreads();
    }
}

}  // namespace quad16

// ---- epilogue helpers.  A lane (column lr, half lh) of a 32 x 32 accumulator block holds rows
// (r/4)*8 + 4*lh + r%4, r = 0..15.  Stores go to `blk` (the block's first column in the tile's first
// row: the same address in every lane, so it stays in scalar registers) plus a 32-bit byte offset:
// `lane_b` (this lane's first row and column) plus a row offset that is again the same in every lane.
// kFull: the whole tile lies inside the matrix, no row is tested.
template <bool kFull>
__device__ __forceinline__ void store_block(char* blk, unsigned lane_b, unsigned ld2, int mi, int nrows, const std::uint16_t (&o)[16]) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int ro = mi * 32 + (r >> 2) * 8 + (r & 3);
        if (kFull || ro < nrows) *reinterpret_cast<std::uint16_t*>(blk + (lane_b + static_cast<unsigned>(ro) * ld2)) = o[r];
    }
}
// Narrows a block of plain results: the conversion instruction, and once more in software (which
// writes NaNs as the host's types do) if a NaN turns up anywhere in the wave's block.
template <typename T>
__device__ __forceinline__ void narrow_block(const float16_t& a, std::uint16_t (&o)[16]) {
    float probe = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        o[r] = Elem<T>::from_f32_finite(a[r]);
        probe += a[r];
    }
    if (__builtin_amdgcn_ballot_w64(probe != probe) != 0) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r = 0; r < 16; ++r) o[r] = Elem<T>::from_f32(a[r]);
    }
}

// The two tile shapes as a kernel sees them.
template <int G>
struct Tile128G {
    static constexpr int kBM = gemm::kBM, kThreads = gemm::kThreads, kBChunks = 4, kGroups = G;
    static constexpr int kShortRows = 0;    // no short-tile form
    using Lds = TileLdsG<G>;
    template <typename T>
    __device__ static __forceinline__ void mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[4],
                                                    const std::uint16_t* const (&b_base)[G], const unsigned (&b_off)[G][4],
                                                    long K, Lds& lds, float16_t (&acc)[G][2][2]) {
        tile_mainloop<T, G>(a_base, a_off, b_base, b_off, K, lds, acc);
    }
};
using Tile128 = Tile128G<2>;
using Tile128x128 = Tile128G<1>;     // one column group: twice the workgroups for problems that would not fill the chip
struct Tile256 {
    static constexpr int kBM = wide::kBM, kThreads = wide::kThreads, kBChunks = 2, kGroups = 2;
    using Lds = wide::TileLds;
    template <typename T>
    __device__ static __forceinline__ void mainloop(const std::uint16_t* a_base, const unsigned (&a_off)[4],
                                                    const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][2],
                                                    long K, Lds& lds, float16_t (&acc)[2][2][2]) {
        wide::tile_mainloop<T>(a_base, a_off, b_base, b_off, K, lds, acc);
    }
    static constexpr int kShortRows = 64;   // a tile with no more valid rows than this can take short_mainloop
    template <typename T>
    __device__ static __forceinline__ void short_mainloop(const std::uint16_t* a_base, unsigned a_off0,
                                                          const std::uint16_t* const (&b_base)[2], const unsigned (&b_off)[2][2],
                                                          long K, Lds& lds, float16_t (&acc)[2]) {
        wide::short_tile_mainloop<T>(a_base, a_off0, b_base, b_off, K, lds, acc);
    }
};

}  // namespace gemm
}  // namespace paras
