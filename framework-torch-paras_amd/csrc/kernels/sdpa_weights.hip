// Attention with returned weights on the matrix cores (bf16 / fp16): the math op
// aten::_scaled_dot_product_attention_math must hand back softmax(q k^T * scale + mask)
// as a tensor (csrc/ops/attention_ops.cpp:128-135), which a flash kernel never forms.
//
// This kernel forms it, narrowing exactly where the reference's composition narrows:
//   s1 = T(q k^T)            fp32 accumulation on MFMA, one rounding     (bmm, vision_ops.cpp:398-406)
//   s2 = T(s1 * scale)       evaluated in double like the host's mul_out  (pointwise_ops.cpp:280-284)
//   s3 = masked_fill(-inf) / T(s2 + mask)                                (attention_ops.cpp:103-125)
//   w  = T(exp(s3 - max) / sum)   row max and row sum over the NARROWED scores (softmax_out, :959-976)
//   out = T(w v)             the narrowed weights are the operand of the second product (attention_ops.cpp:134)
// so the weights differ from the reference's only where fp32 instead of fp64 softmax arithmetic
// lands on the other side of a rounding boundary (one unit in the last place of T, for about one
// weight in a thousand), and `out` differs by the accumulation order of the products.
//
// Two passes over the keys per block of 128 queries (a lane owns a query as in the flash kernel:
// S^T = K Q^T on v_mfma_f32_32x32x16, O^T = V^T W^T):
//   pass 1   scores tile by tile, running row max and row sum (each lane over its own share of the
//            keys; the shares of a query are merged once at the end)
//   pass 2   scores again, weights written to `attn`, and the product with V accumulated
// The arithmetic per score, not memory, sets the pace (two roundings, a scaling, the mask, an
// exponential, a narrowing), so the work of a query block is spread over eight wavefronts: four
// groups of 32 queries times two halves of every 128-key tile.  K / V tiles go global -> registers
// -> LDS, double buffered: the next tile's loads are in flight while the current one is computed,
// one barrier per tile.  Under a causal mask a workgroup takes a pair of query blocks, the i-th
// from the end and the i-th from the start, so every workgroup walks the same number of key tiles;
// blocks of 32 keys that lie wholly below the diagonal skip the per-key tests.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <cmath>
#include <mutex>
#include <set>
#include <utility>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_internal.h"

namespace paras {
namespace {

constexpr int kBN = 64;    // keys per key group and tile
constexpr int kTile = 128; // keys per staged tile: two key groups
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kBM = 128;   // queries per workgroup: 4 waves x 32

typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

struct WeightsParams {
    const std::uint16_t* q;
    const std::uint16_t* k;
    const std::uint16_t* v;
    std::uint16_t*       out;
    std::uint16_t*       attn;
    float*               lse;
    long qs_b, qs_h, qs_l;  // element strides
    long ks_b, ks_h, ks_l;
    long vs_b, vs_h, vs_l;
    int  B, Hq, Hkv, Lq, Lk;
    int  n_qblocks;
    double scale;           // multiplies T(q k^T) in double, as the host engine's mul_out does
    int    scale_is_f32;    // the scale is a float: an fp32 multiply gives the same rounded product
    const unsigned char* mask;
    long ms_b, ms_h, ms_q, ms_k;  // element strides (0 = broadcast)
};

template <typename T> struct Mma16;
template <> struct Mma16<bf16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma16<f16_t> {
    __device__ static __forceinline__ float16_t run(i16x8 a, i16x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

// v_permlane32_swap exchanges lanes 32..63 of its first register with lanes 0..31 of its second:
// fed the same value twice, every lane ends up with the lower half's value in `lo` and the upper
// half's in `hi`.  (Inline asm with the wait states spelled out: see the flash kernel.)
__device__ __forceinline__ void halves(float x, float& lo, float& hi) {
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lo = a;
    hi = b;
}

// kMode: 0 no mask, 1 bool mask bytes (nonzero = attend), 2 additive mask of type T, 3 causal.
//
// Eight wavefronts per workgroup: wave = query group (0..3, 32 queries each) + 4 * key group
// (0..1).  A staged tile holds 128 keys; key group g works on its keys [64 g, 64 g + 64).  The two
// waves that share queries merge their row maxima and sums after pass 1 and their partial W V
// products after pass 2, both through LDS.
template <typename T, int D, int kMode>
__global__ __launch_bounds__(512, 2) void weights_fwd_kernel(const WeightsParams p) {
    using El = Elem<T>;
    constexpr int NW = 8;
    constexpr int KSTEPS = D / 16;
    constexpr int DBLK = D / 32;
    constexpr int CHUNKS = D / 8;          // 16-byte chunks per row
    constexpr int RPI = 64 / CHUNKS;       // rows one wave moves per instruction
    constexpr int NI = kTile / (RPI * NW);
    auto ksw = [](int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); };
    auto vsw = [](int row) { return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); };
    // [K stage 0][K stage 1][V stage 0][V stage 1], kTile * D elements each (the launcher sizes it)
    extern __shared__ __attribute__((aligned(1024))) std::uint16_t tiles[];
    __shared__ float x_m[2][kBM], x_l[2][kBM];
    auto k_buf = [&](int stage) { return tiles + stage * (kTile * D); };
    auto v_buf = [&](int stage) { return tiles + (2 + stage) * (kTile * D); };

    const int nq = p.n_qblocks;
    const int per_bh = kMode == 3 ? (nq + 1) / 2 : nq;            // workgroups per (batch, head)
    // Workgroup w runs on XCD w % 8 (round-robin dispatch): with a head count that divides by 8, the
    // workgroups of one (batch, head) are numbered 8 apart, so that they share its K and V in one L2
    // instead of fetching them once per query block on eight different XCDs.
    int bh, slot_in_bh;
    if ((p.B * p.Hq) % 8 == 0) {
        const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
        bh = (j / per_bh) * 8 + xcd;
        slot_in_bh = j % per_bh;
    } else {
        bh = blockIdx.x / per_bh;
        slot_in_bh = blockIdx.x % per_bh;
    }
    const int b = bh / p.Hq, hq = bh % p.Hq;
    const int hkv = hq / (p.Hq / p.Hkv);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qw = wave & 3, kg = wave >> 2;
    const int lq = lane & 31, lh = lane >> 5;
    const std::uint16_t* kbase = p.k + b * p.ks_b + hkv * p.ks_h;
    const std::uint16_t* vbase = p.v + b * p.vs_b + hkv * p.vs_h;
    const int srow = wave * RPI + lane / CHUNKS, slot = lane % CHUNKS;
    const int grp = lane >> 4, m16 = lane & 15;
    int k_rd[KSTEPS], v_rd[DBLK];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) k_rd[ks] = (kg * kBN + lq) * D + (((2 * ks + lh) ^ ksw(lq)) * 8);
    {
        const int vrow = 4 * lh + (m16 >> 2);
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
            v_rd[db] = (kg * kBN + vrow) * D + (((4 * db + 2 * (grp & 1) + ((m16 & 3) >> 1)) ^ vsw(vrow)) * 8) + 4 * (m16 & 1);
    }
    // staging: 128 rows of K (and V), 16 bytes per thread and step, rows past Lk as zeros; the 16-byte
    // chunks of a row are XOR-swizzled so that operand reads and transposed reads are conflict free
    auto fetch = [&](const std::uint16_t* base, long row_stride, int first, u32x4 (&regs)[NI]) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int row = first + i * RPI * NW + srow;
            regs[i] = u32x4{0u, 0u, 0u, 0u};
            if (row < p.Lk) regs[i] = load16(base + static_cast<long>(row) * row_stride + slot * 8);
        }
    };
    auto put = [&](const u32x4 (&regs)[NI], std::uint16_t* tile, bool is_v) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int r = i * RPI * NW + srow;
            const int sw = is_v ? vsw(r) : ksw(r);
            *reinterpret_cast<u32x4*>(tile + r * D + ((slot ^ sw) * 8)) = regs[i];
        }
    };
    // Rounds to T and widens again.  For the intermediate roundings the conversion instructions serve:
    // they round like the host, and a NaN stays a NaN (its payload does not matter here, only the
    // final narrowing of a weight decides the bits that are written).
    auto round_T = [](float x) { return El::to_f32(El::from_f32_finite(x)); };
    const float scale_f = static_cast<float>(p.scale);

    // causal: the query block `slot_in_bh` from the end, then the same from the start
    const int n_parts = (kMode == 3 && slot_in_bh != nq - 1 - slot_in_bh) ? 2 : 1;
    for (int part = 0; part < n_parts; ++part) {
        const int qblock = kMode == 3 ? (part == 0 ? nq - 1 - slot_in_bh : slot_in_bh) : slot_in_bh;
        const int q0 = qblock * kBM + qw * 32;
        const int my_q = q0 + lq;
        const int qrow = my_q < p.Lq ? my_q : p.Lq - 1;

        i16x8 qreg[KSTEPS];
        {
            const std::uint16_t* qp = p.q + b * p.qs_b + hq * p.qs_h + static_cast<long>(qrow) * p.qs_l;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) qreg[ks] = *reinterpret_cast<const i16x8*>(qp + ks * 16 + lh * 8);
        }
        int n_tiles = (p.Lk + kTile - 1) / kTile;
        if (kMode == 3) {   // keys beyond the workgroup's last query carry zero weight: written as zeros below, not computed
            const int last_q = min(qblock * kBM + kBM, p.Lq) - 1;
            n_tiles = (min(last_q + 1, p.Lk) + kTile - 1) / kTile;
        }

        const unsigned char* mrow = nullptr;
        if constexpr (kMode == 1 || kMode == 2)
            mrow = p.mask + (static_cast<long>(b) * p.ms_b + static_cast<long>(hq) * p.ms_h + static_cast<long>(qrow) * p.ms_q) * (kMode == 1 ? 1 : 2);

        // Narrowed, scaled and masked scores of one 32-key block (block `jb` of this key group's half of
        // the staged tile, first key `key0`): accumulator register r of lane (query lq, half lh) is key
        // key0 + (r/4)*8 + 4*lh + r%4.  `edge`: the block reaches past the row's end or past the diagonal
        // (wave-uniform); only then the keys are tested one by one.
        auto scores = [&](const std::uint16_t* k_lds, int jb, int key0, float16_t& sc) {
            // A block that lies wholly inside a contiguous mask row: the lane asks for its half of its
            // query's 32 keys (16 lh .. + 15) as one 16-byte piece (two for an additive mask) before the
            // MFMAs, and the halves of a query swap every other run of four keys afterwards
            // (v_permlane32_swap: lanes l and l + 32), since half lh owns keys 8 g + 4 lh .. + 3.  Sixteen
            // element loads per block, each touching as many rows as there are queries in the wave, and
            // waited for on the spot, doubled the kernel's time with a mask.
            constexpr int MREGS = kMode == 1 ? 4 : (kMode == 2 ? 8 : 1);
            std::uint32_t mr[MREGS];
            const bool mask_whole = (kMode == 1 || kMode == 2) && p.ms_k == 1 && key0 + 32 <= p.Lk;     // wave-uniform
            if constexpr (kMode == 1 || kMode == 2) {
                if (mask_whole) {
                    typedef u32x4 u32x4_any __attribute__((aligned(1)));
                    constexpr int ES = kMode == 1 ? 1 : 2;
                    const unsigned char* at = mrow + static_cast<long>(key0 + 16 * lh) * ES;
#pragma unroll
                    for (int h = 0; h < ES; ++h) {
                        const u32x4 w = *reinterpret_cast<const u32x4_any*>(at + 16 * h);
#pragma unroll
                        for (int i = 0; i < 4; ++i) mr[4 * h + i] = w[i];
                    }
                }
            }
            // Any other block under a mask: its sixteen elements, asked for before the MFMAs as well (reads
            // past the row's end are clamped into it).
            std::uint32_t me[(kMode == 1 || kMode == 2) ? 16 : 1];
            if constexpr (kMode == 1 || kMode == 2) {
                if (!mask_whole) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = key0 + (r >> 2) * 8 + 4 * lh + (r & 3);
                        const long at = static_cast<long>(key < p.Lk ? key : p.Lk - 1) * p.ms_k;
                        if constexpr (kMode == 1) me[r] = mrow[at];
                        else                      me[r] = *reinterpret_cast<const std::uint16_t*>(mrow + 2 * at);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks)
                sc = Mma16<T>::run(*reinterpret_cast<const i16x8*>(&k_lds[jb * 32 * D + k_rd[ks]]), qreg[ks], sc);
            // T(T(q k^T) * scale).  The host multiplies in double; when the scale is a float the product
            // of it and a value of T is exact in double, so one fp32 multiply rounds to the same float.
            if (p.scale_is_f32) {
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[r] = round_T(round_T(sc[r]) * scale_f);
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sc[r] = round_T(static_cast<float>(static_cast<double>(round_T(sc[r])) * p.scale));
            }
            const bool edge = key0 + 32 > p.Lk || (kMode == 3 && key0 + 31 > q0);
            if constexpr (kMode == 1 || kMode == 2) {
                if (mask_whole) {
                    auto swap = [&](int x, int y) {       // upper half of register x <-> lower half of register y
                        const auto r2 = __builtin_amdgcn_permlane32_swap(mr[x], mr[y], false, false);
                        mr[x] = r2[0];
                        mr[y] = r2[1];
                    };
                    if constexpr (kMode == 1) {
                        swap(0, 1);
                        swap(2, 3);
                        constexpr int reg_of_run[4] = {0, 2, 1, 3};
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (((mr[reg_of_run[r >> 2]] >> (8 * (r & 3))) & 0xffu) == 0) sc[r] = -INFINITY;
                    } else {
                        swap(0, 2);
                        swap(1, 3);
                        swap(4, 6);
                        swap(5, 7);
                        constexpr int reg_of_run[4] = {0, 4, 2, 6};     // first register of each run's pair
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const std::uint16_t bits = static_cast<std::uint16_t>(mr[reg_of_run[r >> 2] + ((r & 3) >> 1)] >> (16 * (r & 1)));
                            sc[r] = round_T(sc[r] + El::to_f32(bits));        // T(s2 + mask)
                        }
                    }
                    return;
                }
            }
            if (kMode == 1 || kMode == 2 || edge) {
                // without a branch per element
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = key0 + (r >> 2) * 8 + 4 * lh + (r & 3);
                    float s = sc[r];
                    bool dead = key >= p.Lk;
                    if constexpr (kMode == 3) dead = dead || key > my_q;
                    if constexpr (kMode == 1) dead = dead || me[r] == 0;
                    if constexpr (kMode == 2) s = round_T(s + El::to_f32(static_cast<std::uint16_t>(me[r])));   // T(s2 + mask)
                    sc[r] = dead ? -INFINITY : s;
                }
            }
        };

        // ---- pass 1: row max and row sum of exp over the narrowed scores
        float m_run = -INFINITY, l_run = 0.f;
        u32x4 kreg[NI], vreg[NI];
        __syncthreads();                       // (second part: everyone is done with the buffers of the first)
        fetch(kbase, p.ks_l, 0, kreg);
        put(kreg, k_buf(0), false);
        __syncthreads();
        for (int t = 0; t < n_tiles; ++t) {
            const std::uint16_t* k_lds = k_buf(t & 1);
            if (t + 1 < n_tiles) fetch(kbase, p.ks_l, (t + 1) * kTile, kreg);   // in flight during this tile's work
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                const int key0 = t * kTile + kg * kBN + jb * 32;
                if (key0 >= p.Lk || (kMode == 3 && key0 > q0 + 31)) continue;   // wave-uniform
                float16_t sc;
                scores(k_lds, jb, key0, sc);
                float mx = sc[0];
#pragma unroll
                for (int r = 1; r < 16; ++r) mx = fmaxf(mx, sc[r]);
                const float m_new = fmaxf(m_run, mx);
                if (m_new != -INFINITY) {
                    // exp(s - m) as 2^(s log2(e) - m log2(e)): one fused multiply-add and the exponential
                    const float shift = -m_new * kLog2e;
                    float add = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) add += __builtin_amdgcn_exp2f(fmaf(sc[r], kLog2e, shift));
                    l_run = (m_run == -INFINITY ? 0.f : l_run * __builtin_amdgcn_exp2f(fmaf(m_run, kLog2e, shift))) + add;
                    m_run = m_new;
                }
            }
            // the other buffer was last read one tile ago, before the barrier that ended that tile
            if (t + 1 < n_tiles) put(kreg, k_buf((t + 1) & 1), false);
            __syncthreads();
        }
        {   // merge the two halves of each query, then the two key groups
            float m_lo, m_hi, l_lo, l_hi;
            halves(m_run, m_lo, m_hi);
            halves(l_run, l_lo, l_hi);
            auto merge = [](float ma, float la, float mb, float lb, float& m_out, float& l_out) {
                const float m_all = fmaxf(ma, mb);
                float l_all = 0.f;
                if (m_all != -INFINITY) {
                    if (ma != -INFINITY) l_all += la * __expf(ma - m_all);
                    if (mb != -INFINITY) l_all += lb * __expf(mb - m_all);
                }
                m_out = m_all;
                l_out = l_all;
            };
            merge(m_lo, l_lo, m_hi, l_hi, m_run, l_run);
            if (lh == 0) {
                x_m[kg][qw * 32 + lq] = m_run;
                x_l[kg][qw * 32 + lq] = l_run;
            }
            __syncthreads();
            // both groups combine in the same order (group 0 first), so they agree to the bit
            merge(x_m[0][qw * 32 + lq], x_l[0][qw * 32 + lq], x_m[1][qw * 32 + lq], x_l[1][qw * 32 + lq], m_run, l_run);
        }
        // A row without a visible key: max = -inf, every exp(-inf - -inf) is NaN, as in the reference's softmax.
        const float inv_l = 1.0f / l_run;
        const float w_shift = -m_run * kLog2e;

        // ---- pass 2: weights out, product with V
        float16_t oacc[DBLK];
#pragma unroll
        for (int i = 0; i < DBLK; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
        std::uint16_t* arow = p.attn + ((static_cast<long>(b) * p.Hq + hq) * p.Lq + qrow) * p.Lk;
        const bool row_live = my_q < p.Lq;
        const bool wide = (p.Lk % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.attn) & 7) == 0);   // 8-byte runs of four weights
        fetch(kbase, p.ks_l, 0, kreg);
        fetch(vbase, p.vs_l, 0, vreg);
        put(kreg, k_buf(0), false);            // (pass 1 ended with barriers: nobody reads stage 0 any more)
        put(vreg, v_buf(0), true);
        __syncthreads();
        for (int t = 0; t < n_tiles; ++t) {
            const std::uint16_t* k_lds = k_buf(t & 1);
            const std::uint16_t* v_lds = v_buf(t & 1);
            if (t + 1 < n_tiles) {
                fetch(kbase, p.ks_l, (t + 1) * kTile, kreg);
                fetch(vbase, p.vs_l, (t + 1) * kTile, vreg);
            }
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                const int key0 = t * kTile + kg * kBN + jb * 32;
                if (key0 >= p.Lk) continue;
                const bool skipped = kMode == 3 && key0 > q0 + 31;   // wave-uniform: this wave's queries see none of these keys
                float16_t sc;
                std::uint32_t pw[8];
                if (!skipped) {
                    scores(k_lds, jb, key0, sc);
                    // The weights are narrowed by the conversion instructions; a NaN among them (a row
                    // without a visible key, a NaN or an infinity in the inputs) shows in their sum, and
                    // then the block is narrowed again the way the host writes NaNs.
                    float w[16], total = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        w[r] = __builtin_amdgcn_exp2f(fmaf(sc[r], kLog2e, w_shift)) * inv_l;
                        total += w[r];
                    }
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        pw[i] = static_cast<std::uint32_t>(El::from_f32_finite(w[2 * i])) | (static_cast<std::uint32_t>(El::from_f32_finite(w[2 * i + 1])) << 16);
                    if (__builtin_amdgcn_ballot_w64(!(total == total)) != 0) {
                        asm volatile("" ::: "memory");
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            pw[i] = static_cast<std::uint32_t>(El::from_f32(w[2 * i])) | (static_cast<std::uint32_t>(El::from_f32(w[2 * i + 1])) << 16);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) pw[i] = 0u;
                }
                if (row_live) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int key = key0 + g * 8 + 4 * lh;
                        if (wide && key + 3 < p.Lk) {
                            // (a plain store on purpose: as a non-temporal one each of these 8-byte pieces goes to memory on its
                            // own instead of being merged into whole lines in L2 -- 597 MB written instead of 306, 615 us instead of 170)
                            *reinterpret_cast<u32x2*>(arow + key) = u32x2{pw[2 * g], pw[2 * g + 1]};
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (key + e < p.Lk) arow[key + e] = static_cast<std::uint16_t>(pw[2 * g + (e >> 1)] >> (16 * (e & 1)));
                        }
                    }
                }
                if (!skipped) {
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const u32x4 pv = {pw[4 * s2], pw[4 * s2 + 1], pw[4 * s2 + 2], pw[4 * s2 + 3]};
#pragma unroll
                        for (int db = 0; db < DBLK; ++db) {
                            const std::uint16_t* vp = v_lds + jb * 32 * D + v_rd[db] + 16 * s2 * D;
                            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp));
                            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp + 8 * D));
                            const i16x8 vf = i16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                            oacc[db] = Mma16<T>::run(vf, __builtin_bit_cast(i16x8, pv), oacc[db]);
                        }
                    }
                }
            }
            if (t + 1 < n_tiles) {
                put(kreg, k_buf((t + 1) & 1), false);
                put(vreg, v_buf((t + 1) & 1), true);
            }
            __syncthreads();
        }
        // causal: the keys past the workgroup's last query were never visited; their weights are zero.
        // The two waves of a query group clear that part of alternate rows, a row at a time with
        // 16-byte stores where the row starts allow it.
        if (kMode == 3 && n_tiles * kTile < p.Lk) {
            const int first = n_tiles * kTile;
            const bool rows16 = (p.Lk % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.attn) & 15) == 0);
            for (int rr = kg; rr < 32; rr += 2) {
                const int row = q0 + rr;
                if (row >= p.Lq) break;
                std::uint16_t* zr = p.attn + ((static_cast<long>(b) * p.Hq + hq) * p.Lq + row) * p.Lk;
                if (rows16) {
                    for (int key = first + lane * 8; key < p.Lk; key += 64 * 8) store16(zr + key, u32x4{0u, 0u, 0u, 0u});
                } else {
                    for (int key = first + lane; key < p.Lk; key += 64) zr[key] = 0;
                }
            }
        }

        // The two key groups' partial products add up: group 1 hands its over through LDS (the tile
        // buffers are free after the last tile's barrier), element (db, r) of lane l of query group qw
        // at [(db*16 + r)][qw*64 + l].
        float* xo = reinterpret_cast<float*>(tiles);
        if (kg == 1) {
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) xo[(db * 16 + r) * 256 + qw * 64 + lane] = oacc[db][r];
        }
        __syncthreads();
        if (kg == 0) {
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] += xo[(db * 16 + r) * 256 + qw * 64 + lane];
            if (row_live) {
                std::uint16_t* op = p.out + ((static_cast<long>(b) * p.Hq + hq) * p.Lq + my_q) * D;
#pragma unroll
                for (int db = 0; db < DBLK; ++db)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d = db * 32 + g * 8 + 4 * lh;
                        u32x2 w;
                        w[0] = static_cast<std::uint32_t>(El::from_f32(oacc[db][4 * g + 0])) | (static_cast<std::uint32_t>(El::from_f32(oacc[db][4 * g + 1])) << 16);
                        w[1] = static_cast<std::uint32_t>(El::from_f32(oacc[db][4 * g + 2])) | (static_cast<std::uint32_t>(El::from_f32(oacc[db][4 * g + 3])) << 16);
                        *reinterpret_cast<u32x2*>(op + d) = w;
                    }
                if (p.lse != nullptr && lh == 0)
                    p.lse[(static_cast<long>(b) * p.Hq + hq) * p.Lq + my_q] = m_run + logf(l_run);
            }
        }
    }   // part
}

template <typename T, int D>
int launch_t(WeightsParams p, int mode, hipStream_t s) {
    p.n_qblocks = (p.Lq + kBM - 1) / kBM;
    const long per_bh = mode == 3 ? (p.n_qblocks + 1) / 2 : p.n_qblocks;      // causal: query blocks in pairs
    const long blocks = static_cast<long>(p.B) * p.Hq * per_bh;
    const dim3 grid(static_cast<unsigned>(blocks)), wg(512);
    constexpr unsigned kLdsBytes = 4u * kTile * D * 2u;     // K and V, two stages each
    // More than 64 KB of LDS has to be asked for by name, once per kernel and device.
    auto allow = [&](const void* fn) {
        static std::mutex mu;
        static std::set<std::pair<int, const void*>> done;
        int dev = 0;
        if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
        std::lock_guard<std::mutex> g(mu);
        if (done.count({dev, fn})) return hipSuccess;
        const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes));
        if (e == hipSuccess) done.insert({dev, fn});
        return e;
    };
    switch (mode) {
        case 0:
            PARAS_HIP_TRY(allow(reinterpret_cast<const void*>(&weights_fwd_kernel<T, D, 0>)));
            hipLaunchKernelGGL((weights_fwd_kernel<T, D, 0>), grid, wg, kLdsBytes, s, p);
            break;
        case 1:
            PARAS_HIP_TRY(allow(reinterpret_cast<const void*>(&weights_fwd_kernel<T, D, 1>)));
            hipLaunchKernelGGL((weights_fwd_kernel<T, D, 1>), grid, wg, kLdsBytes, s, p);
            break;
        case 2:
            PARAS_HIP_TRY(allow(reinterpret_cast<const void*>(&weights_fwd_kernel<T, D, 2>)));
            hipLaunchKernelGGL((weights_fwd_kernel<T, D, 2>), grid, wg, kLdsBytes, s, p);
            break;
        default:
            PARAS_HIP_TRY(allow(reinterpret_cast<const void*>(&weights_fwd_kernel<T, D, 3>)));
            hipLaunchKernelGGL((weights_fwd_kernel<T, D, 3>), grid, wg, kLdsBytes, s, p);
            break;
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool mult8(const int64_t* strides) { return strides[0] % 8 == 0 && strides[1] % 8 == 0 && strides[2] % 8 == 0; }

}  // namespace

bool weights_supported(const paras_sdpa_args& a) {
    if (a.dtype != PARAS_BF16 && a.dtype != PARAS_F16) return false;
    if (a.attn == nullptr) return false;                            // without the weights the flash kernels are the path
    if (a.D != a.Dv || (a.D != 64 && a.D != 128)) return false;
    if (a.mask_kind != 0 && (a.mask == nullptr || a.is_causal)) return false;
    if (a.mask_kind < 0 || a.mask_kind > 2) return false;
    if (a.mask_kind != 0 && a.mask_strides[3] < 0) return false;
    if (a.Lq < 1 || a.Lk < 1) return false;
    if (!std::isfinite(a.scale)) return false;
    if (!aligned16(a.q) || !aligned16(a.k) || !aligned16(a.v) || (reinterpret_cast<uintptr_t>(a.out) & 7) != 0) return false;
    if (!mult8(a.q_strides) || !mult8(a.k_strides) || !mult8(a.v_strides)) return false;
    const int64_t nq = (a.Lq + kBM - 1) / kBM;
    if (a.B * a.Hq * nq > 0x7fffffffLL || a.Lq > 0x3fffffff || a.Lk > 0x3fffffff) return false;
    return true;
}

int launch_weights(const paras_sdpa_args& a, hipStream_t s) {
    WeightsParams p;
    p.q = static_cast<const std::uint16_t*>(a.q);
    p.k = static_cast<const std::uint16_t*>(a.k);
    p.v = static_cast<const std::uint16_t*>(a.v);
    p.out = static_cast<std::uint16_t*>(a.out);
    p.attn = static_cast<std::uint16_t*>(a.attn);
    p.lse = a.lse;
    p.qs_b = a.q_strides[0]; p.qs_h = a.q_strides[1]; p.qs_l = a.q_strides[2];
    p.ks_b = a.k_strides[0]; p.ks_h = a.k_strides[1]; p.ks_l = a.k_strides[2];
    p.vs_b = a.v_strides[0]; p.vs_h = a.v_strides[1]; p.vs_l = a.v_strides[2];
    p.B = static_cast<int>(a.B); p.Hq = static_cast<int>(a.Hq); p.Hkv = static_cast<int>(a.Hkv);
    p.Lq = static_cast<int>(a.Lq); p.Lk = static_cast<int>(a.Lk);
    p.n_qblocks = 0;
    p.scale = a.scale;
    p.scale_is_f32 = static_cast<double>(static_cast<float>(a.scale)) == a.scale ? 1 : 0;
    p.mask = static_cast<const unsigned char*>(a.mask);
    p.ms_b = a.mask_strides[0]; p.ms_h = a.mask_strides[1]; p.ms_q = a.mask_strides[2]; p.ms_k = a.mask_strides[3];
    const int mode = a.is_causal ? 3 : a.mask_kind;
    if (a.dtype == PARAS_BF16)
        return a.D == 128 ? launch_t<bf16_t, 128>(p, mode, s) : launch_t<bf16_t, 64>(p, mode, s);
    return a.D == 128 ? launch_t<f16_t, 128>(p, mode, s) : launch_t<f16_t, 64>(p, mode, s);
}

}  // namespace paras
