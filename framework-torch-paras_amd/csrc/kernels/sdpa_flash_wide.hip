// Flash-attention forward for gfx950, head size 128, 64 queries per wavefront.
//
// Same mathematics and the same lane layout as sdpa_flash.hip (S^T = K Q^T and
// O^T = V^T P^T on v_mfma_f32_32x32x16, a lane owns one query column, online
// softmax with a lazily raised reference point; the reference materialises the
// scores instead: csrc/ops/attention_ops.cpp:101,128).  What differs is the shape
// of a wavefront's work:
//
//   The LDS delivers 128 bytes per clock per CU, and a 32x32x16 MFMA whose K or V
//   operand comes from LDS needs 1 KB of it: four SIMDs issuing one MFMA every 32
//   clocks ask for exactly the LDS's peak.  With 32 queries per wavefront the
//   operand reads are the bound.  Here a wavefront owns TWO 32-query blocks, so
//   every K / V fragment read from LDS feeds two MFMAs, and a workgroup of four
//   wavefronts covers 256 queries, so a staged tile is shared by twice the
//   queries as well.
//
//   64 queries x 128 columns of fp32 output are 128 registers per lane, the query
//   fragments another 64: the kernel runs one wavefront per SIMD with the 512
//   registers of the unified file.  Outputs and queries live in the accumulation
//   half (AGPRs), which only the MFMAs touch; scores, probabilities and operand
//   fragments live in VGPRs.  The compiler does not make that split by itself (it
//   keeps copying between the halves), so the MFMAs of this kernel are inline
//   assembly with the register file of each operand spelled out.  What the
//   compiler cannot see inside them is covered by hand: a VALU read of an MFMA
//   result is kept at least a dozen MFMAs behind it by the schedule, or behind
//   explicit s_nop where it is not (first scores, rescale branch, epilogue).
//
// With nothing else on the SIMD to fill a stall, the schedule inside a block (32
// keys x 64 queries = 32 MFMAs) is flat: one MFMA, then a few VALU instructions
// of the softmax of the block before, then the next MFMA,
//
//   u = 0..15   S(j+1) = K(j+1) Q^T   (k-step u/2, query block u%2)
//   u = 16..31  O^T += V(j)^T P(j)^T  ((query block, key half) = (0,0) (1,0) (0,1) (1,1), four column blocks each)
//   the 16 exp pairs of S(j) sit before MFMA 7e/4, each ahead of the first PV MFMA that needs it;
//   the row maxima of S(j+1) are reduced in u = 27..30
//
// and every operand is requested from LDS at least eight MFMAs before its use:
// the V fragments of block j during its score MFMAs, the K fragments of block
// j+1's score MFMAs (keys of block j+2) during block j's PV MFMAs.  Those keys
// belong to the next K tile, so during tile t a wavefront reads K tile t+1 and V
// tile t while K tile t+2 and V tile t+1 stream in: two buffers each, one
// barrier per tile, and no operand request ever waits for a barrier.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_flash_common.h"

namespace paras {
namespace flash {
namespace {

constexpr int D      = 128;
constexpr int QB     = 2;            // 32-query blocks per wavefront
constexpr int NW     = 4;
constexpr int WQ     = 32 * QB;
constexpr int KSTEPS = D / 16;       // 8
constexpr int DBLK   = D / 32;       // 4
constexpr int CHUNKS = D / 8;        // 16-byte chunks per row
constexpr int RPI    = 64 / CHUNKS;  // rows one wavefront stages per instruction
constexpr int NI     = kBN / (RPI * NW);
static_assert(kWideBM == NW * WQ, "workgroup shape");

// f(integral_constant<int, I>) for I = 0 .. N-1: loop indices the front end sees as constants.
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

template <typename T, bool kCausal>
__global__ __launch_bounds__(256, 1) void flash_wide_kernel(const FlashParams p) {
    auto ksw = [](int row) { return row & 15; };
    auto vsw = [](int row) { return (row & 3) << 2; };

    // Four separate arrays: an LDS read waits for every direct-to-LDS load in flight unless the
    // variables involved prove them disjoint, so the main loop names its buffers at compile time.
    __shared__ __attribute__((aligned(1024))) std::uint16_t k_lds0[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t k_lds1[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t v_lds0[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t v_lds1[kBN * D];
    // A wavefront's 64 x 128 outputs pass through LDS on their way out (16 KB each, its own region:
    // no barrier), so that the global stores write whole rows.
    constexpr int OROW = D + 8;   // row pitch of that region in elements: 16 bytes of padding spread the rows over the banks
    __shared__ __attribute__((aligned(1024))) std::uint16_t o_lds[kWideBM * OROW];
    using Yes = std::true_type;
    using No  = std::false_type;
    using Par0 = std::integral_constant<int, 0>;
    using Par1 = std::integral_constant<int, 1>;
    struct AnyPar { int value; };
    auto kbuf = [&](auto par, bool flip) -> std::uint16_t* {
        if constexpr (std::is_same<decltype(par), AnyPar>::value) return ((par.value ^ (flip ? 1 : 0)) & 1) ? k_lds1 : k_lds0;
        else return (decltype(par)::value != 0) != flip ? k_lds1 : k_lds0;
    };
    auto vbuf = [&](auto par, bool flip) -> std::uint16_t* {
        if constexpr (std::is_same<decltype(par), AnyPar>::value) return ((par.value ^ (flip ? 1 : 0)) & 1) ? v_lds1 : v_lds0;
        else return (decltype(par)::value != 0) != flip ? v_lds1 : v_lds0;
    };

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    // ---- work items.  The grid is one workgroup per CU and every workgroup walks a list of
    // (batch * head, query tile) items of its own: a new workgroup could only start once the one
    // before it had drained (64 KB of LDS and all 512 registers allow one per CU), which left the
    // CU idle for 11 us per item -- launch, first loads, first scores.  Walking the list inside
    // the kernel, the loads of the next item are in flight while the outputs of this one are
    // normalised and stored.
    //   Workgroup w runs on XCD w % 8 (round-robin dispatch), so with a head count that divides
    // by 8 the heads are dealt to the XCDs and the workgroups of an XCD share the K / V of few
    // heads at a time in its L2.  Within such a pool the items are numbered head by head, longest
    // query tile first under the causal rule, and dealt in rounds of one item per workgroup, every
    // other round in reverse order, which evens out the triangle (tile i then tile n-1-i).
    const int nq = p.n_qblocks;
    const int BH = p.B * p.Hq;
    const int n_wg = static_cast<int>(gridDim.x), wg_id = static_cast<int>(blockIdx.x);
    const bool by_xcd = BH % 8 == 0 && n_wg % 8 == 0;
    const int pool_wgs = by_xcd ? n_wg >> 3 : n_wg;
    const int pool_pos = by_xcd ? wg_id >> 3 : wg_id;
    const int pool_items = (by_xcd ? BH >> 3 : BH) * nq;
    // (x / d as a multiply-high by ceil(2^32 / d): exact while x * d < 2^32, which the launcher checks)
    auto fast_div = [](int x, unsigned magic) { return static_cast<int>(__umulhi(static_cast<unsigned>(x), magic)); };
    auto item_at = [&](int round, int& bh, int& qblock) {
        const int i = round * pool_wgs + ((round & 1) ? pool_wgs - 1 - pool_pos : pool_pos);
        if (i >= pool_items) return false;
        const int head = nq == 1 ? i : fast_div(i, p.magic_nq), pos = i - head * nq;
        bh = by_xcd ? head * 8 + (wg_id & 7) : head;
        qblock = kCausal ? nq - 1 - pos : pos;
        return true;
    };

    // ---- the item at hand
    int b, hq, q0, n_tiles, wave_tiles, first_masked[QB];
    __amdgpu_buffer_rsrc_t k_rsrc, v_rsrc;
    i16x8 qreg[QB][KSTEPS];
    const int k_row_bytes = static_cast<int>(p.ks_l) * 2, v_row_bytes = static_cast<int>(p.vs_l) * 2;
    auto make_rsrc = [&](const std::uint16_t* base, int row_bytes) {
        const int bytes = (p.Lk - 1) * row_bytes + D * 2;           // < 2^31: checked by flash_supported
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<std::uint16_t*>(base), 0, bytes, 0x00020000);
    };
    auto load_queries = [&]() {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const int my_q = q0 + 32 * qb + lq;
            const int qrow = my_q < p.Lq ? my_q : p.Lq - 1;
            const std::uint16_t* qp = p.q + b * p.qs_b + hq * p.qs_h + static_cast<long>(qrow) * p.qs_l;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) qreg[qb][ks] = *reinterpret_cast<const i16x8*>(qp + ks * 16 + lh * 8);
        }
    };
    // Everything that depends on the item.
    auto enter_item = [&](int bh, int qblock) {
        b = p.Hq == 1 ? bh : fast_div(bh, p.magic_hq);
        hq = bh - b * p.Hq;
        const int hkv = p.Hq == p.Hkv ? hq : fast_div(hq, p.magic_rep);
        q0 = qblock * kWideBM + wave * WQ;   // query block qb of this wavefront starts at q0 + 32 qb
        k_rsrc = make_rsrc(p.k + b * p.ks_b + hkv * p.ks_h, k_row_bytes);
        v_rsrc = make_rsrc(p.v + b * p.vs_b + hkv * p.vs_h, v_row_bytes);
        n_tiles = (p.Lk + kBN - 1) / kBN;
        if (kCausal) {
            const int last_q = min(qblock * kWideBM + kWideBM, p.Lq) - 1;
            n_tiles = (min(last_q + 1, p.Lk) + kBN - 1) / kBN;
        }
        wave_tiles = kCausal ? min(n_tiles, (q0 + WQ - 1) / kBN + 1) : n_tiles;
        // Block j of query block qb needs masking from its diagonal block on (j * 32 + 31 > first
        // query) and where it reaches past the end of K (j * 32 + 32 > Lk): j >= first_masked[qb].
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) first_masked[qb] = kCausal ? min((q0 + 32 * qb) >> 5, p.Lk >> 5) : (p.Lk >> 5);
    };

    // ---- staging: global rows straight into LDS with buffer loads; the descriptor spans rows
    // [0, Lk) of this (batch, kv head), so rows past the end arrive as zeros without a branch.
    const int srow = wave * RPI + lane / CHUNKS;
    const int slot = lane % CHUNKS;
    const int k_lane = srow * k_row_bytes + ((slot ^ ksw(srow)) * 16);
    const int v_lane = srow * v_row_bytes + ((slot ^ vsw(srow)) * 16);
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto stage_one = [&](__amdgpu_buffer_rsrc_t rsrc, int lane_off, int row_bytes, int first, std::uint16_t* tile, int i) {
        const int r0 = i * RPI * NW;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lptr_t)(tile + (r0 + wave * RPI) * D), 16,
                                                 lane_off + (first + r0) * row_bytes, 0, 0, 0);
    };
    auto stage_rows = [&](__amdgpu_buffer_rsrc_t rsrc, int lane_off, int row_bytes, int first, std::uint16_t* tile) {
#pragma unroll
        for (int i = 0; i < NI; ++i) stage_one(rsrc, lane_off, row_bytes, first, tile, i);
    };
    // What tile t's successor needs beyond what tile t already reads: K tile t+2 (into the buffer
    // of K tile t, which nobody reads any more) and V tile t+1.
    auto stage_pair = [&](int t, auto par) {
        stage_rows(k_rsrc, k_lane, k_row_bytes, (t + 2) * kBN, kbuf(par, false));
        stage_rows(v_rsrc, v_lane, v_row_bytes, (t + 1) * kBN, vbuf(par, true));
    };
    auto publish = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's part of the tiles has landed
        __syncthreads();
    };

    float16_t oacc[QB][DBLK];
    float m_run[QB], l_run[QB];
    // The first tiles of an item: K tiles 0 and 1, V tile 0 (the loop stages the rest).
    auto stage_first = [&]() {
        stage_rows(k_rsrc, k_lane, k_row_bytes, 0, k_lds0);
        stage_rows(k_rsrc, k_lane, k_row_bytes, kBN, k_lds1);
        stage_rows(v_rsrc, v_lane, v_row_bytes, 0, v_lds0);
    };

    const int grp = lane >> 4, m16 = lane & 15;
    int k_rd[KSTEPS], v_rd[DBLK];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) k_rd[ks] = lq * D + (((2 * ks + lh) ^ ksw(lq)) * 8);
    {
        const int vrow = 4 * lh + (m16 >> 2);
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
            v_rd[db] = vrow * D + (((4 * db + 2 * (grp & 1) + ((m16 & 3) >> 1)) ^ vsw(vrow)) * 8) + 4 * (m16 & 1);
    }
    const float lazy_margin = 8.0f / p.scale_log2;

    auto needs_mask = [&](int j, int qb) { return j >= first_masked[qb]; };
    auto apply_mask = [&](int j, int qb, float16_t& sc) {
        const int my_q = q0 + 32 * qb + lq;
        const int last_visible = kCausal ? min(my_q, p.Lk - 1) : p.Lk - 1;
        const int rel = last_visible - j * 32 - 4 * lh;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if ((r >> 2) * 8 + (r & 3) > rel) sc[r] = -INFINITY;
    };
    auto lane_max = [](const float16_t& sc) {
        float mx = sc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(mx, sc[r]);
        return mx;
    };
    // Raise the running maxima where a block max (this lane's half of the keys) asks for it; the
    // two halves of a query only meet inside this rarely taken branch.
    // (the compare builtin hands back the wavefront's lane mask as it stands: a bool fed to the
    // ballot builtin is first turned into 0 / 1 per lane and compared again)
    float raise_at[QB];      // m_run + lazy_margin, kept beside m_run
    auto wants_raise = [&](const float (&mx)[QB]) {
        unsigned long long grow = 0;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) grow |= __builtin_amdgcn_fcmpf(mx[qb], raise_at[qb], 2 /* ordered greater than */);
        return grow != 0;   // wave-uniform, rare after block 0
    };
    auto raise_max = [&](const float (&mx)[QB]) {
        // (pins the outputs in AGPRs up to here: without it their 128 copies to VGPRs are
        // hoisted out of this branch into every block)
        asm volatile("" : "+a"(oacc[0][0]), "+a"(oacc[0][1]), "+a"(oacc[0][2]), "+a"(oacc[0][3]),
                          "+a"(oacc[1][0]), "+a"(oacc[1][1]), "+a"(oacc[1][2]), "+a"(oacc[1][3]));
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float m_new = fmaxf(m_run[qb], half_swap_max(mx[qb]));
            // (equal covers -inf on both sides: a query that has seen no key yet keeps its zeros)
            const float alpha = m_run[qb] == m_new ? 1.f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * p.scale_log2);
            m_run[qb] = m_new;
            raise_at[qb] = m_new + lazy_margin;
            l_run[qb] *= alpha;
#pragma unroll
            for (int i = 0; i < DBLK; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[qb][i][r] *= alpha;
        }
        asm volatile("" : "+a"(oacc[0][0]), "+a"(oacc[0][1]), "+a"(oacc[0][2]), "+a"(oacc[0][3]),
                          "+a"(oacc[1][0]), "+a"(oacc[1][1]), "+a"(oacc[1][2]), "+a"(oacc[1][3]));
    };
    // Scores of block j are complete in `sc`, their in-lane maxima in `mx`, and `raise` says whether
    // those maxima ask for a higher reference point.  Blocks on the diagonal or at the end of K are
    // masked first and their maxima taken again.
    auto finish_scores = [&](int j, float16_t (&sc)[QB], float (&mx)[QB], bool raise) {
        const bool masked = needs_mask(j, 0);        // first_masked[0] <= first_masked[1]: one test covers both
        // One test on the common path, which falls through: both cases are rare and wave-uniform.
        if (__builtin_expect(masked | raise, 0)) {
            if (masked) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    if (needs_mask(j, qb)) {
                        apply_mask(j, qb, sc[qb]);
                        mx[qb] = lane_max(sc[qb]);
                    }
                }
                raise = wants_raise(mx);
            }
            if (raise) raise_max(mx);
        }
    };

    // Operand fragments: kf = the K rows of the block whose scores come next, vf = the V rows of
    // the block whose probabilities are applied now.
    i16x8 kf[KSTEPS], vf[2 * DBLK];
    auto fetch_k = [&](const std::uint16_t* rows, int ks) { kf[ks] = *reinterpret_cast<const i16x8*>(rows + k_rd[ks]); };
    auto fetch_v = [&](const std::uint16_t* rows, int f) {     // f = 4 * (16-key half) + column block
        const std::uint16_t* vp = rows + v_rd[f % DBLK] + 16 * (f / DBLK) * D;
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp + 8 * D));
        vf[f] = i16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    // One block j of 32 keys: exponentials of `cur` = S(j), PV(j) and the score MFMAs of S(j+1)
    // into `nxt`.  `par` is the parity of block j's tile: V(j) lives in the V buffer of that
    // parity, the keys of block j+2 (requested here for block j+1's score MFMAs) in the K buffer
    // of the other one.  On entry kf holds the keys of block j+1.
    //
    // The softmax of S(j) is a list of 128 VALU instructions, dealt four to each of the 32 MFMAs
    // so that neither pipe waits for the other: the 16 exp pairs two at a time (the four fma, the
    // four exp, cvt and add of both, the two sum updates: 14 instructions, no exponential next to
    // its producer or its consumer, so no hazard nop), in
    // the order the PV MFMAs need them -- pair e is finished before MFMA 7(e|1)/4 + 4, ahead of
    // MFMA 16 / 20 / 24 / 28 for the four (query block, key half) groups -- then the 16
    // instructions of the row maxima of S(j+1) under the last four MFMAs.
    auto block = [&](int j, float16_t (&cur)[QB], float16_t (&nxt)[QB], auto par, auto stage_tag) {
        constexpr bool kStage = decltype(stage_tag)::value;
        const std::uint16_t* vrows = vbuf(par, false) + (j & 1) * 32 * D;
        const std::uint16_t* krows = kbuf(par, true) + (j & 1) * 32 * D;
        float mc[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) mc[qb] = m_run[qb] * p.scale_log2;
        u32x4 pw[QB][2];
        float mx[QB], t3[QB][7], ex[16][2], sm[16];
        bool raise = false;
        // v_max3_f32 as written (fmaxf would canonicalise operands that come out of inline assembly)
        auto max3 = [](float a, float b, float c) {
            float r;
            asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
            return r;
        };
        // Instruction o of the list, and (separately, one instruction later: an inline-assembly
        // operand written by the instruction just before costs a hazard nop) the empty asm that
        // pins its result, i.e. keeps the instruction in its slot.
        auto valu_op = [&](auto O, auto PinOnly) {
            constexpr int o = decltype(O)::value;
            constexpr bool pin = decltype(PinOnly)::value;
            if constexpr (o < 0 || o >= 128) {
            } else if constexpr (o < 112) {
                constexpr int k = o / 14, r = o % 14;
                // r: 0-3 fma (a0 a1 b0 b1), 4-7 exp (a0 a1 b0 b1), 8 cvt a, 9 add a, 10 cvt b, 11 add b, 12 sum a, 13 sum b
                constexpr int e = 2 * k + (r < 8 ? ((r & 3) >> 1) : (r < 12 ? ((r - 8) >> 1) : r - 12));   // exp pair 0..15
                constexpr int qb = (e >> 2) & 1, i = (e & 3) + 4 * (e >> 3);       // elements 2i, 2i+1 of cur[qb]
                constexpr int w = r < 8 ? (r & 1) + 2 * (r >> 2) : (r < 12 ? (r & 1) : 2);   // <8: 0,1 fma 2,3 exp; else 0 cvt 1 add 2 sum
                if constexpr (r < 8) {
                    if constexpr (pin) asm volatile("" :: "v"(ex[e][w & 1]));
                    else if constexpr (w < 2) ex[e][w] = fmaf(cur[qb][2 * i + w], p.scale_log2, -mc[qb]);
                    else ex[e][w - 2] = __builtin_amdgcn_exp2f(ex[e][w - 2]);
                } else if constexpr (w == 0) {
                    if constexpr (pin) asm volatile("" :: "v"(pw[qb][i / 4][i % 4]));
                    else pw[qb][i / 4][i % 4] = Mma<T>::pack2(ex[e][0], ex[e][1]);
                } else if constexpr (w == 1) {
                    if constexpr (pin) asm volatile("" :: "v"(sm[e]));
                    else sm[e] = ex[e][0] + ex[e][1];
                } else {
                    if constexpr (pin) asm volatile("" :: "v"(l_run[qb]));
                    else l_run[qb] += sm[e];
                }
            } else {
                constexpr int qb = (o - 112) / 8, r = (o - 112) % 8;
                const float16_t& sv = nxt[qb];
                if constexpr (pin) {
                    if constexpr (r < 7) asm volatile("" :: "v"(t3[qb][r]));
                    else                 asm volatile("" :: "v"(mx[qb]));
                } else if constexpr (r < 5)  t3[qb][r] = max3(sv[3 * r], sv[3 * r + 1], sv[3 * r + 2]);
                else if constexpr (r == 5)   t3[qb][5] = max3(t3[qb][0], t3[qb][1], t3[qb][2]);
                else if constexpr (r == 6)   t3[qb][6] = max3(t3[qb][3], t3[qb][4], sv[15]);
                else                         mx[qb] = fmaxf(t3[qb][5], t3[qb][6]);
            }
        };
        static_for<32>([&](auto U) {
            constexpr int u = decltype(U)::value;
            static_for<4>([&](auto I) {
                constexpr int o = 4 * u + decltype(I)::value;
                valu_op(std::integral_constant<int, o>{}, No{});
                valu_op(std::integral_constant<int, o - 1>{}, Yes{});
            });
            if constexpr (u == 31) valu_op(std::integral_constant<int, 127>{}, Yes{});
            if constexpr (u == 31) raise = wants_raise(mx);          // decided under the last MFMA, acted on after it
            // Two waits per block instead of one per MFMA (an instruction of any kind costs this
            // lone wavefront an issue slot): every request waited for here is eight MFMAs old.
            if constexpr (u == 0 || u == 16) __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
            if constexpr (u < 16) {
                constexpr int c = u >> 1, qb = u & 1;
                if constexpr (c == 0) Mma<T>::score_first(nxt[qb], kf[0], qreg[qb][0]);
                else                  Mma<T>::score_acc(nxt[qb], kf[c], qreg[qb][c]);
                if constexpr (u < 2 * DBLK) fetch_v(vrows, u);
            } else {
                constexpr int g = (u - 16) >> 2, qb = g & 1, s2 = g >> 1, db = (u - 16) & 3;
                oacc[qb][db] = Mma<T>::run(vf[s2 * DBLK + db], __builtin_bit_cast(i16x8, pw[qb][s2]), oacc[qb][db]);
                // The next block's K fragments, under the first eight output MFMAs: the wait in front of
                // the next block's first score MFMA then finds them eight MFMAs old as well (under the last
                // eight, the youngest was requested one MFMA before that wait).  No more registers: all of
                // V's fragments are live here either way, as K's and V's are during the score MFMAs.
                if constexpr (u < 16 + KSTEPS) fetch_k(krows, u - 16);
            }
            if constexpr (kStage && u % 2 == 1 && u / 2 < 2 * NI) {
                // the next tile pair (K tile t+2, V tile t+1), one request every other MFMA of the tile's
                // first sixteen: the wait at the end of the tile then finds them all at least 48 MFMAs old
                // (every fourth MFMA, the last one 34 MFMAs old: 1 % slower)
                constexpr int i = u / 2;
                const int t = j >> 1;
                if constexpr (i < NI) stage_one(k_rsrc, k_lane, k_row_bytes, (t + 2) * kBN, kbuf(par, false), i);
                else                  stage_one(v_rsrc, v_lane, v_row_bytes, (t + 1) * kBN, vbuf(par, true), i - NI);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        finish_scores(j + 1, nxt, mx, raise);
    };
    // Outputs of the item at hand: out = O / l, and the log-sum-exp if asked for.  A lane holds
    // four consecutive columns of its query per accumulator group, i.e. 8-byte pieces of 32
    // different rows per store: they are written to LDS instead (rows padded by 16 bytes, so one
    // address register and immediate offsets do) and read back a row at a time, 16 bytes per
    // lane, four rows per store instruction.
    auto outputs_to_lds = [&](int ob, int ohq, int oq0) {
        std::uint16_t* mine = o_lds + wave * WQ * OROW;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float l_tot = half_swap_sum(l_run[qb]);
            const float inv_l = 1.0f / l_tot;
            const int row = 32 * qb + lq;
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = Mma<T>::pack2(oacc[qb][db][4 * g + 0] * inv_l, oacc[qb][db][4 * g + 1] * inv_l);
                    w[1] = Mma<T>::pack2(oacc[qb][db][4 * g + 2] * inv_l, oacc[qb][db][4 * g + 3] * inv_l);
                    *reinterpret_cast<u32x2*>(mine + row * OROW + (4 * db + g) * 8 + 4 * lh) = w;
                }
            const int my_q = oq0 + row;
            if (p.lse != nullptr && lh == 0 && my_q < p.Lq)
                p.lse[(static_cast<long>(ob) * p.Hq + ohq) * p.Lq + my_q] = m_run[qb] * p.scale + logf(l_tot);
        }
    };
    auto outputs_to_memory = [&](int ob, int ohq, int oq0) {
        const std::uint16_t* mine = o_lds + wave * WQ * OROW;
        std::uint16_t* orow = p.out + ((static_cast<long>(ob) * p.Hq + ohq) * p.Lq + oq0) * D;
        const int chunk = lane & 15, sub = lane >> 4;
        if (oq0 + WQ <= p.Lq) {
            // all of the wavefront's rows exist (wave-uniform): eight reads in flight, then their stores
            // (a test per row makes sixteen branches, each a read, a wait and a store: 1 % of the kernel)
#pragma unroll
            for (int h = 0; h < WQ / 32; ++h) {
                u32x4 v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const u32x4*>(mine + (32 * h + 4 * i + sub) * OROW + chunk * 8);
#pragma unroll
                for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(orow + (32 * h + 4 * i + sub) * D + chunk * 8) = v[i];
            }
            return;
        }
#pragma unroll 1
        for (int i = 0; i < WQ / 4; ++i) {
            const int row = 4 * i + sub;
            const u32x4 v = *reinterpret_cast<const u32x4*>(mine + row * OROW + chunk * 8);
            if (oq0 + row < p.Lq) *reinterpret_cast<u32x4*>(orow + row * D + chunk * 8) = v;
        }
    };

    float16_t s_a[QB], s_b[QB];
    // Every tile runs the same two blocks, the last one included: its second block then forms
    // scores nobody uses (of keys past the end of K or past the diagonal; whatever the LDS rows
    // hold, they are masked to -inf before anything reads them), and a block that lies wholly past
    // the end of K contributes zeros.  One instance of the block code instead of a handful keeps
    // the register assignment of the loop the one that was checked.
    auto tile = [&](int t, auto par) {
        block(2 * t, s_a, s_b, par, Yes{});
        block(2 * t + 1, s_b, s_a, par, No{});
        publish();
    };

    int round = 0;
    {
        int bh, qblock;
        if (!item_at(0, bh, qblock)) return;   // (the grid is never larger than the item count: not expected)
        enter_item(bh, qblock);
        stage_first();
        load_queries();
    }
    for (;;) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            l_run[qb] = 0.f;
#pragma unroll
            for (int i = 0; i < DBLK; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[qb][i][r] = 0.f;
        }
        publish();
        {
            // S(0) from the first half of K tile 0, then the keys of block 1 for block 0's score MFMAs
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) fetch_k(k_lds0, ks);
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    if (ks == 0) Mma<T>::score_first(s_a[qb], kf[0], qreg[qb][0]);
                    else         Mma<T>::score_acc(s_a[qb], kf[ks], qreg[qb][ks]);
                }
            asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s_a[0]), "+v"(s_a[1]));   // MFMA results the compiler cannot see coming
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) fetch_k(k_lds0 + 32 * D, ks);
            // The first reference point is the maximum of block 0 itself: nothing to rescale yet.
            // (Every query sees key 0, so the maximum is finite.)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                if (needs_mask(0, qb)) apply_mask(0, qb, s_a[qb]);
                m_run[qb] = half_swap_max(lane_max(s_a[qb]));
                raise_at[qb] = m_run[qb] + lazy_margin;
            }
        }
        for (int t = 0; t < wave_tiles; t += 2) {
            tile(t, Par0{});
            if (t + 1 >= wave_tiles) break;
            tile(t + 1, Par1{});
        }
        // A wavefront that is done before the others (causal: its diagonal comes first) sends its
        // rows off now, under their MFMAs, and then keeps staging tiles for them.
        const bool early = wave_tiles < n_tiles;
        const int ob = b, ohq = hq, oq0 = q0;
        if (early) {
            outputs_to_lds(ob, ohq, oq0);
            outputs_to_memory(ob, ohq, oq0);
        }
        for (int t = wave_tiles; t < n_tiles; ++t) {
            stage_pair(t, AnyPar{t});
            publish();
        }
        // Nobody reads the tiles of this item any more.
        // Order of the hand-over: the next queries are requested first (registers, the longest
        // latency), then this item's outputs go through the wavefront's own LDS region (an LDS read
        // issued while a dozen direct-to-LDS loads are in flight would wait for them), and only then
        // the next item's first tiles are requested.
        int bh, qblock;
        const bool more = item_at(++round, bh, qblock);
        if (more) {
            enter_item(bh, qblock);
            load_queries();
        }
        if (!early) {
            outputs_to_lds(ob, ohq, oq0);
            outputs_to_memory(ob, ohq, oq0);
        }
        if (more) {
            stage_first();
        }
        if (!more) break;
        // (the queries belong in AGPRs from here on: say so, or the allocator keeps half of them in VGPRs
        // and copies four registers in front of every score MFMA)
        asm volatile("" : "+a"(qreg[0][0]), "+a"(qreg[0][1]), "+a"(qreg[0][2]), "+a"(qreg[0][3]), "+a"(qreg[0][4]), "+a"(qreg[0][5]), "+a"(qreg[0][6]), "+a"(qreg[0][7]),
                          "+a"(qreg[1][0]), "+a"(qreg[1][1]), "+a"(qreg[1][2]), "+a"(qreg[1][3]), "+a"(qreg[1][4]), "+a"(qreg[1][5]), "+a"(qreg[1][6]), "+a"(qreg[1][7]));
    }
}

template <typename T>
int launch_t(FlashParams p, bool causal, hipStream_t s) {
    p.n_qblocks = (p.Lq + kWideBM - 1) / kWideBM;
    const long items = static_cast<long>(p.B) * p.Hq * p.n_qblocks;
    // one workgroup per CU (that is all its LDS and registers hold), each walking its share of the items
    int dev = 0, cus = 0;
    PARAS_HIP_TRY(hipGetDevice(&dev));
    PARAS_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    auto magic = [](long d) { return static_cast<unsigned>(((1ull << 32) + static_cast<unsigned long long>(d) - 1) / static_cast<unsigned long long>(d)); };
    p.magic_nq = magic(p.n_qblocks);
    p.magic_hq = magic(p.Hq);
    p.magic_rep = magic(p.Hq / p.Hkv);
    long blocks = items < cus ? items : cus;
    if (blocks >= 8 && (static_cast<long>(p.B) * p.Hq) % 8 == 0) blocks -= blocks % 8;
    const dim3 grid(static_cast<unsigned>(blocks)), wg(256);
    if (causal) hipLaunchKernelGGL((flash_wide_kernel<T, true>), grid, wg, 0, s, p);
    else        hipLaunchKernelGGL((flash_wide_kernel<T, false>), grid, wg, 0, s, p);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // namespace

bool wide_supported(long B, long Hq, long Lq, long Lk, int head, int mask_kind, bool causal) {
    static const int forced = [] { const char* e = std::getenv("PARAS_FLASH_WIDE"); return e ? std::atoi(e) : -1; }();
    if (head != D || mask_kind != 0) return false;
    // the item arithmetic divides by multiply-high: exact while dividend * divisor < 2^32
    const unsigned long long nq = (static_cast<unsigned long long>(Lq) + kWideBM - 1) / kWideBM;
    const unsigned long long bh = static_cast<unsigned long long>(B) * static_cast<unsigned long long>(Hq);
    if (bh * nq * nq >= (1ull << 32) || bh * static_cast<unsigned long long>(Hq) >= (1ull << 32)) return false;
    if (forced >= 0) return forced != 0;
    // One workgroup per CU and 256 queries per item: it needs a few items per CU to keep them all
    // busy and, under the causal rule, long rows for the items' fixed cost to pay off (measured
    // against the 32-queries-per-wavefront kernel: ahead from 4096 causal / 1024 unmasked queries on).
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return false;
    if (bh * nq < 2ull * static_cast<unsigned long long>(cus)) return false;
    return causal ? (Lq >= 4096 && Lk >= 4096) : (Lq >= 1024 && Lk >= 1024);
}

int launch_flash_wide(FlashParams p, bool causal, bool is_bf16, hipStream_t s) {
    return is_bf16 ? launch_t<bf16_t>(p, causal, s) : launch_t<f16_t>(p, causal, s);
}

}  // namespace flash
}  // namespace paras
