// Flash-attention forward for gfx950 (bf16 / fp16 MFMA, fp32 accumulate).
//
// out = softmax(q k^T * scale [+ causal mask]) v, computed tile by tile with an
// online softmax; the [Lq, Lk] score matrix never exists in memory (the
// reference materialises it: csrc/ops/attention_ops.cpp:101,128).
//
// Work decomposition
//   workgroup = 4 wavefronts = 128 queries of one (batch, head); each wave owns
//   32 queries.  K/V are streamed in tiles of 64 keys through LDS (two buffers
//   each, one barrier per tile), shared by the 4 waves.  Tiles go from global
//   memory straight into LDS (buffer_load_dwordx4 ... lds: no staging registers,
//   no LDS store instructions; the buffer descriptor's range check supplies the
//   zeros for rows outside [0, Lk)); rows are unpadded and the 16-byte chunks of a
//   row are XOR-swizzled so that operand reads stay conflict free.
//
// The products are formed transposed so that a lane always owns ONE query:
//   S^T = K Q^T    A = K tile from LDS (lane: key l%32, 8 consecutive d),
//                  B = Q^T from registers (lane: query l%32, same 8 d)
//                  -> accumulator lane (query l%32, half h=l/32) holds, for a
//                  32-key block, keys (r/4)*8 + 4h + r%4, r = 0..15
//   row max / row sum: in-lane over the accumulator registers plus one
//                  v_permlane32_swap between the two half-waves
//   O^T = V^T P^T  B = P^T straight from the S^T accumulators (converted to
//                  16 bit, no shuffle: the accumulator's key order is simply
//                  used as the contraction order),
//                  A = V^T read from the row-major V tile with
//                  ds_read_b64_tr_b16, which transposes 4 keys x 16 d per
//                  16-lane group in the LDS crossbar
//   rescaling O by exp(m_old - m_new) is a per-lane scalar multiply, and it
//                  is lazy: the running max is only raised (and O, l rescaled)
//                  when a block's row max exceeds it by more than 2^8 in the
//                  exponent domain, so after the first block the rescale is
//                  skipped almost always; the same (possibly stale) max is used
//                  for P and for the row sum, so out = O / l is unchanged.
//   row sums       fp32 adds of the exponentials before they are rounded to the
//                  16-bit operand of the PV product
//
// Software pipeline inside a wave: the unit of work is a 32-key block and the
// score MFMAs run one block ahead,
//
//   block j:   [ S(j+1) = K(j+1) Q^T  MFMAs  |  exp / pack / row-sum of S(j) ]   one fenced schedule,
//              [ O^T += V(j)^T P(j)^T MFMAs  |  in-lane row max of S(j+1)    ]   an MFMA per slot
//              mask S(j+1) on the diagonal / at the end of K; raise the running max if needed (rare branch)
//
// so the matrix pipe has independent work in flight under the softmax VALU
// work of the same wave.  K is staged half a tile ahead of V: K tile u holds
// keys [64u-32, 64u+32), so the two blocks whose scores are computed during V
// tile t (blocks 2t+1, 2t+2) both live in K tile t+1, and K and V need only two
// LDS buffers each with a single barrier per tile.  The operand fragments run
// through a register ring that carries across the two blocks of a tile, and a
// tile's first fragments are requested before the next tile pair is.
//
// Three things in the structure exist to keep the compiler's wait insertion
// exact (it is conservative in ways that serialise this loop otherwise): the
// tiles come through buffer loads (an LDS-direct global load makes every later
// LDS wait a full one), each buffer is its own __shared__ array named at
// compile time in the main loop (an LDS read waits for all direct loads in
// flight unless the variables prove them disjoint), and nothing with a branch
// sits between a fragment's request and the MFMA that consumes it.
//
// An optional mask (bytes, nonzero = attend; or additive values of the tensor type;
// broadcast over any of batch / head / query, any stride along the keys) is applied
// to the finished scores of a block; the mask bytes of block j+1 are requested when
// block j starts.  Queries with no visible key so far carry a running maximum of
// -inf and contribute zeros; a query with no visible key at all ends as 0/0 = NaN,
// like the reference's softmax.
//
// v_mfma_f32_32x32x16_{bf16,f16}: 32 MFMAs per wave per 64-key tile at D=128.
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_flash_common.h"
#include "kernels/sdpa_internal.h"

namespace paras {
namespace {

using namespace flash;

constexpr int kBM = 128;   // queries per workgroup: 4 waves x 32

// kMask: 0 none, 1 bytes (nonzero = attend), 2 additive values of type T.
template <typename T, int D, bool kCausal, int kMask>
__global__ __launch_bounds__(256, (D > 128 ? 1 : 2)) void flash_fwd_kernel(const FlashParams p) {
    static_assert(!(kCausal && kMask != 0), "a mask and the causal rule are mutually exclusive");
    // 32-query blocks per wave.  The code is written for any QB; 2 halves the LDS operand
    // traffic per query but needs one wave per SIMD and measured 30 % slower (nothing hides
    // LDS / barrier latency then), so 1 it is: two waves per SIMD, 256 registers each.
    constexpr int QB     = 1;
    constexpr int NW     = 4;
    constexpr int WQ     = 32 * QB;          // queries per wave
    static_assert(kBM == NW * WQ, "workgroup shape");
    constexpr int KSTEPS = D / 16;
    constexpr int DBLK   = D / 32;
    constexpr int CHUNKS = D / 8;
    constexpr int RPI    = 64 / CHUNKS;
    constexpr int NI     = kBN / (RPI * NW);
    auto ksw = [](int row) { return D >= 128 ? (row & 15) : ((row >> 1) & 7); };
    auto vsw = [](int row) { return D >= 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); };

    // LDS: two tiles each of K and V (4 x 16 KiB per workgroup at D = 128, two workgroups per
    // CU).  They are four separate arrays on purpose: the compiler makes an LDS read wait for
    // every direct-to-LDS load in flight unless it can prove from the variables involved that the
    // two do not overlap, and the point of the double buffer is to read one tile while the next
    // one streams in.  The main loop therefore names its buffers at compile time (`Par`), the
    // rarely taken paths pick them at run time (`AnyPar`) and accept the wait.
    __shared__ __attribute__((aligned(1024))) std::uint16_t k_lds0[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t k_lds1[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t v_lds0[kBN * D];
    __shared__ __attribute__((aligned(1024))) std::uint16_t v_lds1[kBN * D];
    using Par0 = std::integral_constant<int, 0>;
    using Par1 = std::integral_constant<int, 1>;
    struct AnyPar { int value; };
    // buffer of tile index parity `par`; `flip` selects the other one
    auto kbuf = [&](auto par, bool flip) -> std::uint16_t* {
        if constexpr (std::is_same<decltype(par), AnyPar>::value) return ((par.value ^ (flip ? 1 : 0)) & 1) ? k_lds1 : k_lds0;
        else return (decltype(par)::value != 0) != flip ? k_lds1 : k_lds0;
    };
    auto vbuf = [&](auto par, bool flip) -> std::uint16_t* {
        if constexpr (std::is_same<decltype(par), AnyPar>::value) return ((par.value ^ (flip ? 1 : 0)) & 1) ? v_lds1 : v_lds0;
        else return (decltype(par)::value != 0) != flip ? v_lds1 : v_lds0;
    };

    const int nq = p.n_qblocks;
    const int BH = p.B * p.Hq;
    int bh, qi;
    {
        const int idx = blockIdx.x;
        if (BH % 16 == 0) {
            const int xcd = idx & 7, j = idx >> 3;
            const int g = j / (2 * nq), r = j % (2 * nq);
            bh = (2 * g + (r & 1)) * 8 + xcd;
            qi = r >> 1;
        } else if (BH % 8 == 0) {
            const int xcd = idx & 7, j = idx >> 3;
            bh = (j / nq) * 8 + xcd;
            qi = j % nq;
        } else {
            bh = idx / nq;
            qi = idx % nq;
        }
    }
    const int qblock = nq - 1 - qi;
    const int b = bh / p.Hq, hq = bh % p.Hq;
    const int hkv = hq / (p.Hq / p.Hkv);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;
    const int q0 = qblock * kBM + wave * WQ;   // first query of this wave; query block qb starts at q0 + 32 qb

    i16x8 qreg[QB][KSTEPS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int my_q = q0 + 32 * qb + lq;
        const int qrow = my_q < p.Lq ? my_q : p.Lq - 1;
        const std::uint16_t* qp = p.q + b * p.qs_b + hq * p.qs_h + static_cast<long>(qrow) * p.qs_l;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) qreg[qb][ks] = *reinterpret_cast<const i16x8*>(qp + ks * 16 + lh * 8);
    }

    const std::uint16_t* kbase = p.k + b * p.ks_b + hkv * p.ks_h;
    const std::uint16_t* vbase = p.v + b * p.vs_b + hkv * p.vs_h;

    int n_tiles = (p.Lk + kBN - 1) / kBN;
    if (kCausal) {
        const int last_q = min(qblock * kBM + kBM, p.Lq) - 1;
        n_tiles = (min(last_q + 1, p.Lk) + kBN - 1) / kBN;
    }
    const int wave_tiles = kCausal ? min(n_tiles, (q0 + WQ - 1) / kBN + 1) : n_tiles;

    // ---- staging: 64 LDS rows <- global rows first .. first+63, straight from memory into LDS
    // with buffer loads.  The buffer descriptor spans rows [0, Lk) of this (batch, kv head), so
    // rows outside it (before the first key in K tile 0, past the end of K in the last tiles)
    // arrive as zeros without a branch: the hardware range-checks every dword of every lane.
    const int srow = wave * RPI + lane / CHUNKS;
    const int slot = lane % CHUNKS;
    const int k_row_bytes = static_cast<int>(p.ks_l) * 2, v_row_bytes = static_cast<int>(p.vs_l) * 2;
    const int k_lane = srow * k_row_bytes + ((slot ^ ksw(srow)) * 16);
    const int v_lane = srow * v_row_bytes + ((slot ^ vsw(srow)) * 16);
    // Request i of a tile fills rows i * RPI * NW + srow.  That is a multiple of 16 rows further on
    // for heads of up to 128 elements, so the swizzle of the row is the swizzle of srow; with 256
    // elements a request covers 8 rows and every other one lands 8 rows on: bit 3 of the K swizzle flips.
    const int k_lane_odd = D > 128 ? srow * k_row_bytes + ((slot ^ ksw(srow + 8)) * 16) : k_lane;
    static_assert((RPI * NW) % 16 == 0 || (RPI * NW == 8 && D == 256), "the staging swizzle assumes whole groups of 16 (or 8) rows per request");
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto make_rsrc = [&](const std::uint16_t* base, int row_bytes) {
        const int bytes = (p.Lk - 1) * row_bytes + D * 2;           // < 2^31: checked by flash_supported
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<std::uint16_t*>(base), 0, bytes, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t k_rsrc = make_rsrc(kbase, k_row_bytes);
    const __amdgpu_buffer_rsrc_t v_rsrc = make_rsrc(vbase, v_row_bytes);
    struct OfK {}; struct OfV {};
    auto stage_one = [&](__amdgpu_buffer_rsrc_t rsrc, auto which, int row_bytes, int first, std::uint16_t* tile, int i) {
        const int r0 = i * RPI * NW;
        constexpr bool is_k = std::is_same<decltype(which), OfK>::value;
        const int lane_off = is_k ? ((i & 1) ? k_lane_odd : k_lane) : v_lane;      // (i is a constant wherever this is called)
        // a negative offset is a huge unsigned one: out of range like the rows past the end
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lptr_t)(tile + (r0 + wave * RPI) * D), 16,
                                                 lane_off + (first + r0) * row_bytes, 0, 0, 0);
    };
    auto stage_rows = [&](__amdgpu_buffer_rsrc_t rsrc, auto which, int row_bytes, int first, std::uint16_t* tile) {
#pragma unroll
        for (int i = 0; i < NI; ++i) stage_one(rsrc, which, row_bytes, first, tile, i);
    };
    // Requests the pair tile t's blocks need beyond K tile t: K tile t+1 and V tile t (`par` = parity of t).
    auto stage_pair = [&](int t, auto par) {
        stage_rows(k_rsrc, OfK{}, k_row_bytes, (t + 1) * kBN - 32, kbuf(par, true));
        stage_rows(v_rsrc, OfV{}, v_row_bytes, t * kBN, vbuf(par, false));
    };
    // Barrier that publishes every tile requested so far.
    auto publish = [&]() {
        // s_waitcnt simm16 on gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8.  The
        // builtin (not inline asm) so that the compiler's own wait bookkeeping sees the loads retire.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    };

    float16_t oacc[QB][DBLK];
    float m_run[QB], l_run[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int i = 0; i < DBLK; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[qb][i][r] = 0.f;
    }

    stage_rows(k_rsrc, OfK{}, k_row_bytes, -32, k_lds0);   // K tile 0: keys 0..31 in its upper half
    stage_pair(0, Par0{});
    publish();

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

    auto needs_mask = [&](int j, int qb) { return (kCausal && j * 32 + 31 > q0 + 32 * qb) || j * 32 + 32 > p.Lk; };
    auto apply_mask = [&](int j, int qb, float16_t& sc) {
        const int my_q = q0 + 32 * qb + lq;
        const int last_visible = kCausal ? min(my_q, p.Lk - 1) : p.Lk - 1;
        const int rel = last_visible - j * 32 - 4 * lh;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if ((r >> 2) * 8 + (r & 3) > rel) sc[r] = -INFINITY;
    };
    // ---- optional user mask.  Lane (query, half lh) needs, for block j, keys j*32 + 8g + 4 lh + i
    // (g, i = 0..3; accumulator register 4g + i): four runs of four consecutive keys.  The runs of
    // block j+1 are requested at the start of block j and applied when its scores are finished.
    constexpr int MREGS = kMask == 0 ? 1 : (kMask == 1 ? 4 : 8);
    const unsigned char* mrow = nullptr;
    if constexpr (kMask != 0) {
        const int my_q = q0 + lq;
        const long qrow = my_q < p.Lq ? my_q : p.Lq - 1;
        mrow = p.mask + (static_cast<long>(b) * p.ms_b + static_cast<long>(hq) * p.ms_h + qrow * p.ms_q) * (kMask == 1 ? 1 : 2);
    }
    // A mask that is contiguous along the keys, with Lk >= 4: a run that hangs over the end of the
    // row is read from the row's last four elements and shifted down, so no load leaves the row and
    // no branch is needed; keys >= Lk get zero bits and are masked by the end-of-K rule.  Any other
    // stride along the keys (0: a view that broadcasts one value per query over the keys; > 1: slices
    // and transposed views) is read element by element into the same registers -- sixteen small
    // loads per block instead of four, requested a block ahead like the runs.
    //   A block that lies wholly inside a contiguous row is not read as four runs per lane (a wavefront's
    // 64 lanes then touch 64 different places four times over) but as one 16-byte piece per lane of
    // the block's 32 (bool) or 64 (additive: two pieces) bytes of its query's row: half lh holds keys
    // 16 lh .. 16 lh + 15 and needs keys 8 g + 4 lh .. + 3, so the two halves of a query swap every
    // other run when the mask is applied (v_permlane32_swap: lanes l and l + 32).
    const bool mask_runs = p.ms_k == 1 && p.Lk >= 4;       // uniform
    auto mask_whole_block = [&](int j) { return mask_runs && j * 32 + 32 <= p.Lk; };      // uniform
    auto mask_load = [&](int j, std::uint32_t (&mr)[MREGS]) {
        if constexpr (kMask != 0) {
            typedef std::uint32_t u32_any __attribute__((aligned(1)));
            typedef u32x4 u32x4_any __attribute__((aligned(1)));
            if (mask_whole_block(j)) {
                constexpr int ES = kMask == 1 ? 1 : 2;
                const unsigned char* at = mrow + (j * 32 + 16 * lh) * ES;
#pragma unroll
                for (int h = 0; h < ES; ++h) {
                    const u32x4 w = *reinterpret_cast<const u32x4_any*>(at + 16 * h);
#pragma unroll
                    for (int i = 0; i < 4; ++i) mr[4 * h + i] = w[i];
                }
                return;
            }
            if (!mask_runs) {
                constexpr int ES = kMask == 1 ? 1 : 2;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    std::uint32_t e[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = min(j * 32 + 8 * g + 4 * lh + i, p.Lk - 1);   // (keys past the end: any value, the end-of-K rule masks them)
                        const unsigned char* at = mrow + static_cast<long>(key) * p.ms_k * ES;
                        if constexpr (kMask == 1) e[i] = *at;
                        else                      e[i] = *reinterpret_cast<const std::uint16_t*>(at);
                    }
                    if constexpr (kMask == 1) {
                        mr[g] = e[0] | (e[1] << 8) | (e[2] << 16) | (e[3] << 24);
                    } else {
                        mr[2 * g] = e[0] | (e[1] << 16);
                        mr[2 * g + 1] = e[2] | (e[3] << 16);
                    }
                }
                return;
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int key = j * 32 + 8 * g + 4 * lh;
                const int at = min(key, p.Lk - 4);
                const unsigned sh = static_cast<unsigned>(key - at);          // 0 unless the run hangs over
                if constexpr (kMask == 1) {
                    const std::uint32_t w = *reinterpret_cast<const u32_any*>(mrow + at);
                    mr[g] = sh < 4 ? w >> (8 * sh) : 0u;
                } else {
                    const std::uint64_t w = static_cast<std::uint64_t>(*reinterpret_cast<const u32_any*>(mrow + 2 * at)) |
                                            (static_cast<std::uint64_t>(*reinterpret_cast<const u32_any*>(mrow + 2 * at + 4)) << 32);
                    const std::uint64_t v = sh < 4 ? w >> (16 * sh) : 0ull;
                    mr[2 * g] = static_cast<std::uint32_t>(v);
                    mr[2 * g + 1] = static_cast<std::uint32_t>(v >> 32);
                }
            }
        }
    };
    // With a mask the scores are narrowed where the host engine narrows them (attention_ops.cpp:101-128:
    // the product, the scaled product and the sum with an additive mask are tensors of T): a row that
    // sees few keys is decided by one or two scores, and a 2^-9 step on one of them is several per cent
    // on its weight.  The scores leave here scaled; the kernel's scale is 1 in these variants.
    auto round_T = [](float x) { return Elem<T>::to_f32(Elem<T>::from_f32_finite(x)); };
    auto mask_apply = [&](int j, const std::uint32_t (&loaded)[MREGS], float16_t& sc) {
        std::uint32_t mr[MREGS];
#pragma unroll
        for (int i = 0; i < MREGS; ++i) mr[i] = loaded[i];
        if constexpr (kMask != 0) {
            if (mask_whole_block(j)) {
                // registers as loaded: the lane's own sixteen keys.  Lower half: keeps its runs 0 and 2 (bool:
                // one register each; additive: two), gets runs 0 and 2 of the upper half for its runs 1 and 3.
                auto swap = [&](int x, int y) {       // upper half of register x <-> lower half of register y
                    const auto r = __builtin_amdgcn_permlane32_swap(mr[x], mr[y], false, false);
                    mr[x] = r[0];
                    mr[y] = r[1];
                };
                if constexpr (kMask == 1) {
                    swap(0, 1);
                    swap(2, 3);
                    const std::uint32_t t = mr[1];    // runs in order: registers 0, 2, 1, 3
                    mr[1] = mr[2];
                    mr[2] = t;
                } else {
                    swap(0, 2);
                    swap(1, 3);
                    swap(4, 6);
                    swap(5, 7);
                    const std::uint32_t t2 = mr[2], t3 = mr[3];     // runs in order: registers (0,1), (4,5), (2,3), (6,7)
                    mr[2] = mr[4];
                    mr[3] = mr[5];
                    mr[4] = t2;
                    mr[5] = t3;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = round_T(round_T(sc[r]) * p.score_scale);
        }
        if constexpr (kMask == 1) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (((mr[r >> 2] >> (8 * (r & 3))) & 0xffu) == 0) sc[r] = -INFINITY;
        } else if constexpr (kMask == 2) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const std::uint16_t bits = static_cast<std::uint16_t>(mr[r >> 1] >> (16 * (r & 1)));
                sc[r] = round_T(sc[r] + Elem<T>::to_f32(bits));
            }
        }
    };
    auto lane_max = [](const float16_t& sc) {
        float mx = sc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(mx, sc[r]);
        return mx;
    };
    // Raise the running max of query block qb if block max `mx` (this lane's half) needs it.  The
    // test runs on each lane's own half of the keys; the two halves of a query are only brought
    // together inside the rare branch.
    auto raise_max = [&](float (&mx)[QB]) {
        // (the compare builtin hands back the wavefront's lane mask as it stands; a bool fed to the
        // ballot builtin is first turned into 0 / 1 per lane and compared again)
        unsigned long long grow = 0;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) grow |= __builtin_amdgcn_fcmpf(mx[qb], m_run[qb] + lazy_margin, 2 /* ordered greater than */);
        if (__builtin_expect(grow != 0, 0)) {  // wave-uniform, rare after block 0: the common path falls through
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const float m_new = fmaxf(m_run[qb], half_swap_max(mx[qb]));
                // (equal covers -inf on both sides: a query that has seen no key yet keeps its zeros)
                const float alpha = m_run[qb] == m_new ? 1.f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * p.scale_log2);
                m_run[qb] = m_new;
                l_run[qb] *= alpha;
#pragma unroll
                for (int i = 0; i < DBLK; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[qb][i][r] *= alpha;
            }
        }
    };
    // Mask where needed, then raise.  `mx` holds the unmasked in-lane maxima on entry.
    auto finish_scores = [&](int j, float16_t (&sc)[QB], float (&mx)[QB], const std::uint32_t (&mr)[MREGS]) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            if constexpr (kMask != 0) mask_apply(j, mr, sc[qb]);
            if (__builtin_expect(needs_mask(j, qb), 0)) apply_mask(j, qb, sc[qb]);
            if (kMask != 0 || needs_mask(j, qb)) mx[qb] = lane_max(sc[qb]);
        }
        raise_max(mx);
    };

    // One block: exponentials of `cur` = S(j) and, if kNext, the MFMAs of S(j+1) into `nxt`,
    // then PV(j).  The MFMA part is a fixed schedule of KSTEPS + 2*DBLK slots (QB MFMAs per
    // slot, sharing one LDS fragment), fenced so that the compiler keeps the order.  Fragment
    // reads run two slots ahead through a ring of four registers that lives across blocks: a
    // block expects the operands of its first two slots in flight and, in its last two slots,
    // requests those of its successor (`tail`: KFirst = a block that starts with score MFMAs,
    // VFirst = one that only has PV left, NoTail = the successor's rows are not resident yet).
    // The 8*QB exp pairs (2 fma + 2 exp + cvt + 2 add each) are spread between the MFMAs so the
    // matrix pipe has an instruction in flight while the VALU works.  P(s2=0) is complete
    // before the first PV MFMA, P(s2=1) before the first PV MFMA that uses it; the row maxima
    // of S(j+1) are reduced as a tree in the slots after the last exp pair, so the rescale
    // decision is ready when the last MFMA issues.
    i16x8 frag[4];
    constexpr int NS = KSTEPS + 2 * DBLK;                 // slot c >= KSTEPS: PV(s2 = (c-KSTEPS)/DBLK, db = (c-KSTEPS)%DBLK)
    static_assert(NS % 4 == 0 && KSTEPS % 4 == 0, "the fragment ring is indexed by slot % 4 across blocks");
    // `par` is the parity of block j's tile (j >> 1): V(j) lives in the V buffer of that parity,
    // the K rows of block j+1 in the K buffer of the other one.
    auto fetch = [&](int j, int c, auto par) {            // operand of slot c of block j -> frag[c % 4]
        if (c < KSTEPS) {
            const std::uint16_t* kt = kbuf(par, true) + ((j + 2) & 1) * 32 * D;   // rows of block j+1
            frag[c % 4] = *reinterpret_cast<const i16x8*>(kt + k_rd[c]);
        } else {
            const std::uint16_t* vt = vbuf(par, false) + (j & 1) * 32 * D;
            const int s2 = (c - KSTEPS) / DBLK, db = (c - KSTEPS) % DBLK;
            const std::uint16_t* vp = vt + v_rd[db] + 16 * s2 * D;
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp + 8 * D));
            frag[c % 4] = i16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
    };
    struct KFirst {}; struct VFirst {}; struct NoTail {};
    auto first_fetches = [&](int j, auto kind, auto par) {   // what block j's first two slots consume
        constexpr int s0 = std::is_same<decltype(kind), KFirst>::value ? 0 : KSTEPS;
        fetch(j, s0, par);
        fetch(j, s0 + 1, par);
    };
    auto block = [&](int j, float16_t (&cur)[QB], float16_t (&nxt)[QB], auto next_tag, auto tail, auto par, auto stage_tag) {
        constexpr bool kNext = decltype(next_tag)::value;
        constexpr bool kStage = decltype(stage_tag)::value;
        constexpr bool kTail = !std::is_same<decltype(tail), NoTail>::value;
        constexpr int S0 = kNext ? 0 : KSTEPS;           // first slot that exists
        static_assert(QB == 1, "the max tree below is written for one query block per wave");
        float mc[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            mc[qb] = m_run[qb] * p.scale_log2;
            // every key so far masked out: the reference point is arbitrary, and it must not be -inf
            if constexpr (kMask != 0) mc[qb] = m_run[qb] == -INFINITY ? 0.f : mc[qb];
        }
        std::uint32_t mnext[MREGS];
        if constexpr (kNext) mask_load(j + 1, mnext);
        u32x4 pw[QB][2];
        float mx[QB], t3[5], t2[2];
        auto exp_pair = [&](int qb, int i) {              // elements 2i, 2i+1 of cur[qb]
            const float e0 = __builtin_amdgcn_exp2f(fmaf(cur[qb][2 * i], p.scale_log2, -mc[qb]));
            const float e1 = __builtin_amdgcn_exp2f(fmaf(cur[qb][2 * i + 1], p.scale_log2, -mc[qb]));
            const std::uint32_t w = Mma<T>::pack2(e0, e1);
            // Plain adds of the unrounded exponentials: v_dot2_f32_bf16 on the packed pair is one
            // instruction instead of two, but it runs on the matrix pipe's side and stalls the
            // MFMA next to it (measured: 4 % of the kernel).
            l_run[qb] += e0 + e1;
            asm volatile("" : "+v"(l_run[qb]));           // keeps the row-sum update in this slot
            pw[qb][i / 4][i % 4] = w;
        };
        // pair (qb, i) is issued just before the MFMAs of slot pair_slot(qb, i)
        auto pair_slot = [](int qb, int i) {
            if (i < 4) return kNext ? (qb * 4 + i) * KSTEPS / (4 * QB) : KSTEPS;
            return KSTEPS + (qb * 4 + i - 4) * DBLK / (4 * QB);
        };
        constexpr int MAX0 = KSTEPS + DBLK + (DBLK >= 4 ? 1 : 0);   // after the last exp pair; S(j+1) finished KSTEPS slots ago

#pragma unroll
        for (int c = S0; c < NS; ++c) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (pair_slot(qb, i) == c) exp_pair(qb, i);
            if (c < KSTEPS) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    if (c == 0) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) nxt[qb][r] = 0.f;
                    }
                    nxt[qb] = Mma<T>::run(frag[c % 4], qreg[qb][c], nxt[qb]);
                }
            } else {
                const int s2 = (c - KSTEPS) / DBLK, db = (c - KSTEPS) % DBLK;
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
                    oacc[qb][db] = Mma<T>::run(frag[c % 4], __builtin_bit_cast(i16x8, pw[qb][s2]), oacc[qb][db]);
            }
            if constexpr (kStage) {
                // The next tile pair (K tile t+2, V tile t+1), one request every other slot: all of
                // them at the start of the tile, from every wave at once right after the barrier,
                // cost 1.5 % (they queue up in front of the waves' first MFMAs).
                static_assert(2 * (2 * NI - 1) < NS, "the requests fit the block's slots");
                if (c % 2 == 0 && c / 2 < 2 * NI) {
                    const int i = c / 2, t = j >> 1;
                    if (i < NI) stage_one(k_rsrc, OfK{}, k_row_bytes, (t + 2) * kBN - 32, kbuf(par, false), i);
                    else        stage_one(v_rsrc, OfV{}, v_row_bytes, (t + 1) * kBN, vbuf(par, true), i - NI);
                }
            }
            if (c + 2 < NS) fetch(j, c + 2, par);
            else if constexpr (kTail)    // only ever the second block of the same tile: same parity
                fetch(j + 1, (std::is_same<decltype(tail), KFirst>::value ? 0 : KSTEPS) + (c + 2 - NS), par);
            if constexpr (kNext && kMask == 0) {      // (with a user mask the maxima are taken after masking)
                const float16_t& sv = nxt[0];
                if (c == MAX0) {
#pragma unroll
                    for (int g = 0; g < 5; ++g) {
                        t3[g] = fmaxf(fmaxf(sv[3 * g], sv[3 * g + 1]), sv[3 * g + 2]);
                        asm volatile("" : "+v"(t3[g]));   // keeps the reduction in this slot
                    }
                }
                if (c == MAX0 + 1) {
                    t2[0] = fmaxf(fmaxf(t3[0], t3[1]), t3[2]);
                    t2[1] = fmaxf(fmaxf(t3[3], t3[4]), sv[15]);
                    mx[0] = fmaxf(t2[0], t2[1]);
                    asm volatile("" : "+v"(mx[0]));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (kNext) finish_scores(j + 1, nxt, mx, mnext);
    };
    using Yes = std::true_type;
    using No  = std::false_type;

    float16_t s_a[QB], s_b[QB];
    if (wave_tiles > 0) {
        // S(0): keys 0..31 = rows 32..63 of K tile 0
        float mx[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s_a[qb][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks)
                s_a[qb] = Mma<T>::run(*reinterpret_cast<const i16x8*>(&k_lds0[32 * D + k_rd[ks]]), qreg[qb][ks], s_a[qb]);
            mx[qb] = lane_max(s_a[qb]);
        }
        std::uint32_t m0[MREGS];
        mask_load(0, m0);
        finish_scores(0, s_a, mx, m0);
    }
    // One tile of the main loop (`par` = parity of t, a compile-time name for the buffers; two
    // tiles per trip).  The tile's first block also requests the next tile pair (= stage_pair(t + 1)).
    auto tile = [&](int t, auto par) {
        first_fetches(2 * t, KFirst{}, par);
        __builtin_amdgcn_sched_barrier(0);                // keep the reads ahead of the requests
        block(2 * t, s_a, s_b, Yes{}, KFirst{}, par, Yes{});
        block(2 * t + 1, s_b, s_a, Yes{}, NoTail{}, par, No{}); // its successor's K rows arrive with the barrier below
        publish();
    };
    int t_main = 0;
    for (; t_main + 2 < wave_tiles; t_main += 2) {
        tile(t_main, Par0{});
        tile(t_main + 1, Par1{});
    }
    if (t_main + 1 < wave_tiles) {
        tile(t_main, Par0{});
        ++t_main;
    }
    if (wave_tiles > 0) {  // the wave's last tile: nothing to compute ahead in its second block
        const int t = wave_tiles - 1;
        const AnyPar par{t};
        if (t + 1 < n_tiles) stage_pair(t + 1, AnyPar{t + 1});
        // The tile's second block contributes nothing when it starts past the end of K or, for a
        // causal wave, past the wave's last query (every other wave's diagonal tile).
        const int second0 = (2 * t + 1) * 32;
        if (second0 >= p.Lk || (kCausal && second0 > q0 + WQ - 1)) {
            first_fetches(2 * t, VFirst{}, par);
            block(2 * t, s_a, s_b, No{}, NoTail{}, par, No{});
        } else {
            first_fetches(2 * t, KFirst{}, par);
            block(2 * t, s_a, s_b, Yes{}, VFirst{}, par, No{});
            block(2 * t + 1, s_b, s_a, No{}, NoTail{}, par, No{});
        }
        publish();
    }
    for (int t = wave_tiles; t < n_tiles; ++t) {           // done early (causal): keep staging for the other waves
        if (t + 1 < n_tiles) stage_pair(t + 1, AnyPar{t + 1});
        publish();
    }

#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int my_q = q0 + 32 * qb + lq;
        const float l_tot = half_swap_sum(l_run[qb]);
        const float inv_l = 1.0f / l_tot;
        if (my_q < p.Lq) {
            std::uint16_t* op = p.out + ((static_cast<long>(b) * p.Hq + hq) * p.Lq + my_q) * D;
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = db * 32 + g * 8 + 4 * lh;
                    u32x2 w;
                    w[0] = Mma<T>::pack2(oacc[qb][db][4 * g + 0] * inv_l, oacc[qb][db][4 * g + 1] * inv_l);
                    w[1] = Mma<T>::pack2(oacc[qb][db][4 * g + 2] * inv_l, oacc[qb][db][4 * g + 3] * inv_l);
                    *reinterpret_cast<u32x2*>(op + d) = w;
                }
            if (p.lse != nullptr && lh == 0)
                p.lse[(static_cast<long>(b) * p.Hq + hq) * p.Lq + my_q] = m_run[qb] * p.scale + logf(l_tot);
        }
    }
}

template <typename T, int D>
int launch_t(FlashParams p, bool causal, int mask_kind, hipStream_t s) {
    p.n_qblocks = (p.Lq + kBM - 1) / kBM;
    const long blocks = static_cast<long>(p.B) * p.Hq * p.n_qblocks;
    const dim3 grid(static_cast<unsigned>(blocks)), wg(256);
    if (causal)              hipLaunchKernelGGL((flash_fwd_kernel<T, D, true, 0>), grid, wg, 0, s, p);
    else if (mask_kind == 1) hipLaunchKernelGGL((flash_fwd_kernel<T, D, false, 1>), grid, wg, 0, s, p);
    else if (mask_kind == 2) hipLaunchKernelGGL((flash_fwd_kernel<T, D, false, 2>), grid, wg, 0, s, p);
    else                     hipLaunchKernelGGL((flash_fwd_kernel<T, D, false, 0>), grid, wg, 0, s, p);
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool mult8(const int64_t* strides) { return strides[0] % 8 == 0 && strides[1] % 8 == 0 && strides[2] % 8 == 0; }

}  // namespace

bool flash_supported(const paras_sdpa_args& a) {
    if (a.dtype != PARAS_BF16 && a.dtype != PARAS_F16) return false;
    if (a.D != a.Dv || (a.D != 64 && a.D != 128 && a.D != 256)) return false;
    if (a.attn != nullptr) return false;                            // the weights are never formed here
    if (a.mask_kind != 0 && (a.mask == nullptr || a.is_causal)) return false;
    if (a.mask_kind < 0 || a.mask_kind > 2) return false;
    if (a.mask_kind != 0 && a.mask_strides[3] < 0) return false;
    if (a.Lq < 1 || a.Lk < 1) return false;
    if (!(a.scale > 0.0) || !std::isfinite(a.scale)) return false;  // the running max is taken on raw scores
    if (!aligned16(a.q) || !aligned16(a.k) || !aligned16(a.v) || !aligned16(a.out)) return false;
    if (!mult8(a.q_strides) || !mult8(a.k_strides) || !mult8(a.v_strides)) return false;
    const int64_t nq = (a.Lq + kBM - 1) / kBM;
    if (a.B * a.Hq * nq > 0x7fffffffLL || a.Lq > 0x3fffffff || a.Lk > 0x3fffffff) return false;
    // K / V tiles are fetched with 32-bit byte offsets against a buffer descriptor per (batch, head)
    // that spans rows [0, Lk); offsets of rows up to one tile outside it must not wrap into it.
    for (const int64_t* st : {a.k_strides, a.v_strides}) {
        if (st[2] < 0) return false;
        if ((a.Lk + 2 * kBN) * st[2] * 2 + a.D * 2 >= 0x7fffffffLL) return false;
    }
    return true;
}

bool flash_uses_wide(const paras_sdpa_args& a) {
    return flash::wide_supported(a.B, a.Hq, a.Lq, a.Lk, static_cast<int>(a.D), a.mask_kind, a.is_causal != 0);
}

int launch_flash(const paras_sdpa_args& a, hipStream_t s) {
    FlashParams p;
    p.q = static_cast<const std::uint16_t*>(a.q);
    p.k = static_cast<const std::uint16_t*>(a.k);
    p.v = static_cast<const std::uint16_t*>(a.v);
    p.out = static_cast<std::uint16_t*>(a.out);
    p.lse = a.lse;
    p.qs_b = a.q_strides[0]; p.qs_h = a.q_strides[1]; p.qs_l = a.q_strides[2];
    p.ks_b = a.k_strides[0]; p.ks_h = a.k_strides[1]; p.ks_l = a.k_strides[2];
    p.vs_b = a.v_strides[0]; p.vs_h = a.v_strides[1]; p.vs_l = a.v_strides[2];
    p.B = static_cast<int>(a.B); p.Hq = static_cast<int>(a.Hq); p.Hkv = static_cast<int>(a.Hkv);
    p.Lq = static_cast<int>(a.Lq); p.Lk = static_cast<int>(a.Lk);
    p.n_qblocks = 0;  // set by the launcher for the workgroup size it picks
    p.scale = static_cast<float>(a.scale);
    p.scale_log2 = static_cast<float>(a.scale * 1.4426950408889634);
    p.mask = static_cast<const unsigned char*>(a.mask);
    p.ms_b = a.mask_strides[0]; p.ms_h = a.mask_strides[1]; p.ms_q = a.mask_strides[2]; p.ms_k = a.mask_strides[3];
    p.score_scale = static_cast<float>(a.scale);
    if (a.mask_kind != 0) {          // the masked variants scale the scores themselves, between two narrowings
        p.scale = 1.0f;
        p.scale_log2 = 1.4426950408889634f;
    }
    const bool causal = a.is_causal != 0;
    const int mk = a.mask_kind;
    if (flash_uses_wide(a)) return launch_flash_wide(p, causal, a.dtype == PARAS_BF16, s);
    if (a.dtype == PARAS_BF16)
        return a.D == 256 ? launch_t<bf16_t, 256>(p, causal, mk, s) : a.D == 128 ? launch_t<bf16_t, 128>(p, causal, mk, s) : launch_t<bf16_t, 64>(p, causal, mk, s);
    return a.D == 256 ? launch_t<f16_t, 256>(p, causal, mk, s) : a.D == 128 ? launch_t<f16_t, 128>(p, causal, mk, s) : launch_t<f16_t, 64>(p, causal, mk, s);
}

}  // namespace paras
