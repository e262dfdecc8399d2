// Split-KV decode attention for gfx950: few query rows per KV head (query
// length x GQA group <= 16), long K/V, bf16 / fp16, head dim 64 or 128.  The job is
// HBM-bound -- every K and V byte is read exactly once, K/V heads are never
// replicated for GQA (the reference copies them Hq/Hkv times:
// csrc/ops/tensor_ops.cpp:687-729) -- so the design is about keeping many
// independent 16-byte loads in flight, not about MFMA rate.
//
// grid = (splits, B*Hkv).  A workgroup owns one contiguous chunk of keys of one
// KV head; each of its 4 waves streams a quarter of the chunk in 32-key tiles:
//   S^T = K Q^T   v_mfma_f32_16x16x32: A = K rows loaded straight from HBM
//                 into registers (lane: key l%16, d = 32*step + 8*(l/16)..+7),
//                 B = the <=16 query rows (padded with zeros), in registers
//   online softmax per query (lane l%16), max shared by the 4 lane groups
//   O^T += V^T P^T  A = V^T via ds_read_b64_tr_b16 from a per-wave LDS tile
//                 (V is the one operand whose contraction index is not
//                 contiguous in memory), B = P^T from the S^T accumulators
// The 4 waves merge their (max, sum, O) in LDS; with more than one split the
// partial goes to the workspace and decode_combine_kernel merges the splits.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>

#include "core/device_context.h"
#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_internal.h"

namespace paras {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves   = 4;
constexpr int kTile    = 32;        // keys per wave per step
// V row stride in LDS is D + 16 elements: 8 consecutive rows x 32 B then hit 64 distinct banks
// (288-byte rows at D = 128, 160-byte rows at D = 64).
constexpr int kMaxRows = 16;        // query rows per KV head (MFMA N)

typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

struct DecodeParams {
    const std::uint16_t* q;
    const std::uint16_t* k;
    const std::uint16_t* v;
    std::uint16_t* out;
    float* lse;
    float* part_o;   // [pairs, splits, 16, D]
    float* part_ml;  // [pairs, splits, 2, 16]
    long qs_b, qs_h, qs_l, ks_b, ks_h, ks_l, vs_b, vs_h, vs_l;
    int B, Hq, Hkv, Lq, Lk, G, R;
    int splits, chunk;  // keys per workgroup
    float scale_log2, scale;
    // optional mask (element strides; 0 = broadcast): bytes that are zero / non-zero, or additive values of the tensor dtype
    const unsigned char* mask;
    long ms_b, ms_h, ms_q, ms_k;
    float inv_scale;    // the scores are kept unscaled: an additive mask value m enters as m / scale
};

template <typename T> struct Mma16;
template <> struct Mma16<bf16_t> {
    __device__ static __forceinline__ float4_t run(i16x8 a, i16x8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ std::uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(std::uint32_t, __builtin_convertvector(v, bf16x2));
    }
};
template <> struct Mma16<f16_t> {
    __device__ static __forceinline__ float4_t run(i16x8 a, i16x8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ std::uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(std::uint32_t, __builtin_convertvector(v, f16x2));
    }
};

// Combine over the 4 lane groups (lanes l, l^16, l^32, l^48) that share a query.
__device__ __forceinline__ float group_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16, kWave));
    return fmaxf(x, __shfl_xor(x, 32, kWave));
}
__device__ __forceinline__ float group_sum(float x) {
    x += __shfl_xor(x, 16, kWave);
    return x + __shfl_xor(x, 32, kWave);
}

// kMask: 0 = none, 1 = bool (true = attend), 2 = additive values of dtype T
template <typename T, int D, int kMask>
__global__ __launch_bounds__(kThreads, (D > 128 ? 1 : 2)) void decode_split_kernel(const DecodeParams p) {
    constexpr int kD = D, kVS = D + 16;
    constexpr int KS = D / 32;           // 32-wide contraction steps of q k^T
    constexpr int DB = D / 16;           // 16-wide output blocks of O^T
    constexpr int VCH = kTile * D / 8 / 64;   // 16-byte chunks of a V tile per lane
    // Per-wave V tiles (double buffered); reused as fp32 merge space at the end.
    __shared__ __attribute__((aligned(16))) std::uint16_t v_lds[kWaves][2][kTile * (D + 16)];
    __shared__ float m_lds[kWaves][kMaxRows], l_lds[kWaves][kMaxRows];

    const int split = blockIdx.x, pair = blockIdx.y;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 15, lg = lane >> 4;

    // ---- the query rows of this KV head: row r = gi*Lq + i  (head hkv*G+gi, position i)
    i16x8 qreg[KS];
    {
        const bool live = lq < p.R;
        const int gi = live ? lq / p.Lq : 0, qi = live ? lq % p.Lq : 0;
        const std::uint16_t* qp = p.q + b * p.qs_b + static_cast<long>(hkv * p.G + gi) * p.qs_h + static_cast<long>(qi) * p.qs_l;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            i16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            qreg[ks] = live ? *reinterpret_cast<const i16x8*>(qp + 32 * ks + 8 * lg) : z;
        }
    }

    // ---- this lane's mask row (query row lq): the 8 keys it scores per tile are 4 lg .. 4 lg + 3 of each 16-key block
    const unsigned char* mrow = nullptr;
    if constexpr (kMask != 0) {
        const bool live = lq < p.R;
        const int gi = live ? lq / p.Lq : 0, qi = live ? lq % p.Lq : 0;
        mrow = p.mask + (static_cast<long>(b) * p.ms_b + static_cast<long>(hkv * p.G + gi) * p.ms_h + static_cast<long>(qi) * p.ms_q) * (kMask == 1 ? 1 : 2);
    }

    // ---- this wave's key range
    const int chunk0 = split * p.chunk;
    const int chunk1 = min(chunk0 + p.chunk, p.Lk);
    const int wlen = (p.chunk / kWaves);  // chunk is a multiple of kWaves*kTile
    const int k_begin = chunk0 + wave * wlen;
    const int k_end = min(k_begin + wlen, chunk1);
    const int n_tiles = k_end > k_begin ? (k_end - k_begin + kTile - 1) / kTile : 0;

    const std::uint16_t* kbase = p.k + b * p.ks_b + hkv * p.ks_h;
    const std::uint16_t* vbase = p.v + b * p.vs_b + hkv * p.vs_h;

    i16x8 kcur[2][KS], knext[2][KS];
    u32x4 vst[VCH];
    auto load_k = [&](int t, i16x8 (&dst)[2][KS]) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            int key = k_begin + t * kTile + kb * 16 + lq;
            key = key < p.Lk ? key : p.Lk - 1;  // masked later; keep the load in bounds
            const std::uint16_t* kp = kbase + static_cast<long>(key) * p.ks_l + 8 * lg;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) dst[kb][ks] = __builtin_bit_cast(i16x8, load16_nt(kp + 32 * ks));  // read once: keep it out of the caches
        }
    };
    auto load_v = [&](int t) {
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = lane + i * 64;  // 16-byte chunk of the 32 x D tile
            const int row = c / (D / 8), col = (c % (D / 8)) * 8;
            const int key = k_begin + t * kTile + row;
            vst[i] = key < k_end ? load16_nt(vbase + static_cast<long>(key) * p.vs_l + col) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_v = [&](int buf) {
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = lane + i * 64;
            const int row = c / (D / 8), col = (c % (D / 8)) * 8;
            *reinterpret_cast<u32x4*>(&v_lds[wave][buf][row * kVS + col]) = vst[i];
        }
    };

    float4_t oacc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) oacc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // Every wave starts at a tile of its own within its range and wraps around: the workgroups and
    // waves, which advance in step, would otherwise always be the same power of two apart in memory.
    const int rot = n_tiles > 1 ? (pair * 5 + split * 3 + wave * 7) % n_tiles : 0;
    auto tile_of = [&](int t) {
        const int tt = t + rot;
        return tt >= n_tiles ? tt - n_tiles : tt;
    };
    if (n_tiles > 0) {
        load_k(tile_of(0), kcur);
        load_v(tile_of(0));
        store_v(0);
    }
    // ds_read_tr lane offsets: group lg reads keys 4*lg + (m/4) (+16), 4 d's at 4*(m%4)
    const int v_off = (4 * lg + (lq >> 2)) * kVS + 4 * (lq & 3);

    for (int t = 0; t < n_tiles; ++t) {
        const int buf = t & 1;
        if (t + 1 < n_tiles) {
            load_k(tile_of(t + 1), knext);
            load_v(tile_of(t + 1));
        }
        // S^T for two 16-key blocks
        float4_t sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            sacc[kb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sacc[kb] = Mma16<T>::run(kcur[kb][ks], qreg[ks], sacc[kb]);
        }
        const int key0 = k_begin + tile_of(t) * kTile;
        if constexpr (kMask != 0) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    int key = key0 + kb * 16 + 4 * lg + r;
                    key = key < p.Lk ? key : p.Lk - 1;                       // keys past the end are masked below anyway
                    if constexpr (kMask == 1) {
                        if (mrow[static_cast<long>(key) * p.ms_k] == 0) sacc[kb][r] = -INFINITY;
                    } else {
                        const std::uint16_t bits = *reinterpret_cast<const std::uint16_t*>(mrow + static_cast<long>(key) * p.ms_k * 2);
                        sacc[kb][r] = fmaf(Elem<T>::to_f32(bits), p.inv_scale, sacc[kb][r]);
                    }
                }
        }
        if (key0 + kTile > k_end) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (key0 + kb * 16 + 4 * lg + r >= k_end) sacc[kb][r] = -INFINITY;
        }
        float mloc = fmaxf(fmaxf(fmaxf(sacc[0][0], sacc[0][1]), fmaxf(sacc[0][2], sacc[0][3])),
                           fmaxf(fmaxf(sacc[1][0], sacc[1][1]), fmaxf(sacc[1][2], sacc[1][3])));
        mloc = group_max(mloc);
        const float m_new = fmaxf(m_run, mloc);
        // (with a mask every key so far may be masked out: -inf on both sides keeps the zeros, and the
        // reference point of the exponentials must not be -inf)
        const float alpha = m_run == m_new ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * p.scale_log2);
        const float mc = m_new == -INFINITY ? 0.f : m_new * p.scale_log2;
        m_run = m_new;
        float lsum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(fmaf(sacc[kb][r], p.scale_log2, -mc));
                sacc[kb][r] = e;
                lsum += e;
            }
        l_run = l_run * alpha + lsum;
#pragma unroll
        for (int i = 0; i < DB; ++i) oacc[i] *= alpha;
        // P^T operand: contraction order e<4 -> key 4*lg+e, e>=4 -> key 16+4*lg+(e-4)
        u32x4 w;
        w[0] = Mma16<T>::pack2(sacc[0][0], sacc[0][1]);
        w[1] = Mma16<T>::pack2(sacc[0][2], sacc[0][3]);
        w[2] = Mma16<T>::pack2(sacc[1][0], sacc[1][1]);
        w[3] = Mma16<T>::pack2(sacc[1][2], sacc[1][3]);
        const i16x8 pb = __builtin_bit_cast(i16x8, w);

        // Make this wave's LDS tile (written by its own lanes) visible to all of its lanes.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const std::uint16_t* vp = &v_lds[wave][buf][v_off + db * 16];
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(vp + 16 * kVS));
            const i16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            oacc[db] = Mma16<T>::run(a, pb, oacc[db]);
        }
        if (t + 1 < n_tiles) {
            store_v(buf ^ 1);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) kcur[kb][ks] = knext[kb][ks];
        }
    }

    // ---- merge the 4 waves: O^T lane (query lq, group lg) holds d = 16*db + 4*lg + r
    const float l_wave = group_sum(l_run);
    __syncthreads();  // everyone is done with the V tiles
    float* o_lds = reinterpret_cast<float*>(&v_lds[0][0][0]);  // [wave][16][D] floats: 32 KB / 16 KB, inside the V tiles' space
    static_assert(sizeof(float) * kWaves * kMaxRows * D <= sizeof(std::uint16_t) * kWaves * 2 * kTile * kVS, "merge space");
    if (lq < p.R) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_lds[(wave * kMaxRows + lq) * kD + 16 * db + 4 * lg + r] = oacc[db][r];
        if (lg == 0) {
            m_lds[wave][lq] = m_run;
            l_lds[wave][lq] = l_wave;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < p.R * kD; idx += kThreads) {
        const int r = idx / kD, d = idx % kD;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) M = fmaxf(M, m_lds[w][r]);
        float L = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float mw = m_lds[w][r];
            const float f = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mw - M) * p.scale_log2);
            L += l_lds[w][r] * f;
            O += o_lds[(w * kMaxRows + r) * kD + d] * f;
        }
        if (p.splits == 1) {
            const int gi = r / p.Lq, qi = r % p.Lq;
            const long orow = (static_cast<long>(b) * p.Hq + hkv * p.G + gi) * p.Lq + qi;
            const float val = O / L;
            p.out[orow * kD + d] = static_cast<std::uint16_t>(Mma16<T>::pack2(val, 0.f) & 0xffffu);
            if (p.lse && d == 0) p.lse[orow] = M * p.scale + logf(L);
        } else {
            const long slot = static_cast<long>(pair) * p.splits + split;
            p.part_o[(slot * kMaxRows + r) * kD + d] = O;
            if (d == 0) {
                p.part_ml[(slot * 2 + 0) * kMaxRows + r] = M;
                p.part_ml[(slot * 2 + 1) * kMaxRows + r] = L;
            }
        }
    }
}

// One workgroup of D threads (one per d) per (pair, query row).
template <typename T, int D>
__global__ __launch_bounds__(D) void decode_combine_kernel(const DecodeParams p) {
    constexpr int kD = D;
    const int pair = blockIdx.x, r = blockIdx.y, d = threadIdx.x;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv;
    // (both loops unrolled by eight: the loads of eight splits are in flight together, not one
    // round trip to L2 per split)
    float M = -INFINITY;
#pragma unroll 8
    for (int s = 0; s < p.splits; ++s) M = fmaxf(M, p.part_ml[((static_cast<long>(pair) * p.splits + s) * 2) * kMaxRows + r]);
    float L = 0.f, O = 0.f;
#pragma unroll 8
    for (int s = 0; s < p.splits; ++s) {
        const long slot = static_cast<long>(pair) * p.splits + s;
        const float ms = p.part_ml[(slot * 2) * kMaxRows + r];
        const float f = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((ms - M) * p.scale_log2);
        L += p.part_ml[(slot * 2 + 1) * kMaxRows + r] * f;
        O += p.part_o[(slot * kMaxRows + r) * kD + d] * f;
    }
    const int gi = r / p.Lq, qi = r % p.Lq;
    const long orow = (static_cast<long>(b) * p.Hq + hkv * p.G + gi) * p.Lq + qi;
    p.out[orow * kD + d] = static_cast<std::uint16_t>(Mma16<T>::pack2(O / L, 0.f) & 0xffffu);
    if (p.lse && d == 0) p.lse[orow] = M * p.scale + logf(L);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool mult8(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

// Split count: about two workgroups per CU in all (measured over batch 1 ... 256 and 512 ... 131072
// keys: more splits than that only add partial results for the combine kernel to read, fewer leave
// CUs idle), each wave keeping at least two tiles.  A large batch fills the chip without any split.
void plan(const paras_sdpa_args& a, int* splits, int* chunk) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto* st = DeviceContext::instance().device(dev);
    const long cus = st ? st->compute_units : 256;
    const long pairs = a.B * a.Hkv;
    const long unit = kWaves * kTile;                        // 128 keys: one tile per wave
    const long max_splits = (a.Lk + 2 * unit - 1) / (2 * unit);  // >= 2 tiles per wave
    long want = (cus * 2 + pairs - 1) / pairs;
    if (want > max_splits) want = max_splits;
    if (want < 1) want = 1;
    long ch = (a.Lk + want - 1) / want;
    ch = (ch + unit - 1) / unit * unit;
    *chunk = static_cast<int>(ch);
    *splits = static_cast<int>((a.Lk + ch - 1) / ch);
}

}  // namespace

bool decode_supported(const paras_sdpa_args& a) {
    if (a.dtype != PARAS_BF16 && a.dtype != PARAS_F16) return false;
    if (a.D != a.Dv || (a.D != 64 && a.D != 128 && a.D != 256)) return false;
    if (a.attn != nullptr || a.is_causal) return false;
    if (a.mask_kind != 0 && (a.mask == nullptr || a.mask_kind > 2)) return false;
    if (a.Hkv < 1 || a.Hq % a.Hkv != 0) return false;
    const int64_t rows = a.Lq * (a.Hq / a.Hkv);
    if (rows < 1 || rows > kMaxRows) return false;
    if (a.Lk < 1 || a.Lk > 0x3fffffff || a.B * a.Hkv > 65535) return false;
    if (!(a.scale > 0.0) || !std::isfinite(a.scale)) return false;
    if (!aligned16(a.q) || !aligned16(a.k) || !aligned16(a.v)) return false;
    if (!mult8(a.q_strides) || !mult8(a.k_strides) || !mult8(a.v_strides)) return false;
    return true;
}

size_t decode_workspace(const paras_sdpa_args& a) {
    int splits = 1, chunk = 0;
    plan(a, &splits, &chunk);
    if (splits == 1) return 0;
    const size_t slots = static_cast<size_t>(a.B * a.Hkv) * splits;
    return slots * (kMaxRows * a.D + 2 * kMaxRows) * sizeof(float);
}

int launch_decode(const paras_sdpa_args& a, void* workspace, hipStream_t s) {
    DecodeParams p;
    p.q = static_cast<const std::uint16_t*>(a.q);
    p.k = static_cast<const std::uint16_t*>(a.k);
    p.v = static_cast<const std::uint16_t*>(a.v);
    p.out = static_cast<std::uint16_t*>(a.out);
    p.lse = a.lse;
    p.qs_b = a.q_strides[0]; p.qs_h = a.q_strides[1]; p.qs_l = a.q_strides[2];
    p.ks_b = a.k_strides[0]; p.ks_h = a.k_strides[1]; p.ks_l = a.k_strides[2];
    p.vs_b = a.v_strides[0]; p.vs_h = a.v_strides[1]; p.vs_l = a.v_strides[2];
    p.B = (int)a.B; p.Hq = (int)a.Hq; p.Hkv = (int)a.Hkv; p.Lq = (int)a.Lq; p.Lk = (int)a.Lk;
    p.G = (int)(a.Hq / a.Hkv);
    p.R = p.G * p.Lq;
    plan(a, &p.splits, &p.chunk);
    p.scale = static_cast<float>(a.scale);
    p.scale_log2 = static_cast<float>(a.scale * 1.4426950408889634);
    const size_t slots = static_cast<size_t>(a.B * a.Hkv) * p.splits;
    p.part_o = static_cast<float*>(workspace);
    p.part_ml = p.part_o ? p.part_o + slots * kMaxRows * a.D : nullptr;
    const dim3 grid(p.splits, static_cast<unsigned>(a.B * a.Hkv));
    p.mask = static_cast<const unsigned char*>(a.mask);
    p.ms_b = a.mask_strides[0]; p.ms_h = a.mask_strides[1]; p.ms_q = a.mask_strides[2]; p.ms_k = a.mask_strides[3];
    p.inv_scale = static_cast<float>(1.0 / a.scale);
    const bool bf = a.dtype == PARAS_BF16;
    const dim3 block(kThreads);
    const dim3 g2(static_cast<unsigned>(a.B * a.Hkv), p.R);
#define PARAS_DECODE_LAUNCH(T_, D_)                                                                        \
    do {                                                                                                   \
        if (a.mask_kind == 0)      hipLaunchKernelGGL((decode_split_kernel<T_, D_, 0>), grid, block, 0, s, p); \
        else if (a.mask_kind == 1) hipLaunchKernelGGL((decode_split_kernel<T_, D_, 1>), grid, block, 0, s, p); \
        else                       hipLaunchKernelGGL((decode_split_kernel<T_, D_, 2>), grid, block, 0, s, p); \
        PARAS_HIP_TRY(hipGetLastError());                                                                  \
        if (p.splits > 1) {                                                                                \
            hipLaunchKernelGGL((decode_combine_kernel<T_, D_>), g2, dim3(D_), 0, s, p);                    \
            PARAS_HIP_TRY(hipGetLastError());                                                              \
        }                                                                                                  \
    } while (0)
    if (a.D == 256) {
        if (bf) PARAS_DECODE_LAUNCH(bf16_t, 256);
        else    PARAS_DECODE_LAUNCH(f16_t, 256);
    } else if (a.D == 128) {
        if (bf) PARAS_DECODE_LAUNCH(bf16_t, 128);
        else    PARAS_DECODE_LAUNCH(f16_t, 128);
    } else {
        if (bf) PARAS_DECODE_LAUNCH(bf16_t, 64);
        else    PARAS_DECODE_LAUNCH(f16_t, 64);
    }
#undef PARAS_DECODE_LAUNCH
    return PARAS_OK;
}

}  // namespace paras
