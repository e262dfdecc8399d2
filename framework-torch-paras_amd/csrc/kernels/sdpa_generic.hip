// General scaled-dot-product attention for gfx950: any dtype (fp32, fp64,
// bf16, fp16), any head size, bool / additive masks, causal, GQA, and the
// optional [B,Hq,Lq,Lk] weights the math op returns.
//
// This kernel follows the reference's composed path step by step
// (csrc/ops/attention_ops.cpp:101-135) and narrows to the tensor dtype where
// that path does, so its output and its weights agree with the host engine to
// the last bit wherever the summation order does not matter:
//   s  = T(sum_d q*k)                    bmm result (vision_ops.cpp:398-406)
//   s  = T(s * scale)                    mul.out (pointwise_ops.cpp:280-284)
//   s  = -inf where masked / T(s + bias) masked_fill / add
//   p  = T(exp(s - max) / sum exp)       _softmax, fp64 (pointwise_ops.cpp:954-977)
//   o  = T(sum_j p*v)                    second bmm
// All arithmetic is fp64 (78 TFLOP/s of it on this part; this path serves
// small and unusual shapes, the large regular ones go to the MFMA kernels).
//
// One 256-thread workgroup per (batch, head, query) row.  Scores are not
// stored: pass 1 finds the row max, pass 2 the denominator, pass 3 recomputes
// each score, writes the weights (if asked) and accumulates p*v with threads
// spread over the head dim, staging kChunk probabilities at a time in LDS.
#include <hip/hip_runtime.h>

#include <cmath>

#include "core/device_math.h"
#include "core/status.h"
#include "kernels/sdpa_internal.h"

namespace paras {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kChunk = 1024;  // keys staged per step of pass 3
constexpr int kMaxD  = 512;   // head dim of q held in LDS

struct GenericParams {
    const void* q; const void* k; const void* v; void* out; void* attn; float* lse;
    const void* mask;
    int mask_kind, is_causal;
    long B, Hq, Hkv, Lq, Lk, D, Dv;
    long qs[3], ks[3], vs[3], ms[4];
    double scale;
};

template <typename T>
__device__ __forceinline__ double narrow(double v) {
    return Elem<T>::to_f64(Elem<T>::from_f64(v));
}

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

template <typename T>
__global__ __launch_bounds__(kBlock) void sdpa_generic_kernel(const GenericParams p) {
    using E = Elem<T>;
    using S = typename E::store_t;
    __shared__ double qs[kMaxD];
    __shared__ double pbuf[kChunk];
    __shared__ double slots[kWaves];

    const long row = blockIdx.x;  // over B*Hq*Lq
    const long i = row % p.Lq;
    const long h = (row / p.Lq) % p.Hq;
    const long b = row / (p.Lq * p.Hq);
    const long hkv = h / (p.Hq / p.Hkv);
    const int tid = threadIdx.x;

    const S* qrow = static_cast<const S*>(p.q) + b * p.qs[0] + h * p.qs[1] + i * p.qs[2];
    const S* kb = static_cast<const S*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
    const S* vb = static_cast<const S*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
    for (long d = tid; d < p.D; d += kBlock) qs[d] = E::to_f64(qrow[d]);
    __syncthreads();

    const double scale = p.scale;
    const long mrow = b * p.ms[0] + h * p.ms[1] + i * p.ms[2];
    const double ninf = -INFINITY;

    auto score = [&](long j) -> double {
        const S* kr = kb + j * p.ks[2];
        double acc = 0.0;
        for (long d = 0; d < p.D; ++d) acc += qs[d] * E::to_f64(kr[d]);
        double s = narrow<T>(acc);
        s = narrow<T>(s * scale);
        if (p.is_causal) {
            if (j > i) s = ninf;
        } else if (p.mask_kind == 1) {
            if (static_cast<const unsigned char*>(p.mask)[mrow + j * p.ms[3]] == 0) s = ninf;
        } else if (p.mask_kind == 2) {
            s = narrow<T>(s + E::to_f64(static_cast<const S*>(p.mask)[mrow + j * p.ms[3]]));
        }
        return s;
    };

    // pass 1: row max
    double m = ninf;
    for (long j = tid; j < p.Lk; j += kBlock) m = fmax(m, score(j));
    m = block_reduce(m, slots, true);
    // pass 2: denominator
    double sum = 0.0;
    for (long j = tid; j < p.Lk; j += kBlock) sum += exp(score(j) - m);
    sum = block_reduce(sum, slots, false);

    // pass 3: weights and output
    S* arow = p.attn ? static_cast<S*>(p.attn) + row * p.Lk : nullptr;
    constexpr int kMaxDvPerThread = kMaxD / kBlock;
    double acc[kMaxDvPerThread];
#pragma unroll
    for (int r = 0; r < kMaxDvPerThread; ++r) acc[r] = 0.0;
    for (long c0 = 0; c0 < p.Lk; c0 += kChunk) {
        const long cn = p.Lk - c0 < kChunk ? p.Lk - c0 : kChunk;
        __syncthreads();
        for (long jj = tid; jj < cn; jj += kBlock) {
            const long j = c0 + jj;
            const S pw = E::from_f64(exp(score(j) - m) / sum);
            if (arow) arow[j] = pw;
            pbuf[jj] = E::to_f64(pw);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kMaxDvPerThread; ++r) {
            const long d = tid + r * kBlock;
            if (d < p.Dv) {
                double a = acc[r];
                for (long jj = 0; jj < cn; ++jj) a += pbuf[jj] * E::to_f64(vb[(c0 + jj) * p.vs[2] + d]);
                acc[r] = a;
            }
        }
    }
    S* orow = static_cast<S*>(p.out) + row * p.Dv;
#pragma unroll
    for (int r = 0; r < kMaxDvPerThread; ++r) {
        const long d = tid + r * kBlock;
        if (d < p.Dv) orow[d] = E::from_f64(acc[r]);
    }
    if (p.lse && tid == 0) p.lse[row] = static_cast<float>(m + log(sum));
}

}  // namespace

size_t generic_workspace(const paras_sdpa_args&) { return 0; }

int launch_generic(const paras_sdpa_args& a, void*, hipStream_t s) {
    if (a.D > kMaxD || a.Dv > kMaxD)
        return fail(PARAS_ERR_UNSUPPORTED, "paras sdpa: head dim %lld/%lld exceeds %d", (long long)a.D,
                    (long long)a.Dv, kMaxD);
    const long rows = a.B * a.Hq * a.Lq;
    if (rows > 0x7fffffffL) return fail(PARAS_ERR_UNSUPPORTED, "paras sdpa: too many query rows");
    GenericParams p;
    p.q = a.q; p.k = a.k; p.v = a.v; p.out = a.out; p.attn = a.attn; p.lse = a.lse; p.mask = a.mask;
    p.mask_kind = a.mask_kind; p.is_causal = a.is_causal;
    p.B = a.B; p.Hq = a.Hq; p.Hkv = a.Hkv; p.Lq = a.Lq; p.Lk = a.Lk; p.D = a.D; p.Dv = a.Dv;
    for (int i = 0; i < 3; ++i) { p.qs[i] = a.q_strides[i]; p.ks[i] = a.k_strides[i]; p.vs[i] = a.v_strides[i]; }
    for (int i = 0; i < 4; ++i) p.ms[i] = a.mask_strides[i];
    p.scale = a.scale;
    const dim3 grid(static_cast<unsigned>(rows)), block(kBlock);
    switch (a.dtype) {
        case PARAS_F32:  hipLaunchKernelGGL((sdpa_generic_kernel<float>), grid, block, 0, s, p); break;
        case PARAS_F64:  hipLaunchKernelGGL((sdpa_generic_kernel<double>), grid, block, 0, s, p); break;
        case PARAS_BF16: hipLaunchKernelGGL((sdpa_generic_kernel<bf16_t>), grid, block, 0, s, p); break;
        case PARAS_F16:  hipLaunchKernelGGL((sdpa_generic_kernel<f16_t>), grid, block, 0, s, p); break;
        default: return fail(PARAS_ERR_INVALID, "paras sdpa: unknown dtype %d", a.dtype);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // namespace paras
