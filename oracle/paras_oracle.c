/*
 * paras_oracle.c -- CPU restatement of the arithmetic of Torch-ParaS's host
 * engine ("paras:0") for the fused transformer hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (libparas_hip.so, _C.so,
 * the torch_paras package) links, loads or calls this file.  It is used by
 * tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, as
 * the checker and as the timed CPU baseline -- never as the thing shipped.
 *
 * Each function cites the reference lines it restates (paths relative to the
 * reference tree).  The common rule of that engine: load the element, widen
 * to double, evaluate in double, narrow once to the tensor dtype.  Narrowing
 * to bf16/fp16 goes double -> float -> 16-bit (c10::BFloat16 and c10::Half
 * only have float constructors), so there are two roundings; both are kept.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   every function below is compared bit for bit with the reference's own
 *   CPU flavor built from its sources (oracle/_ref, oracle/Makefile.ref) on
 *   seeded inputs, and independently against closed forms / torch-CPU library
 *   routines / brute force (the checks the reference's own tests make:
 *   tests/test_fused_ops.py, tests/test_attention_norm_ops.py,
 *   tests/test_pointwise_ops.py:224-267,369-413,
 *   tests/test_matmul_sort_creation_ops.py:133-139).
 *   po_matmul_nt is the exception: the reference bounces GEMMs to ATen-CPU
 *   (csrc/ops/vision_ops.cpp:388-406; libtorch_cpu, third party, pinned
 *   torch==2.5.1 in docs/INSTALL.md:34), whose blocking order is not part of
 *   the reference.  Here it accumulates in double and rounds once; for bf16 /
 *   fp16 operands its last-bit agreement with ATen is "parity unpinned" (the
 *   reference's GEMM tests are fp32-only at 1e-4).
 *
 * Build: gcc -O2 -fPIC -shared -std=c11 -fopenmp -ffp-contract=off
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { PO_F32 = 0, PO_F16 = 1, PO_BF16 = 2, PO_F64 = 3 };

/* ------------------------------------------------------------------------- */
/* dtype conversion, as c10 does it on the host                              */
/* ------------------------------------------------------------------------- */
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* c10::detail::round_to_nearest_even (c10/util/BFloat16.h) */
static inline uint16_t f32_to_bf16(float f) {
    if (isnan(f)) return 0x7FC0;
    uint32_t u = f32_bits(f);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static inline float bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* IEEE binary16 <-> binary32, round to nearest even (what c10::Half does,
 * in software or with F16C). */
static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        float v = ldexpf((float)man, -24);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}
static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);          /* NaN  */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);         /* >= 65536 -> inf (also true inf) */
    if (a < 0x33000000u) return sign;                                 /* < 2^-25 -> 0 */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
    int shift = e < -14 ? (13 + (-14 - e)) : 13;                      /* bits dropped */
    uint32_t keep = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) keep++;
    uint32_t out;
    if (e < -14) out = keep;                                          /* subnormal (may carry into normal) */
    else out = ((uint32_t)(e + 15) << 10) + (keep - 0x400u);          /* carry propagates into exponent */
    if (out >= 0x7C00u) out = 0x7C00u;
    return (uint16_t)(sign | out);
}

static inline double ld(const void* p, long i, int dt) {
    switch (dt) {
        case PO_F32:  return (double)((const float*)p)[i];
        case PO_F64:  return ((const double*)p)[i];
        case PO_BF16: return (double)bf16_to_f32(((const uint16_t*)p)[i]);
        default:      return (double)f16_to_f32(((const uint16_t*)p)[i]);
    }
}
static inline void st(void* p, long i, int dt, double v) {
    switch (dt) {
        case PO_F32:  ((float*)p)[i] = (float)v; break;
        case PO_F64:  ((double*)p)[i] = v; break;
        case PO_BF16: ((uint16_t*)p)[i] = f32_to_bf16((float)v); break;
        default:      ((uint16_t*)p)[i] = f32_to_f16((float)v); break;
    }
}
/* value of a double after one trip through the tensor dtype */
static inline double rnd(double v, int dt) {
    switch (dt) {
        case PO_F32:  return (double)(float)v;
        case PO_F64:  return v;
        case PO_BF16: return (double)bf16_to_f32(f32_to_bf16((float)v));
        default:      return (double)f16_to_f32(f32_to_f16((float)v));
    }
}
double po_round_to_dtype(double v, int dt) { return rnd(v, dt); }

/* ------------------------------------------------------------------------- */
/* Host execution engine: host_parallel_chunks                               */
/* (csrc/compat/paras_compat.cpp:142-195): serial when n <= grain or one     */
/* thread; else chunks = min(threads, ceil(n/grain)) equal slices claimed     */
/* dynamically by the team.                                                   */
/* ------------------------------------------------------------------------- */
static int  g_threads = 0;        /* 0 = omp_get_max_threads() */
static long g_grain   = 16384;

void po_set_threads(int n) { g_threads = n; }
int  po_get_threads(void) { return g_threads > 0 ? g_threads : omp_get_max_threads(); }
void po_set_grain(long g) { if (g > 0) g_grain = g; }

typedef void (*chunk_fn)(void* ctx, long begin, long end);

static void parallel_chunks(long n, chunk_fn body, void* ctx) {
    if (n <= 0) return;
    const long threads = po_get_threads();
    if (threads <= 1 || n <= g_grain) { body(ctx, 0, n); return; }
    long chunks = (n + g_grain - 1) / g_grain;
    if (chunks > threads) chunks = threads;
    const long per = (n + chunks - 1) / chunks;
    long next = 0;
#pragma omp parallel num_threads((int)chunks)
    {
        for (;;) {
            long c;
#pragma omp atomic capture
            c = next++;
            if (c >= chunks) break;
            long b = c * per, e = b + per < n ? b + per : n;
            if (b < e) body(ctx, b, e);
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Fused RMSNorm  (csrc/ops/fused_ops.cpp:67-85)                              */
/* one work item per row; ss sequential over j in double                     */
/* ------------------------------------------------------------------------- */
typedef struct { const void *x, *w; void* out; float* rstd; long H; double eps; int dt; } rms_ctx;
static void rms_body(void* c_, long b, long e) {
    rms_ctx* c = (rms_ctx*)c_;
    for (long r = b; r < e; ++r) {
        const long base = r * c->H;
        double ss = 0.0;
        for (long j = 0; j < c->H; ++j) { const double v = ld(c->x, base + j, c->dt); ss += v * v; }
        const double rms = 1.0 / sqrt(ss / (double)c->H + c->eps);
        c->rstd[r] = (float)rms;
        for (long j = 0; j < c->H; ++j)
            st(c->out, base + j, c->dt, ld(c->x, base + j, c->dt) * rms * ld(c->w, j, c->dt));
    }
}
void po_rms_norm(const void* x, const void* w, void* out, float* rstd, long rows, long H, double eps, int dt) {
    if (rows == 0 || H == 0) return;                       /* fused_ops.cpp:57 */
    rms_ctx c = {x, w, out, rstd, H, eps, dt};
    parallel_chunks(rows, rms_body, &c);
}

/* rms_norm_backward (csrc/ops/fused_ops.cpp:105-156) */
typedef struct { const void *go, *x, *w; const float* rstd; void *gx, *gw; long rows, H; int dt; } rmsb_ctx;
static void rmsb_dx_body(void* c_, long b, long e) {
    rmsb_ctx* c = (rmsb_ctx*)c_;
    for (long r = b; r < e; ++r) {
        const long base = r * c->H;
        const double rr = (double)c->rstd[r];
        double dot = 0.0;
        for (long j = 0; j < c->H; ++j)
            dot += ld(c->go, base + j, c->dt) * ld(c->w, j, c->dt) * ld(c->x, base + j, c->dt);
        const double coef = rr * rr * rr / (double)c->H;
        for (long j = 0; j < c->H; ++j) {
            const double gj = ld(c->go, base + j, c->dt), wj = ld(c->w, j, c->dt), xj = ld(c->x, base + j, c->dt);
            st(c->gx, base + j, c->dt, gj * wj * rr - coef * xj * dot);
        }
    }
}
static void rmsb_dw_body(void* c_, long b, long e) {
    rmsb_ctx* c = (rmsb_ctx*)c_;
    for (long j = b; j < e; ++j) {
        double acc = 0.0;
        for (long r = 0; r < c->rows; ++r)
            acc += ld(c->go, r * c->H + j, c->dt) * ld(c->x, r * c->H + j, c->dt) * (double)c->rstd[r];
        st(c->gw, j, c->dt, acc);
    }
}
void po_rms_norm_bwd(const void* go, const void* x, const void* w, const float* rstd, void* gx, void* gw,
                     long rows, long H, int dt) {
    if (rows == 0 || H == 0) return;
    rmsb_ctx c = {go, x, w, rstd, gx, gw, rows, H, dt};
    parallel_chunks(rows, rmsb_dx_body, &c);
    parallel_chunks(H, rmsb_dw_body, &c);
}

/* ------------------------------------------------------------------------- */
/* Fused SwiGLU (csrc/ops/fused_ops.cpp:185-190) and backward (:218-226)      */
/* ------------------------------------------------------------------------- */
typedef struct { const void *a, *b, *c; void *o1, *o2; int dt; } ew_ctx;
static void swiglu_body(void* c_, long b, long e) {
    ew_ctx* c = (ew_ctx*)c_;
    for (long i = b; i < e; ++i) {
        const double g = ld(c->a, i, c->dt);
        const double s = g / (1.0 + exp(-g));
        st(c->o1, i, c->dt, s * ld(c->b, i, c->dt));
    }
}
void po_swiglu(const void* gate, const void* up, void* out, long n, int dt) {
    ew_ctx c = {gate, up, NULL, out, NULL, dt};
    parallel_chunks(n, swiglu_body, &c);
}
static void swiglub_body(void* c_, long b, long e) {
    ew_ctx* c = (ew_ctx*)c_;
    for (long i = b; i < e; ++i) {
        const double dy = ld(c->a, i, c->dt), g = ld(c->b, i, c->dt), u = ld(c->c, i, c->dt);
        const double s = 1.0 / (1.0 + exp(-g));
        st(c->o2, i, c->dt, dy * g * s);                               /* grad_up   */
        st(c->o1, i, c->dt, dy * u * (s * (1.0 + g * (1.0 - s))));    /* grad_gate */
    }
}
void po_swiglu_bwd(const void* go, const void* gate, const void* up, void* ggate, void* gup, long n, int dt) {
    ew_ctx c = {go, gate, up, ggate, gup, dt};
    parallel_chunks(n, swiglub_body, &c);
}

/* rotate_half / backward (csrc/ops/fused_ops.cpp:254-263, 290-299) */
void po_rotate_half(const void* x, void* out, long rows, long D, int backward, int dt) {
    const long half = D / 2, n = rows * D;
    for (long flat = 0; flat < n; ++flat) {
        const long col = flat % D;
        const long src = flat - col + (col < half ? col + half : col - half);
        const int negate = backward ? !(col < half) : (col < half);
        if (negate) st(out, flat, dt, -ld(x, src, dt));
        else if (dt == PO_F32) ((float*)out)[flat] = ((const float*)x)[src];
        else if (dt == PO_F64) ((double*)out)[flat] = ((const double*)x)[src];
        else ((uint16_t*)out)[flat] = ((const uint16_t*)x)[src];
    }
}

/* ------------------------------------------------------------------------- */
/* Elementwise primitives (unary_kernel / binary_kernel,                      */
/* csrc/ops/pointwise_ops.cpp:33-85): operands are already in the output      */
/* dtype (to_compute, :55-60, casts a wrapped scalar to it first), flat and   */
/* the same length; broadcasting is done by the caller.                       */
/* ------------------------------------------------------------------------- */
enum { PO_OP_ADD = 0, PO_OP_MUL = 1, PO_OP_DIV = 2, PO_OP_SUB = 3 };
typedef struct { const void *a, *b; void* o; int op; double alpha; int dt; } bin_ctx;
static void bin_body(void* c_, long b, long e) {
    bin_ctx* c = (bin_ctx*)c_;
    for (long i = b; i < e; ++i) {
        const double x = ld(c->a, i, c->dt), y = ld(c->b, i, c->dt);
        double r;
        switch (c->op) {
            case PO_OP_ADD: r = x + c->alpha * y; break;   /* add_out :259-265 */
            case PO_OP_SUB: r = x - c->alpha * y; break;
            case PO_OP_MUL: r = x * y; break;              /* mul_out :280-284 */
            default:        r = x / y; break;
        }
        st(c->o, i, c->dt, r);
    }
}
void po_binary(int op, const void* a, const void* b, void* out, long n, double alpha, int dt) {
    bin_ctx c = {a, b, out, op, alpha, dt};
    parallel_chunks(n, bin_body, &c);
}
/* tensor (op) scalar: the scalar is narrowed to the tensor dtype before the
 * double evaluation (to_compute :55-60), e.g. bf16(1/sqrt(128)) = 0.08837890625 */
typedef struct { const void* a; void* o; int op; double s, alpha; int dt; } bins_ctx;
static void bins_body(void* c_, long b, long e) {
    bins_ctx* c = (bins_ctx*)c_;
    for (long i = b; i < e; ++i) {
        const double x = ld(c->a, i, c->dt);
        double r;
        switch (c->op) {
            case PO_OP_ADD: r = x + c->alpha * c->s; break;
            case PO_OP_SUB: r = x - c->alpha * c->s; break;
            case PO_OP_MUL: r = x * c->s; break;
            default:        r = x / c->s; break;
        }
        st(c->o, i, c->dt, r);
    }
}
void po_binary_scalar(int op, const void* a, double scalar, void* out, long n, double alpha, int dt) {
    bins_ctx c = {a, out, op, rnd(scalar, dt), alpha, dt};
    parallel_chunks(n, bins_body, &c);
}

enum { PO_UN_POW = 0, PO_UN_RSQRT = 1, PO_UN_SILU = 2, PO_UN_SCALE = 3 };
typedef struct { const void* a; void* o; int op; double p; int dt; } un_ctx;
static void un_body(void* c_, long b, long e) {
    un_ctx* c = (un_ctx*)c_;
    for (long i = b; i < e; ++i) {
        const double v = ld(c->a, i, c->dt);
        double r;
        switch (c->op) {
            case PO_UN_POW:   r = pow(v, c->p); break;                 /* pow_scalar_out :403-407 */
            case PO_UN_RSQRT: r = 1.0 / sqrt(v); break;                /* rsqrt_out :370-373 */
            case PO_UN_SILU:  r = v / (1.0 + exp(-v)); break;          /* silu_out :460-464 */
            default:          r = v * c->p; break;                     /* post_scale of mean, :216-219 */
        }
        st(c->o, i, c->dt, r);
    }
}
void po_unary(int op, const void* a, void* out, long n, double param, int dt) {
    un_ctx c = {a, out, op, param, dt};
    parallel_chunks(n, un_body, &c);
}

/* masked_fill_ with a scalar (csrc/ops/scatter_ops.cpp:43-71): where mask is
 * nonzero the element becomes value narrowed to the dtype. */
void po_masked_fill(void* data, const uint8_t* mask, double value, long n, int dt) {
    for (long i = 0; i < n; ++i) if (mask[i]) st(data, i, dt, value);
}
/* tril of an all-ones bool [Lq, Lk] (csrc/ops/indexing_ops.cpp:533-579):
 * keep (col - row) <= diagonal.  Writes 1 where kept. */
void po_tril_ones(uint8_t* out, long Lq, long Lk, long diagonal) {
    for (long r = 0; r < Lq; ++r)
        for (long c = 0; c < Lk; ++c) out[r * Lk + c] = (uint8_t)((c - r) <= diagonal);
}

/* Sum over the last (contiguous) dim: reduce_outer with double accumulator,
 * sequential j, narrowed to the dtype (csrc/ops/pointwise_ops.cpp:168-225,
 * csrc/core/kernels.h:134-144).  The reduce_full branch (out_n <= 64 and
 * red_n >= 65536) adds 1024 strided partial sums and then the partials in
 * order (kernels.h:109-132). */
typedef struct { const void* in; void* out; long red_n; int dt; } sum_ctx;
static void sum_body(void* c_, long b, long e) {
    sum_ctx* c = (sum_ctx*)c_;
    for (long o = b; o < e; ++o) {
        double acc = 0.0;
        for (long j = 0; j < c->red_n; ++j) acc = acc + ld(c->in, o * c->red_n + j, c->dt);
        st(c->out, o, c->dt, acc);
    }
}
void po_sum_last(const void* in, void* out, long out_n, long red_n, int dt) {
    if (out_n <= 64 && red_n >= 65536) {
        for (long o = 0; o < out_n; ++o) {
            const long stripes = red_n < 1024 ? red_n : 1024;
            double result = 0.0;
            for (long s = 0; s < stripes; ++s) {
                double acc = 0.0;
                for (long i = s; i < red_n; i += stripes) acc = acc + ld(in, o * red_n + i, dt);
                result = result + acc;
            }
            st(out, o, dt, result);
        }
        return;
    }
    sum_ctx c = {in, out, red_n, dt};
    parallel_chunks(out_n, sum_body, &c);
}
/* Sum over a middle dim of a contiguous [outer, red, inner] tensor (the MoE
 * combine sums the k slots of [T, k, H]); same accumulator rule. */
typedef struct { const void* in; void* out; long red_n, inner; int dt; } summ_ctx;
static void summ_body(void* c_, long b, long e) {
    summ_ctx* c = (summ_ctx*)c_;
    for (long o = b; o < e; ++o) {
        const long outer = o / c->inner, in_ = o % c->inner;
        double acc = 0.0;
        for (long j = 0; j < c->red_n; ++j) acc = acc + ld(c->in, (outer * c->red_n + j) * c->inner + in_, c->dt);
        st(c->out, o, c->dt, acc);
    }
}
void po_sum_mid(const void* in, void* out, long outer, long red_n, long inner, int dt) {
    summ_ctx c = {in, out, red_n, inner, dt};
    parallel_chunks(outer * inner, summ_body, &c);
}

/* _softmax over the last dim (csrc/ops/pointwise_ops.cpp:954-977): max, then
 * sum of exp(v-m), then exp(v-m)/sum, all in double; one work item per row. */
typedef struct { const void* in; void* out; long n; int dti, dto; } sm_ctx;
static void sm_body(void* c_, long b, long e) {
    sm_ctx* c = (sm_ctx*)c_;
    for (long o = b; o < e; ++o) {
        const long base = o * c->n;
        double m = -INFINITY;
        for (long j = 0; j < c->n; ++j) { const double v = ld(c->in, base + j, c->dti); if (v > m) m = v; }
        double sum = 0.0;
        for (long j = 0; j < c->n; ++j) sum += exp(ld(c->in, base + j, c->dti) - m);
        for (long j = 0; j < c->n; ++j) st(c->out, base + j, c->dto, exp(ld(c->in, base + j, c->dti) - m) / sum);
    }
}
void po_softmax_last(const void* in, void* out, long rows, long n, int dt_in, int dt_out) {
    sm_ctx c = {in, out, n, dt_in, dt_out};
    parallel_chunks(rows, sm_body, &c);
}

/* topk over the last dim (csrc/ops/pointwise_ops.cpp:1325-1378): k selection
 * scans, each bounded by the previous (value, index); ties go to the lower
 * index; output sorted. */
typedef struct { const void* in; void* vals; int64_t* idx; long n, k; int largest, dt; } tk_ctx;
static void tk_body(void* c_, long b, long e) {
    tk_ctx* c = (tk_ctx*)c_;
    for (long o = b; o < e; ++o) {
        double prev_val = 0.0; long prev_idx = -1; int has_prev = 0;
        for (long s = 0; s < c->k; ++s) {
            double best_val = 0.0; long best_idx = -1; int has_best = 0;
            for (long j = 0; j < c->n; ++j) {
                const double v = ld(c->in, o * c->n + j, c->dt);
                int within;
                if (!has_prev) within = 1;
                else if (c->largest) within = (v < prev_val) || (v == prev_val && j > prev_idx);
                else within = (v > prev_val) || (v == prev_val && j > prev_idx);
                if (!within) continue;
                int better;
                if (!has_best) better = 1;
                else if (c->largest) better = (v > best_val) || (v == best_val && j < best_idx);
                else better = (v < best_val) || (v == best_val && j < best_idx);
                if (better) { best_val = v; best_idx = j; has_best = 1; }
            }
            st(c->vals, o * c->k + s, c->dt, best_val);
            c->idx[o * c->k + s] = best_idx;
            prev_val = best_val; prev_idx = best_idx; has_prev = 1;
        }
    }
}
void po_topk_last(const void* in, long rows, long n, long k, int largest, void* vals, int64_t* idx, int dt) {
    if (rows == 0 || k == 0) return;
    tk_ctx c = {in, vals, idx, n, k, largest, dt};
    parallel_chunks(rows, tk_body, &c);
}

/* argsort(stable=True) of one int64 row, ascending (csrc/ops/sort_ops.cpp:
 * 129-166: std::stable_sort on the index vector).  A stable merge sort. */
static void merge_sort_idx(const int64_t* key, int64_t* idx, int64_t* tmp, long n) {
    for (long width = 1; width < n; width *= 2) {
        for (long lo = 0; lo < n; lo += 2 * width) {
            long mid = lo + width < n ? lo + width : n, hi = lo + 2 * width < n ? lo + 2 * width : n;
            long i = lo, j = mid, o = lo;
            while (i < mid && j < hi) tmp[o++] = (key[idx[j]] < key[idx[i]]) ? idx[j++] : idx[i++];
            while (i < mid) tmp[o++] = idx[i++];
            while (j < hi) tmp[o++] = idx[j++];
        }
        memcpy(idx, tmp, (size_t)n * sizeof(int64_t));
    }
}
void po_argsort_stable_i64(const int64_t* key, int64_t* out, long n) {
    int64_t* tmp = (int64_t*)malloc((size_t)(n > 0 ? n : 1) * sizeof(int64_t));
    for (long i = 0; i < n; ++i) out[i] = i;
    merge_sort_idx(key, out, tmp, n);
    free(tmp);
}

/* index_select of rows (csrc/ops/indexing_ops.cpp:98-152): out[i] = src[idx[i]] */
void po_index_select_rows(const void* src, const int64_t* idx, void* out, long nidx, long row_bytes) {
    for (long i = 0; i < nidx; ++i)
        memcpy((char*)out + i * row_bytes, (const char*)src + idx[i] * row_bytes, (size_t)row_bytes);
}

/* C[M,N] = A[M,K] * B[N,K]^T, double accumulate, one narrowing.  Stands in
 * for the ATen-CPU GEMM the reference bounces to (csrc/ops/vision_ops.cpp:
 * 388-406); see the header note on what pins it. */
void po_matmul_nt(const void* A, const void* B, void* C, long M, long N, long K, int dt) {
#pragma omp parallel for schedule(static) num_threads(po_get_threads())
    for (long m = 0; m < M; ++m)
        for (long n = 0; n < N; ++n) {
            double acc = 0.0;
            for (long k = 0; k < K; ++k) acc += ld(A, m * K + k, dt) * ld(B, n * K + k, dt);
            st(C, m * N + n, dt, acc);
        }
}
/* C[M,N] = A[M,K] * B[K,N] */
void po_matmul_nn(const void* A, const void* B, void* C, long M, long N, long K, int dt) {
#pragma omp parallel for schedule(static) num_threads(po_get_threads())
    for (long m = 0; m < M; ++m)
        for (long n = 0; n < N; ++n) {
            double acc = 0.0;
            for (long k = 0; k < K; ++k) acc += ld(A, m * K + k, dt) * ld(B, k * N + n, dt);
            st(C, m * N + n, dt, acc);
        }
}
