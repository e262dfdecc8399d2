/*
 * paras_hip.h -- C ABI of libparas_hip.so: the MI355X (gfx950) device layer
 * behind the `paras` PyTorch device.
 *
 * Everything that crosses this boundary is a plain pointer, an integer or a
 * double; no torch / ATen / C++ types appear.  All device pointers are plain
 * HBM addresses obtained from paras_alloc() or from any other HIP allocation
 * of the same process.  `stream` is a hipStream_t passed as void* and used as
 * given on the calling thread's current HIP device (NULL is HIP's null
 * stream); paras_stream(device) hands out the context's own stream.  Launches
 * are asynchronous on that stream.
 *
 * Every function returns PARAS_OK (0) or a negative paras_status; the text of
 * the last failure on the calling thread is returned by paras_last_error().
 * Nothing here throws and nothing here falls back to the host: if no HIP
 * device or no gfx950 code object is usable the call fails.
 *
 * The reference (Torch-ParaS) has no C ABI: its ops are C++ functions in
 * anonymous namespaces registered with the PyTorch dispatcher, running on
 * `compat::Queue`.  Each entry point below names the reference function whose
 * arithmetic it replaces (paths relative to the reference tree).
 */
#ifndef PARAS_HIP_H
#define PARAS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PARAS_API __attribute__((visibility("default")))

typedef enum paras_status {
    PARAS_OK              = 0,
    PARAS_ERR_INVALID     = -1, /* bad argument (shape, dtype, null pointer)   */
    PARAS_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for  */
    PARAS_ERR_HIP         = -3, /* a HIP runtime call failed                   */
    PARAS_ERR_NO_DEVICE   = -4, /* no usable HIP device                        */
    PARAS_ERR_OOM         = -5  /* hipMalloc failed                            */
} paras_status;

/* Element types.  Values are part of the ABI. */
typedef enum paras_dtype {
    PARAS_F32  = 0,
    PARAS_F16  = 1,
    PARAS_BF16 = 2,
    PARAS_F64  = 3
} paras_dtype;

/* ------------------------------------------------------------------------- */
/* Library / error state                                                     */
/* ------------------------------------------------------------------------- */

/* Text of the last error raised on the calling thread ("" if none). */
PARAS_API const char* paras_last_error(void);

/* ABI version of this header (bumped on any incompatible change). */
PARAS_API int paras_abi_version(void);

/* ------------------------------------------------------------------------- */
/* Device context (replaces compat::enumerate_devices / compat::Queue,        */
/* csrc/compat/paras_compat.h:69-221, and Context, csrc/core/context.h:43-74) */
/* Device i is HIP device i.  One non-blocking stream per device.            */
/* ------------------------------------------------------------------------- */

/* Number of HIP devices; 0 (never an error) when none is visible. */
PARAS_API int paras_device_count(void);

/* Copies the device's marketing name into buf (NUL-terminated, truncated). */
PARAS_API int paras_device_name(int device, char* buf, size_t buflen);

/* Compute-unit count and total HBM bytes of the device. */
PARAS_API int paras_device_info(int device, int* compute_units, uint64_t* hbm_bytes);

/* The context's stream for `device` (a hipStream_t), created on first use. */
PARAS_API int paras_stream(int device, void** stream_out);

/* 1 in a process forked after the context was built (HIP state does not
 * survive fork; csrc/core/context.cpp:33-38, 106-109), else 0. */
PARAS_API int paras_is_bad_fork(void);

/* Blocks until all work queued on the context stream of `device` is done
 * (Context::synchronize, csrc/core/context.cpp:69). */
PARAS_API int paras_synchronize(int device);

/* ------------------------------------------------------------------------- */
/* Binned HBM allocator (replaces MemoryPool, csrc/core/allocator.cpp:53-122) */
/* Same contract: request rounded up to a power of two, at least 256 bytes     */
/* (above 1 GiB: to a multiple of 256 MiB); freed blocks are cached per size   */
/* class unless PARAS_NO_CACHE=1; backing store is hipMalloc (device HBM,      */
/* never managed memory).                                                      */
/* ------------------------------------------------------------------------- */

PARAS_API int paras_alloc(int device, size_t nbytes, void** ptr_out);
/* Returns the block to the pool; an unknown pointer is PARAS_ERR_INVALID
 * (csrc/core/allocator.cpp:92-94). */
PARAS_API int paras_free(int device, void* ptr);
/* Synchronizes the device, then hipFree()s every cached block
 * (Context::empty_cache, csrc/core/context.cpp:96-100). */
PARAS_API int paras_empty_cache(int device);
/* Bytes held from hipMalloc (live + cached) and bytes sitting in the cache. */
PARAS_API int paras_memory_stats(int device, uint64_t* allocated, uint64_t* cached);
/* Size class a request of nbytes lands in (pure function, no device needed). */
PARAS_API size_t paras_round_size(size_t nbytes);

/* Copies (replace Queue::copy / Queue::memset, paras_compat.cpp:326-391).
 * kind: 0 host->device, 1 device->host, 2 device->device.  Host->device and
 * device->host copies return after the data has arrived; device->device
 * copies are queued on the context stream. */
PARAS_API int paras_memcpy(int device, void* dst, const void* src, size_t nbytes, int kind);
PARAS_API int paras_memset(int device, void* dst, int value, size_t nbytes);

/* Strided copy of an n-dimensional view (ndim <= 8), element strides, on the
 * given stream (replaces device_to_device_copy, csrc/ops/tensor_ops.cpp:
 * 211-250).  src_dtype == dst_dtype copies elem_size-byte elements of any
 * type; otherwise both must be paras_dtype float types and the copy narrows /
 * widens as static_cast does on the host. */
PARAS_API int paras_copy_strided(const void* src, void* dst, int ndim, const int64_t* sizes,
                                 const int64_t* src_strides, const int64_t* dst_strides,
                                 int elem_size, int src_dtype, int dst_dtype, void* stream);
/* Strided fill with one elem_size-byte value given as its bit pattern
 * (replaces fill_, csrc/ops/tensor_ops.cpp:333-370). */
PARAS_API int paras_fill_strided(void* dst, int ndim, const int64_t* sizes, const int64_t* strides,
                                 int elem_size, uint64_t value_bits, void* stream);

/* dst[o, i, :] = src[o, index[i], :] for a dense src seen as [outer, n_src,
 * inner_bytes] and int64 device indices (replaces index_select_out,
 * csrc/ops/indexing_ops.cpp:96-150; embedding lookups are dim 0).  Indices
 * outside [0, n_src) are clamped into it. */
PARAS_API int paras_index_select(const void* src, const int64_t* index, void* dst, int64_t outer,
                                 int64_t n_src, int64_t n_index, int64_t inner_bytes, void* stream);

/* Elementwise out = T(a op alpha*b) with broadcasting, evaluated as the host
 * engine does (replaces binary_kernel, csrc/ops/pointwise_ops.cpp:63-85, with
 * add_out :262-268, sub_out :271-277, mul_out :280-283, div_out :299-302).
 * op: 0 add, 1 sub, 2 mul, 3 div (alpha is used by add and sub only).  a and b
 * are views of the output's shape (element strides, 0 = broadcast); out is
 * dense; all three of the same paras_dtype float type. */
PARAS_API int paras_binary_strided(int op, const void* a, const void* b, void* out, int ndim,
                                   const int64_t* sizes, const int64_t* a_strides,
                                   const int64_t* b_strides, double alpha, int dtype, void* stream);

/* ------------------------------------------------------------------------- */
/* Fused RMSNorm (replaces ptsycl::rms_norm, csrc/ops/fused_ops.cpp:43-88)    */
/*   ss = sum_j x[r][j]^2 ; rstd[r] = 1/sqrt(ss/H + eps)                      */
/*   out[r][j] = T( x[r][j] * rstd[r] * w[j] )   (single rounding)            */
/* x, out: [rows, H] contiguous, dtype T; w: [H] dtype T; rstd: [rows] fp32.  */
/* rows == 0 or H == 0 is a no-op.                                            */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_rms_norm_fwd(const void* x, const void* w, void* out, float* rstd,
                                 int64_t rows, int64_t H, double eps, int dtype,
                                 void* stream);

/* (replaces ptsycl::rms_norm_backward, csrc/ops/fused_ops.cpp:90-157)
 *   dot = sum_j g*w*x ; dx = g*w*rstd - rstd^3/H * x * dot ;
 *   dw[j] = sum_r g[r][j]*x[r][j]*rstd[r]
 * `workspace` must hold paras_rms_norm_bwd_workspace(rows, H) bytes of device
 * memory (partial column sums). */
PARAS_API size_t paras_rms_norm_bwd_workspace(int64_t rows, int64_t H);
PARAS_API int paras_rms_norm_bwd(const void* grad_out, const void* x, const void* w,
                                 const float* rstd, void* grad_x, void* grad_w,
                                 void* workspace, int64_t rows, int64_t H, int dtype,
                                 void* stream);

/* ------------------------------------------------------------------------- */
/* Fused SwiGLU (replaces ptsycl::swiglu, csrc/ops/fused_ops.cpp:162-194)     */
/*   out[i] = T( gate[i]/(1+exp(-gate[i])) * up[i] ), contiguous, n elements  */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n,
                               int dtype, void* stream);

/* (replaces ptsycl::swiglu_backward, csrc/ops/fused_ops.cpp:196-229)
 *   s = sigmoid(g); dup = dy*g*s ; dgate = dy*u*s*(1+g*(1-s)) */
PARAS_API int paras_swiglu_bwd(const void* grad_out, const void* gate, const void* up,
                               void* grad_gate, void* grad_up, int64_t n, int dtype,
                               void* stream);

/* The composed forms, which narrow to the tensor dtype after every step:
 * aten::rms_norm over the trailing H elements of each row, w may be NULL
 * (replaces ptsycl::rms_norm, csrc/ops/rms_swiglu_ops.cpp:43-75:
 * pow(2) -> mean -> + eps -> rsqrt -> x * inv -> * w), and
 * torch_paras::swiglu(x, gate) = x * T(silu(gate))
 * (csrc/ops/rms_swiglu_ops.cpp:83-86). */
PARAS_API int paras_rms_norm_composed_fwd(const void* x, const void* w, void* out, int64_t rows,
                                          int64_t H, double eps, int dtype, void* stream);
PARAS_API int paras_swiglu_composed_fwd(const void* x, const void* gate, void* out, int64_t n,
                                        int dtype, void* stream);

/* ------------------------------------------------------------------------- */
/* rotate_half (replaces ptsycl::rotate_half(+_backward),                     */
/* csrc/ops/fused_ops.cpp:234-302): out = cat(-x2, x1) over the last dim D    */
/* (backward: cat(g2, -g1)).  x, out: [rows, D] contiguous, D even.           */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_rotate_half(const void* x, void* out, int64_t rows, int64_t D,
                                int backward, int dtype, void* stream);

/* ------------------------------------------------------------------------- */
/* Scaled dot-product attention forward                                       */
/* (replaces ptsycl::sdpa_math, csrc/ops/attention_ops.cpp:71-136, with its   */
/* GEMMs csrc/ops/vision_ops.cpp:398-406, its mask ops                        */
/* csrc/ops/indexing_ops.cpp:574-579 / csrc/ops/scatter_ops.cpp:43-71 and its */
/* softmax csrc/ops/pointwise_ops.cpp:926-981)                                */
/*   out = softmax(q k^T * scale + mask) v                                    */
/* Causal masking is top-left aligned: query i sees keys 0..i whatever Lk is  */
/* (attention_ops.cpp:103-116).  GQA: query head h reads kv head              */
/* h / (Hq/Hkv); K/V are never replicated.  A row whose keys are all masked   */
/* yields NaN, as the reference's softmax does.                               */
/* ------------------------------------------------------------------------- */
typedef struct paras_sdpa_args {
    const void* q;      /* [B, Hq,  Lq, D ]  last dim contiguous              */
    const void* k;      /* [B, Hkv, Lk, D ]                                   */
    const void* v;      /* [B, Hkv, Lk, Dv]                                   */
    void*       out;    /* [B, Hq,  Lq, Dv]  contiguous                       */
    void*       attn;   /* optional [B, Hq, Lq, Lk] contiguous, dtype of q:
                           the softmax weights the math op returns; NULL
                           skips them (needed for the flash kernels)          */
    float*      lse;    /* optional [B, Hq, Lq] natural-log sum-exp; or NULL  */
    const void* mask;   /* optional mask broadcast to [B, Hq, Lq, Lk]         */
    int32_t     mask_kind;      /* 0 none, 1 bool (1 byte, nonzero = attend),
                                   2 additive in the dtype of q               */
    int32_t     is_causal;      /* mutually exclusive with mask               */
    int32_t     dtype;          /* paras_dtype of q, k, v, out, attn          */
    int32_t     reserved;
    int64_t     B, Hq, Hkv, Lq, Lk, D, Dv;
    int64_t     q_strides[3];   /* element strides of dims B, H, L            */
    int64_t     k_strides[3];
    int64_t     v_strides[3];
    int64_t     mask_strides[4];/* element strides over B,Hq,Lq,Lk (0 = bcast)*/
    double      scale;          /* multiplies q k^T exactly as given          */
} paras_sdpa_args;

/* Scratch bytes the chosen kernel needs for these shapes (0 for most). */
PARAS_API size_t paras_sdpa_workspace(const paras_sdpa_args* args);
/* `workspace` may be NULL when paras_sdpa_workspace() returned 0. */
PARAS_API int paras_sdpa_fwd(const paras_sdpa_args* args, void* workspace, void* stream);
/* Name of the kernel paras_sdpa_fwd would pick: "flash_mfma" (bf16 / f16 heads of
 * 64, 128 or 256 elements; "flash_mfma_wide" where its 64-queries-per-wavefront
 * form runs: head size 128, no mask, at least two 256-query tiles per CU, rows of
 * 4096 causal / 1024 unmasked on), "decode_split" (heads of 64, 128 or 256),
 * "math_mfma" (bf16 / f16 with the weights returned), "padded_mfma" (bf16 / f16
 * head sizes below 256 other than 64 and 128: q, k, v copied into the workspace with
 * zero columns up to 64, 128 or 256, then flash_mfma / decode_split; the workspace
 * must be 256-byte aligned), "composed" (what none of these takes, from about
 * 3e7 multiply-adds and 64 queries and keys on: the reference's own composition,
 * csrc/ops/attention_ops.cpp:101-135, run as two batched paras_gemm_nt products
 * around one scale / mask / softmax row kernel, scores in `attn` or in the
 * 256-byte aligned workspace, a bounded piece at a time) or "generic". */
PARAS_API const char* paras_sdpa_kernel_name(const paras_sdpa_args* args);

/* ------------------------------------------------------------------------- */
/* MoE routing.  No reference function; each step is defined by a reference   */
/* primitive:                                                                 */
/*   topk  (csrc/ops/pointwise_ops.cpp:1292-1381): k largest of E logits,     */
/*         sorted descending, ties to the lower expert index;                 */
/*   _softmax over the k kept logits in fp32 (pointwise_ops.cpp:926-981);     */
/*   stable argsort of the flattened [T*k] expert ids                         */
/*         (csrc/ops/sort_ops.cpp:129-166): expert-major, (token,slot) order  */
/*         kept inside an expert;                                             */
/*   counts / offsets = histogram and exclusive cumsum                        */
/*         (pointwise_ops.cpp:1221-1265).                                     */
/* logits: [T, E] dtype `dtype`; topi: [T, k] int64; topw: [T, k] fp32;       */
/* order: [T*k] int64 (order[p] = t*k + slot of the p-th routed row);         */
/* inv_order: [T*k] int64 (position of flat slot in `order`; may be NULL);    */
/* counts: [E] int64; offsets: [E+1] int64.  1 <= k <= E <= 256 (up to 64     */
/* experts and 8 choices a token's logits and choices stay in registers;      */
/* beyond that they are re-read from memory, several times slower per token). */
/* `workspace`: paras_moe_route_workspace(T,E,k) bytes of device memory        */
/* (per-workgroup expert counts; contents on entry do not matter).  Up to      */
/* 65536 tokens the whole routing is one kernel: its workgroups publish their  */
/* counts stamped with the call's epoch and poll each other's.  Outside graph  */
/* capture that kernel is the only launch and the stamped counts live in the   */
/* library's own device memory (8 areas of 131,328 bytes per GPU, one per      */
/* stream by a hash of the handle; calls that overlap on one area stay exact   */
/* and turn slower: a workgroup waits about 300 us for the others' counts and  */
/* then counts for itself); on a stream that is being captured, or with        */
/* PARAS_ROUTE_OWN_SCRATCH=0, they live in `workspace`, which a fill kernel    */
/* queued in front clears.                                                     */
/* ------------------------------------------------------------------------- */
PARAS_API size_t paras_moe_route_workspace(int64_t T, int64_t E, int64_t k);
PARAS_API int paras_moe_route(const void* logits, int64_t T, int64_t E, int64_t k,
                              int dtype, int64_t* topi, float* topw, int64_t* order,
                              int64_t* inv_order, int64_t* counts, int64_t* offsets,
                              void* workspace, void* stream);
/* How many workgroups of paras_moe_route / paras_moe_route_noalloc stopped waiting
 * for the others and counted for themselves since the library was loaded, on the
 * current device (a diagnostic with no counterpart in the reference: results are
 * the same either way; a number that keeps growing says the routing kernel's
 * workgroups are not resident together, i.e. the chip is oversubscribed).
 * Synchronous: it copies one word from the device. */
PARAS_API int paras_moe_route_give_ups(uint64_t* count);

/* paras_moe_route for callers that cannot allocate (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and same outputs, bit for bit,
 * without the workspace: the per-workgroup counts live in a fixed array in the
 * library's device image (131,328 bytes per GPU, held until the process ends),
 * cleared by a fill kernel queued in front of the routing kernel.  Limits: 1 <= T <= 65536 tokens, E <= 64; larger
 * inputs are PARAS_ERR_INVALID.  The call allocates nothing and frees nothing.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU
 * (two streams, two threads) race; calls queued on one stream do not. */
PARAS_API int paras_moe_route_noalloc(const void* logits, int64_t T, int64_t E, int64_t k,
                                      int dtype, int64_t* topi, float* topw, int64_t* order,
                                      int64_t* inv_order, int64_t* counts, int64_t* offsets,
                                      void* stream);

/* ------------------------------------------------------------------------- */
/* MoE grouped expert FFN with SwiGLU.  Per routed row p (expert e):          */
/*   xp = x[order[p] / k]                                   (index_select,    */
/*                                   csrc/ops/indexing_ops.cpp:98-152)        */
/*   g = T(xp W_gate[e]^T), u = T(xp W_up[e]^T)             (mm_out,          */
/*                                   csrc/ops/vision_ops.cpp:388-396)         */
/*   h = T(silu(g) * u)                                     (fused_ops.cpp    */
/*                                   :162-194)                                */
/*   y = T(h W_down[e]^T)                                                     */
/*   out[t] = T( sum_slot T(y[inv_order[t*k+slot]] * T(topw[t][slot])) )      */
/*                                   (mul_out / sum_out,                      */
/*                                    pointwise_ops.cpp:280-284,766-774)      */
/* x: [T, H]; w_gate, w_up: [E, I, H]; w_down: [E, H, I]; out: [T, H];        */
/* all dtype `dtype` (bf16 or f16), GEMMs accumulate in fp32.  H and I that   */
/* are multiples of 64, with 16-byte aligned tensors, run on the MFMA tiles;  */
/* other sizes or alignments on general kernels (at most 65535 routed rows,   */
/* far slower), never on the host.                                            */
/* `workspace`: paras_moe_ffn_workspace(T,k,H,I) bytes of device memory.      */
/* ------------------------------------------------------------------------- */
PARAS_API size_t paras_moe_ffn_workspace(int64_t T, int64_t k, int64_t H, int64_t I,
                                         int dtype);
PARAS_API int paras_moe_ffn(const void* x, const void* w_gate, const void* w_up,
                            const void* w_down, const float* topw, const int64_t* order,
                            const int64_t* inv_order, const int64_t* offsets,
                            void* out, void* workspace, int64_t T, int64_t E, int64_t k,
                            int64_t H, int64_t I, int dtype, void* stream);

/* ------------------------------------------------------------------------- */
/* Dense NT GEMM (replaces the host bounce of mm / bmm / addmm / linear,       */
/* csrc/ops/vision_ops.cpp:248-309 (LinearFunction), :388-423 (mm_out,         */
/* bmm_out, addmm_out): copy to CPU, ATen GEMM with fp32 accumulation and one  */
/* rounding, copy back).  Per batch b:                                         */
/*   C[b] = T( alpha * A[b] B[b]^T + beta * addend[b] )                        */
/* A [M, K] rows lda apart, B [N, K] rows ldb apart (both contiguous along K:  */
/* x W^T of nn.Linear, q k^T), C [M, N] rows ldc apart; batch strides in       */
/* elements (0 = shared).  addend may be NULL; ld_add = 0 broadcasts one row   */
/* (a bias) over the M rows.  All four float dtypes.  bf16 / f16 with K a       */
/* multiple of 64 and 16-byte aligned operand rows run on the MFMA kernels     */
/* (fp32 accumulation, one rounding); fp32 tensors with at least 32 tiles of   */
/* 128 x 128 outputs on the fp32 MFMA kernel (full fp32 multiplies, any K and  */
/* alignment); everything else -- fp64 tensors, small fp32 products, 16-bit    */
/* ones with other K or alignments -- on a general kernel (fp32 accumulation,  */
/* fp64 for fp64 tensors), so no product needs a host path.                    */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_gemm_nt(const void* a, const void* b, const void* addend, void* c,
                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                            int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                            int64_t stride_b, int64_t stride_c, int64_t stride_add,
                            double alpha, double beta, int dtype, void* stream);
/* The same product with a caller-provided workspace of                        */
/* paras_gemm_nt_workspace(M, N, K, batch, dtype) bytes (0 for shapes that     */
/* need none; 16-byte aligned).  With it, bf16 / f16 products of 32 to 128     */
/* rows (decode-time projections) split the contraction over workgroups and    */
/* read the activations once per 128 weight rows; the partial sums are added   */
/* in a fixed order.  Without it (NULL) the call is paras_gemm_nt.  (Same      */
/* reference lines as above.)                                                  */
PARAS_API size_t paras_gemm_nt_workspace(int64_t M, int64_t N, int64_t K, int64_t batch,
                                         int dtype);
PARAS_API int paras_gemm_nt_ws(const void* a, const void* b, const void* addend, void* c,
                               int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                               int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                               int64_t stride_b, int64_t stride_c, int64_t stride_add,
                               double alpha, double beta, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* Row softmax and row top-k (replace softmax_out / topk_out,                  */
/* csrc/ops/pointwise_ops.cpp:926-981 and :1292-1381), over the last dim of a  */
/* contiguous [rows, n] tensor.                                                */
/*   softmax: fp64 per row, out_j = T_out(exp(v_j - max) / sum); dtype_out is  */
/*            dtype_in, or PARAS_F32 for a 16-bit input (half_to_float).       */
/*   top-k:   values [rows, k] (dtype of x) and int64 indices [rows, k], sorted,*/
/*            largest != 0 -> descending; ties go to the lower index.  Rows    */
/*            containing NaN have no defined order.                            */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_softmax_rows(const void* x, void* out, int64_t rows, int64_t n,
                                 int dtype_in, int dtype_out, void* stream);
PARAS_API int paras_topk_rows(const void* x, void* values, int64_t* indices, int64_t rows,
                              int64_t n, int64_t k, int largest, int dtype, void* stream);

/* ------------------------------------------------------------------------- */
/* Measurement aid (no counterpart in the reference): the rate, in TFLOP/s,    */
/* that the current device sustains on a register-only loop of                 */
/* v_mfma_f32_32x32x16_bf16 on random operands, with `waves_per_simd` (1 or 2) */
/* wavefronts per SIMD and `valu_per_mfma` (0 or 2) independent fp32           */
/* instructions after each MFMA.  The published dense bf16 peak assumes        */
/* 2.4 GHz; under this load the part is power limited and clocks lower, so     */
/* bench.py reports this figure beside the attention and GEMM figures of the   */
/* same process.  Blocks for about 0.2 s (150 ms of untimed load first: a short */
/* burst runs at a clock the part does not hold); allocates and frees 0.5 MB;  */
/* runs on the null stream.                                                    */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_mfma_rate_probe(int waves_per_simd, int valu_per_mfma, double* tflops);

/* ------------------------------------------------------------------------- */
/* Measurement aid (no counterpart in the reference): bytes per nanosecond and */
/* CU that one four-wavefront workgroup per CU pulls through the vector cache  */
/* when it does nothing but stream a region of `region_kib` KiB of its own     */
/* (a power of two, 8 ... 1024) over and over: with 64 KiB the regions of an   */
/* XCD's 32 workgroups stay in its 4 MB L2, with 256 KiB and more they come    */
/* from the last-level cache.  `to_lds` != 0: buffer loads that write LDS      */
/* directly (what a GEMM's staging would use); 0: loads into registers.  Tells */
/* whether a kernel's operand traffic is anywhere near what the memory side    */
/* delivers.  Blocks for a few ms; allocates and frees CUs x region bytes;     */
/* runs on the null stream.                                                    */
/* ------------------------------------------------------------------------- */
PARAS_API int paras_l2_stream_probe(int to_lds, int region_kib, double* bytes_per_ns_per_cu);

#ifdef __cplusplus
}
#endif
#endif /* PARAS_HIP_H */
