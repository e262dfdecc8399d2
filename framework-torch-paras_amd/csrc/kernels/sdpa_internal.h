// Launchers of the attention kernels; the C ABI entry point in sdpa.hip
// validates the request, picks one of them and calls it.
#pragma once

#include <hip/hip_runtime.h>

#include "paras_hip.h"

namespace paras {

// MFMA flash forward: bf16/f16, D == Dv in {64, 128}, no explicit mask
// (causal or none), no attention weights returned.
bool flash_supported(const paras_sdpa_args& a);
int  launch_flash(const paras_sdpa_args& a, hipStream_t s);
// Whether launch_flash takes its 64-queries-per-wavefront form (head size 128, no mask, enough
// long rows to fill the chip with one workgroup per CU); only meaningful when flash_supported.
bool flash_uses_wide(const paras_sdpa_args& a);

// Split-KV decode: short query (Lq * Hq/Hkv <= 16), long K/V, bf16/f16,
// D == Dv in {64, 128}, optional bool / additive mask, not causal.
bool   decode_supported(const paras_sdpa_args& a);
size_t decode_workspace(const paras_sdpa_args& a);
int    launch_decode(const paras_sdpa_args& a, void* workspace, hipStream_t s);

// MFMA attention that also returns the softmax weights (the math op): bf16/f16,
// D == Dv in {64, 128}, causal / bool / additive masks contiguous along the keys.
bool weights_supported(const paras_sdpa_args& a);
int  launch_weights(const paras_sdpa_args& a, hipStream_t s);

// The reference's composition run step by step with the library's own batched products and one
// row kernel (fp32 / fp64 tensors, head sizes and layouts the fused kernels do not take), for
// problems big enough that the general kernel would take milliseconds.
bool   composed_supported(const paras_sdpa_args& a);
size_t composed_workspace(const paras_sdpa_args& a);
int    launch_composed(const paras_sdpa_args& a, void* workspace, void* stream, hipStream_t s);

// paras_gemm_nt_ws (gemm.hip) with two hints for causal attention, which the fp32 matrix-core kernel
// uses and the others ignore: causal_kind 1 = the product is a score matrix of which row r only needs
// columns <= r + causal_first (tiles wholly beyond stay unwritten), 2 = `a` is such a matrix after
// its softmax (zeros beyond the diagonal), so a tile of rows contracts only as far as its last row sees.
int gemm_nt_causal(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                   int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                   void* workspace, size_t workspace_bytes, void* stream, int causal_kind, long causal_first);

// Everything else (fp32/fp64, any head size, other layouts).
size_t generic_workspace(const paras_sdpa_args& a);
int    launch_generic(const paras_sdpa_args& a, void* workspace, hipStream_t s);

}  // namespace paras
