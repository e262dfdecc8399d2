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
    int  m_tiles, n_units;      // row tiles (128 or 256 rows), 256-column units
    float alpha, beta;
};

// S = Tile128 (4 waves, 128 rows) or Tile256 (8 waves, 256 rows; for problems with at least
// 128 tiles of 256 x 256).
template <typename T, typename S>
__global__ __launch_bounds__(S::kThreads, 2) void dense_gemm_nt_kernel(const DenseParams p) {
    using El = Elem<T>;
    __shared__ __attribute__((aligned(16))) typename S::Lds lds;

    // Column units innermost: the workgroups running together share the A row panel
    // (and, across m-tiles, stream the same B panels through L2).
    const long per_batch = static_cast<long>(p.m_tiles) * p.n_units;
    const long bidx = blockIdx.x / per_batch, rem = blockIdx.x % per_batch;
    const int mt = static_cast<int>(rem / p.n_units), nu = static_cast<int>(rem % p.n_units);
    const long row0 = static_cast<long>(mt) * S::kBM, n0 = static_cast<long>(nu) * 2 * kBN;
    const std::uint16_t* A = p.a + bidx * p.sa;
    const std::uint16_t* B = p.b + bidx * p.sb;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    unsigned a_off[4], b_off[2][S::kBChunks];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * S::kThreads;
        long arow = row0 + (c >> 3);
        if (arow >= p.M) arow = p.M - 1;     // clamped rows are computed but never stored
        a_off[i] = static_cast<unsigned>(arow * p.lda + (c & 7) * 8);
    }
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < S::kBChunks; ++i) {
            const int c = tid + i * S::kThreads;
            long brow = n0 + g * kBN + (c >> 3);
            if (brow >= p.N) brow = p.N - 1;
            b_off[g][i] = static_cast<unsigned>(brow * p.ldb + (c & 7) * 8);
        }
    const std::uint16_t* const b_base[2] = {B, B};
    float16_t acc[2][2][2];
    S::template mainloop<T>(A, a_off, b_base, b_off, p.K, lds, acc);

    std::uint16_t* C = p.c + bidx * p.sc;
    const std::uint16_t* ADD = p.add ? p.add + bidx * p.sadd : nullptr;
#pragma unroll
    for (int g = 0; g < 2; ++g)
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

template <typename T, typename S>
void launch_dense(const DenseParams& p, unsigned grid, hipStream_t s) {
    hipLaunchKernelGGL((dense_gemm_nt_kernel<T, S>), dim3(grid), dim3(S::kThreads), 0, s, p);
}

}  // namespace
}  // namespace paras

extern "C" {

int paras_gemm_nt(const void* a, const void* b, const void* addend, void* c, int64_t M, int64_t N, int64_t K,
                  int64_t lda, int64_t ldb, int64_t ldc, int64_t ld_add, int64_t batch, int64_t stride_a,
                  int64_t stride_b, int64_t stride_c, int64_t stride_add, double alpha, double beta, int dtype,
                  void* stream) {
    using namespace paras;
    PARAS_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "paras_gemm_nt: negative shape");
    if (M == 0 || N == 0 || batch == 0) return PARAS_OK;
    PARAS_REQUIRE(dtype == PARAS_BF16 || dtype == PARAS_F16, "paras_gemm_nt: dtype must be bf16 or f16");
    if (K == 0 || K % gemm::kBK != 0)
        return fail(PARAS_ERR_UNSUPPORTED, "paras_gemm_nt: the contraction size (%lld) must be a positive multiple of %d",
                    (long long)K, gemm::kBK);
    PARAS_REQUIRE(a && b && c, "paras_gemm_nt: null pointer");
    PARAS_REQUIRE(lda >= K && ldb >= K && ldc >= N && (addend == nullptr || ld_add == 0 || ld_add >= N),
                  "paras_gemm_nt: a leading dimension is smaller than its row");
    if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) != 0 || lda % 8 != 0 || ldb % 8 != 0 ||
        stride_a % 8 != 0 || stride_b % 8 != 0)
        return fail(PARAS_ERR_UNSUPPORTED, "paras_gemm_nt: operand rows must be 16-byte aligned");
    const int64_t n_units = (N + 2 * gemm::kBN - 1) / (2 * gemm::kBN);
    const int64_t wide_tiles = (M + gemm::wide::kBM - 1) / gemm::wide::kBM * n_units * batch;
    // measured: faster from half a round of one workgroup per CU upwards (given rows to fill a tile)
    const bool use_wide = wide_tiles >= 128 && M > gemm::kBM;
    const int64_t bm = use_wide ? gemm::wide::kBM : gemm::kBM;
    const int64_t m_tiles = (M + bm - 1) / bm;
    PARAS_REQUIRE(m_tiles * n_units * batch <= 0x7fffffffLL, "paras_gemm_nt: too many tiles");
    if (M * lda >= (1LL << 32) || N * ldb >= (1LL << 32))
        return fail(PARAS_ERR_UNSUPPORTED, "paras_gemm_nt: an operand matrix spans 2^32 elements or more");
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
    p.m_tiles = static_cast<int>(m_tiles); p.n_units = static_cast<int>(n_units);
    p.alpha = static_cast<float>(alpha); p.beta = static_cast<float>(beta);
    const unsigned blocks = static_cast<unsigned>(m_tiles * n_units * batch);
    if (use_wide) {
        if (dtype == PARAS_BF16) launch_dense<bf16_t, gemm::Tile256>(p, blocks, s);
        else                     launch_dense<f16_t, gemm::Tile256>(p, blocks, s);
    } else {
        if (dtype == PARAS_BF16) launch_dense<bf16_t, gemm::Tile128>(p, blocks, s);
        else                     launch_dense<f16_t, gemm::Tile128>(p, blocks, s);
    }
    PARAS_HIP_TRY(hipGetLastError());
    return PARAS_OK;
}

}  // extern "C"
