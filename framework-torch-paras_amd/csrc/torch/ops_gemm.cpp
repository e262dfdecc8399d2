// aten::mm / bmm / addmm for the `paras` device (and through them nn.Linear,
// torch.matmul, F.linear: they decompose to these with the weight as a
// transposed view).  The reference copies both operands to the host, runs the
// ATen-CPU GEMM and copies the result back (csrc/ops/vision_ops.cpp:388-423,
// 248-309); here every float product runs on the device (paras_gemm_nt: fp32
// accumulation -- fp64 for fp64 tensors -- and one rounding, as ATen-CPU does):
// bf16 / fp16 with a contraction size that is a multiple of 64 on the MFMA
// kernels, everything else on the general kernel.  Integer and mixed-dtype
// products are not part of this surface and raise.
#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

bool is_16bit_float(const Tensor& t) { return t.scalar_type() == c10::kBFloat16 || t.scalar_type() == c10::kHalf; }
bool is_float(const Tensor& t) {
    return is_16bit_float(t) || t.scalar_type() == c10::kFloat || t.scalar_type() == c10::kDouble;
}

// What the MFMA kernels want of an operand: rows contiguous along the last dim, row stride a
// multiple of 8 elements, 16-byte aligned base.  The general kernel only needs unit last stride.
bool rows_ok(const Tensor& t, bool mfma) {
    if (t.stride(-1) != 1 || t.stride(-2) < t.size(-1)) return false;
    return !mfma || (t.stride(-2) % 8 == 0 && (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15) == 0);
}
bool wants_mfma(const Tensor& a) { return is_16bit_float(a) && a.size(-1) > 0 && a.size(-1) % 64 == 0; }
Tensor as_rows(const Tensor& t, bool mfma) { return rows_ok(t, mfma) ? t : t.contiguous(); }

// `mat2` of a product A @ mat2 as the [N, K] row-major operand the NT kernel reads:
// a transposed view (the weight.t() of nn.Linear) is used in place, anything else is
// transposed with one strided device copy.
Tensor as_nt_operand(const Tensor& mat2, bool mfma) {
    Tensor bt = mat2.transpose(-1, -2);
    return rows_ok(bt, mfma) ? bt : bt.contiguous();
}

void check_dtypes(const Tensor& a, const Tensor& b, const char* what) {
    require_same_device(what, a, {{"mat2", &b}});
    TORCH_CHECK(a.scalar_type() == b.scalar_type(), "paras ", what, ": operand dtypes differ");
    TORCH_CHECK(is_float(a), "paras ", what, ": only float dtypes (fp32, fp64, bf16, fp16) are supported on the device");
}

// out[b] = alpha * a[b] @ mat2[b] + beta * addend; batch < 0: plain matrices
Tensor run_gemm(const Tensor& a_in, const Tensor& mat2, const c10::optional<Tensor>& addend, double alpha, double beta,
                int64_t batch) {
    const bool mfma = wants_mfma(a_in);
    Tensor a = as_rows(a_in, mfma), bt = as_nt_operand(mat2, mfma);
    const int64_t M = a.size(-2), K = a.size(-1), N = bt.size(-2);
    std::vector<int64_t> shape = batch >= 0 ? std::vector<int64_t>{batch, M, N} : std::vector<int64_t>{M, N};
    Tensor out = at::empty(shape, a.options());
    if (out.numel() == 0) return out;
    const void* add_ptr = nullptr;
    int64_t ld_add = 0, s_add = 0;
    Tensor add;
    if (addend.has_value() && addend->defined() && beta != 0.0) {
        add = addend->expand({M, N});                        // bias [N] or [1, N] -> row stride 0; full matrix -> its stride
        if (add.stride(-1) != 1 || (add.stride(-2) != 0 && add.stride(-2) < N)) add = add.contiguous();
        add_ptr = add.data_ptr();
        ld_add = add.stride(-2);
    }
    const int64_t nb = batch >= 0 ? batch : 1;
    const int code = require_float_code(a, "paras gemm");
    // few-row products (decode-time projections) run faster with a workspace for split partial sums
    const size_t ws_bytes = paras_gemm_nt_workspace(M, N, K, nb, code);
    Tensor ws;
    if (ws_bytes > 0) ws = at::empty({static_cast<int64_t>(ws_bytes)}, a.options().dtype(c10::kByte));
    check(paras_gemm_nt_ws(a.data_ptr(), bt.data_ptr(), add_ptr, out.data_ptr(), M, N, K, a.stride(-2), bt.stride(-2), N, ld_add,
                           nb, batch >= 0 ? a.stride(0) : 0, batch >= 0 ? bt.stride(0) : 0, M * N, s_add, alpha, beta, code,
                           ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, stream_for(a)));
    return out;
}

Tensor mm(const Tensor& self, const Tensor& mat2) {
    TORCH_CHECK(self.dim() == 2 && mat2.dim() == 2, "paras mm: both arguments must be 2-D");
    TORCH_CHECK(self.size(1) == mat2.size(0), "paras mm: shapes cannot be multiplied (", self.size(0), "x", self.size(1), " and ",
                mat2.size(0), "x", mat2.size(1), ")");
    check_dtypes(self, mat2, "mm");
    return run_gemm(self, mat2, c10::nullopt, 1.0, 0.0, -1);
}

Tensor bmm(const Tensor& self, const Tensor& mat2) {
    TORCH_CHECK(self.dim() == 3 && mat2.dim() == 3, "paras bmm: both arguments must be 3-D");
    TORCH_CHECK(self.size(0) == mat2.size(0) && self.size(2) == mat2.size(1), "paras bmm: shapes cannot be multiplied");
    check_dtypes(self, mat2, "bmm");
    // the MFMA kernels need batch strides that keep rows 16-byte aligned; dense copies otherwise
    const bool mfma = wants_mfma(self);
    Tensor a = (rows_ok(self, mfma) && (!mfma || self.stride(0) % 8 == 0)) ? self : self.contiguous();
    Tensor bt = mat2.transpose(-1, -2);
    if (!(rows_ok(bt, mfma) && (!mfma || bt.stride(0) % 8 == 0))) bt = bt.contiguous();
    return run_gemm(a, bt.transpose(-1, -2), c10::nullopt, 1.0, 0.0, self.size(0));
}

Tensor addmm(const Tensor& self, const Tensor& mat1, const Tensor& mat2, const at::Scalar& beta, const at::Scalar& alpha) {
    TORCH_CHECK(mat1.dim() == 2 && mat2.dim() == 2, "paras addmm: matrices must be 2-D");
    TORCH_CHECK(mat1.size(1) == mat2.size(0), "paras addmm: shapes cannot be multiplied");
    check_dtypes(mat1, mat2, "addmm");
    TORCH_CHECK(self.scalar_type() == mat1.scalar_type(), "paras addmm: operand dtypes differ");
    require_same_device("addmm", mat1, {{"self", &self}});
    return run_gemm(mat1, mat2, self, alpha.toDouble(), beta.toDouble(), -1);
}

}  // namespace

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
    m.impl("mm", mm);
    m.impl("bmm", bmm);
    m.impl("addmm", addmm);
}

}  // namespace paras_torch
