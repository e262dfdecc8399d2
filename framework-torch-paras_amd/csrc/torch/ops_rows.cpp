// aten::_softmax and aten::topk for the `paras` device (the reference's
// softmax / topk, csrc/ops/pointwise_ops.cpp:983-989 and :1383-1394): the
// reduced dim is moved last, the rows go through paras_softmax_rows /
// paras_topk_rows, and the result is moved back.  Float dtypes run on the
// device; integer top-k keeps the host route.
#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

bool is_float_type(const Tensor& t) {
    const auto st = t.scalar_type();
    return st == c10::kFloat || st == c10::kDouble || st == c10::kBFloat16 || st == c10::kHalf;
}

Tensor softmax(const Tensor& self, int64_t dim, bool half_to_float) {
    const int64_t d = c10::maybe_wrap_dim(dim, self.dim());
    TORCH_CHECK(is_float_type(self), "paras softmax: floating-point tensors only");
    const bool is16 = self.scalar_type() == c10::kBFloat16 || self.scalar_type() == c10::kHalf;
    TORCH_CHECK(!half_to_float || is16, "paras softmax: half_to_float needs a 16-bit input");
    const auto out_dtype = half_to_float ? c10::kFloat : self.scalar_type();
    if (self.dim() == 0) return at::ones({}, self.options().dtype(out_dtype));
    Tensor in = self.movedim(d, -1).contiguous();
    Tensor out = at::empty(in.sizes(), in.options().dtype(out_dtype));
    const int64_t n = in.size(-1);
    if (in.numel() > 0)
        check(paras_softmax_rows(in.data_ptr(), out.data_ptr(), in.numel() / n, n, require_float_code(in, "paras softmax"),
                                 require_float_code(out, "paras softmax"), stream_for(in)));
    return out.movedim(-1, d).contiguous();
}

std::tuple<Tensor, Tensor> topk(const Tensor& self, c10::SymInt k_sym, int64_t dim, bool largest, bool sorted) {
    const int64_t k = k_sym.guard_int(__FILE__, __LINE__);
    const int64_t d = c10::maybe_wrap_dim(dim, self.dim());
    const int64_t n = self.dim() == 0 ? 1 : self.size(d);
    TORCH_CHECK(k >= 0 && k <= n, "paras topk: k out of range");
    if (!is_float_type(self) || self.dim() == 0) {
        auto r = at::topk(self.to(c10::Device(c10::kCPU)), k, dim, largest, sorted);
        return {std::get<0>(r).to(self.device()), std::get<1>(r).to(self.device())};
    }
    Tensor in = self.movedim(d, -1).contiguous();
    std::vector<int64_t> shape(in.sizes().begin(), in.sizes().end());
    shape.back() = k;
    Tensor values = at::empty(shape, in.options());
    Tensor indices = at::empty(shape, in.options().dtype(c10::kLong));
    if (values.numel() > 0)
        check(paras_topk_rows(in.data_ptr(), values.data_ptr(), indices.data_ptr<int64_t>(), in.numel() / n, n, k, largest ? 1 : 0,
                              require_float_code(in, "paras topk"), stream_for(in)));
    return {values.movedim(-1, d).contiguous(), indices.movedim(-1, d).contiguous()};
}

}  // namespace

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
    m.impl("_softmax", softmax);
    m.impl("topk", topk);
}

}  // namespace paras_torch
