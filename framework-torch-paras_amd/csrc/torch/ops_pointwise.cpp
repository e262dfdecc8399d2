// aten::add / sub / mul / div (Tensor overloads and their in-place forms), cat and
// index_select (and through it embedding) for the `paras` device: the residual adds, RoPE products and scalings between
// the fused ops of a decoder block.  The reference evaluates them in its host
// engine's binary_kernel (csrc/ops/pointwise_ops.cpp:63-85, 262-302: both
// operands in the output dtype, a wrapped scalar narrowed to it first,
// result = T(a op alpha*b) in double); paras_binary_strided does the same on the
// GPU for float tensors, with broadcasting (two float dtypes are converted to the
// promoted one on the device first).  Anything else (integer tensors) takes ATen
// on host copies.
#include "paras_torch.h"

#include <ATen/ExpandUtils.h>

namespace paras_torch {
namespace {

using at::Tensor;

enum Op { kAdd = 0, kSub = 1, kMul = 2, kDiv = 3 };

bool is_host_number(const Tensor& t) { return !is_paras(t) && t.dim() == 0; }

// The device computes when `self` is a float paras tensor and `other` is a paras tensor of the
// same dtype or a zero-dim host tensor (a Python number, or a scalar tensor: neither promotes a
// float tensor's dtype unless it is complex).
bool device_takes(const Tensor& self, const Tensor& other) {
    if (!is_paras(self) || float_code(self.scalar_type()) < 0) return false;
    if (is_paras(other)) return other.scalar_type() == self.scalar_type() && other.device() == self.device();
    return is_host_number(other) && !other.is_complex();
}

Tensor on_host(const Tensor& t) { return is_paras(t) ? t.to(c10::Device(c10::kCPU)) : t; }

Tensor host_route(int op, const Tensor& self, const Tensor& other, const at::Scalar& alpha) {
    const Tensor a = on_host(self), b = on_host(other);
    Tensor r = op == kAdd ? at::add(a, b, alpha) : op == kSub ? at::sub(a, b, alpha) : op == kMul ? at::mul(a, b) : at::div(a, b);
    return r.to(is_paras(self) ? self.device() : other.device());
}

// `into`, when given, is a dense tensor of the broadcast shape that receives the result (the
// in-place forms pass `self`: element i is read before it is written by the same lane).
Tensor run(int op, const Tensor& self, const Tensor& other, double alpha, const Tensor* into = nullptr) {
    Tensor b = other;
    if (!is_paras(other)) {
        // the number, narrowed to the tensor's dtype as the reference does, as a one-element device tensor
        b = at::empty({}, self.options());
        b.fill_(other.to(self.scalar_type()).item());
    }
    const std::vector<int64_t> shape = at::infer_size(self.sizes(), b.sizes());
    TORCH_CHECK(shape.size() <= 8, "paras: tensor rank ", shape.size(), " exceeds kernel limit of 8");
    const Tensor a = self.expand(shape), bb = b.expand(shape);
    Tensor out = into != nullptr ? *into : at::empty(shape, self.options());
    if (out.numel() == 0) return out;
    check(paras_binary_strided(op, a.data_ptr(), bb.data_ptr(), out.data_ptr(), static_cast<int>(shape.size()), shape.data(),
                               a.strides().data(), bb.strides().data(), alpha, require_float_code(self, "paras binary op"),
                               stream_for(self)));
    return out;
}

bool float_pair_on_one_device(const Tensor& a, const Tensor& b) {
    return is_paras(a) && is_paras(b) && a.device() == b.device() && float_code(a.scalar_type()) >= 0 &&
           float_code(b.scalar_type()) >= 0;
}

Tensor binary(int op, const Tensor& self, const Tensor& other, const at::Scalar& alpha) {
    if (device_takes(self, other)) return run(op, self, other, alpha.toDouble());
    // number (op) tensor: add and mul commute; the others go to the host
    if ((op == kAdd || op == kMul) && is_host_number(self) && device_takes(other, self)) return run(op, other, self, alpha.toDouble());
    // Float tensors of two dtypes: both are brought to the promoted dtype on the device (the
    // reference's binary_kernel converts both operands to the output's dtype, which the structured
    // op has set to the promoted one; csrc/ops/pointwise_ops.cpp:66-69).
    if (float_pair_on_one_device(self, other)) {
        const auto common = at::result_type(self, other);
        if (float_code(common) >= 0) return run(op, self.to(common), other.to(common), alpha.toDouble());
    }
    return host_route(op, self, other, alpha);
}

// True when writing `self` element by element while `other` is being read cannot change what is read:
// different storages, or the very same view.
bool safe_to_write_in_place(const Tensor& self, const Tensor& other) {
    if (!is_paras(other) || !other.storage().is_alias_of(self.storage())) return true;
    return other.data_ptr() == self.data_ptr() && other.sizes() == self.sizes() && other.strides() == self.strides();
}

// In-place forms keep self's dtype: the reference converts `other` to it first and computes there
// (binary_kernel(self, other, self), csrc/ops/pointwise_ops.cpp:292-296).
Tensor& binary_(int op, Tensor& self, const Tensor& other, const at::Scalar& alpha) {
    Tensor b = other;
    if (float_pair_on_one_device(self, other) && other.scalar_type() != self.scalar_type()) b = other.to(self.scalar_type());
    if (device_takes(self, b)) {
        const std::vector<int64_t> shape = at::infer_size(self.sizes(), b.sizes());
        TORCH_CHECK(self.sizes().equals(shape), "paras: output with shape ", self.sizes(), " doesn't match the broadcast shape ", shape);
        if (self.is_contiguous() && safe_to_write_in_place(self, b)) {
            run(op, self, b, alpha.toDouble(), &self);
            return self;
        }
    }
    Tensor r = binary(op, self, b, alpha);
    TORCH_CHECK(r.sizes() == self.sizes(), "paras: output with shape ", self.sizes(), " doesn't match the broadcast shape ", r.sizes());
    TORCH_CHECK(at::canCast(r.scalar_type(), self.scalar_type()), "result type ", r.scalar_type(),
                " can't be cast to the desired output type ", self.scalar_type());
    self.copy_(r);
    return self;
}

Tensor add(const Tensor& self, const Tensor& other, const at::Scalar& alpha) { return binary(kAdd, self, other, alpha); }
Tensor sub(const Tensor& self, const Tensor& other, const at::Scalar& alpha) { return binary(kSub, self, other, alpha); }
Tensor mul(const Tensor& self, const Tensor& other) { return binary(kMul, self, other, 1); }
Tensor div(const Tensor& self, const Tensor& other) { return binary(kDiv, self, other, 1); }
Tensor& add_(Tensor& self, const Tensor& other, const at::Scalar& alpha) { return binary_(kAdd, self, other, alpha); }
Tensor& sub_(Tensor& self, const Tensor& other, const at::Scalar& alpha) { return binary_(kSub, self, other, alpha); }
Tensor& mul_(Tensor& self, const Tensor& other) { return binary_(kMul, self, other, 1); }
Tensor& div_(Tensor& self, const Tensor& other) { return binary_(kDiv, self, other, 1); }

// cat as the reference composes it (csrc/ops/pointwise_ops.cpp:1558-1590): the inputs are copied
// into slices of the result by the device's strided copy.
Tensor cat(const at::ITensorListRef& tensors, int64_t dim) {
    auto list = tensors.materialize();
    TORCH_CHECK(!list.empty(), "cat: expected non-empty tensor list");
    const Tensor* first = nullptr;
    for (const auto& r : list)
        if (!(r.get().dim() == 1 && r.get().numel() == 0)) { first = &r.get(); break; }    // legacy empty tensors are skipped
    if (first == nullptr) return at::empty({0}, list[0].get().options());
    const int64_t d = c10::maybe_wrap_dim(dim, first->dim());
    std::vector<int64_t> shape = first->sizes().vec();
    shape[d] = 0;
    for (const auto& r : list) {
        const Tensor& t = r.get();
        if (t.dim() == 1 && t.numel() == 0) continue;
        TORCH_CHECK(t.dim() == first->dim() && t.scalar_type() == first->scalar_type() && is_paras(t),
                    "paras cat: tensors must share rank, dtype and device");
        for (int64_t k = 0; k < t.dim(); ++k)
            TORCH_CHECK(k == d || t.size(k) == first->size(k), "paras cat: sizes must match except in dimension ", d);
        shape[d] += t.size(d);
    }
    Tensor out = at::empty(shape, first->options());
    int64_t off = 0;
    for (const auto& r : list) {
        const Tensor& t = r.get();
        if (t.numel() == 0) continue;
        out.narrow(d, off, t.size(d)).copy_(t);
        off += t.size(d);
    }
    return out;
}

Tensor index_select(const Tensor& self, int64_t dim, const Tensor& index) {
    TORCH_CHECK(index.dim() <= 1, "paras index_select: index must be 0-D or 1-D");
    TORCH_CHECK(index.scalar_type() == c10::kLong || index.scalar_type() == c10::kInt, "paras index_select: index must be int32 or int64");
    const int64_t d = c10::maybe_wrap_dim(dim, self.dim());
    Tensor idx = (index.dim() == 0 ? index.unsqueeze(0) : index).to(self.device(), c10::kLong).contiguous();
    Tensor src = self.dim() == 0 ? self.reshape({1}) : self.contiguous();
    std::vector<int64_t> shape = src.sizes().vec();
    int64_t outer = 1, inner = 1;
    for (int64_t k = 0; k < d; ++k) outer *= shape[k];
    for (int64_t k = d + 1; k < src.dim(); ++k) inner *= shape[k];
    const int64_t n_src = shape[d];
    shape[d] = idx.numel();
    Tensor out = at::empty(shape, src.options());
    if (out.numel() > 0)
        check(paras_index_select(src.data_ptr(), idx.data_ptr<int64_t>(), out.data_ptr(), outer, n_src, idx.numel(),
                                 inner * static_cast<int64_t>(src.element_size()), stream_for(self)));
    return self.dim() == 0 ? out.reshape({}) : out;
}

}  // namespace

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
    m.impl("cat", cat);
    m.impl("index_select", index_select);
    m.impl("add.Tensor", add);
    m.impl("sub.Tensor", sub);
    m.impl("mul.Tensor", mul);
    m.impl("div.Tensor", div);
    m.impl("add_.Tensor", add_);
    m.impl("sub_.Tensor", sub_);
    m.impl("mul_.Tensor", mul_);
    m.impl("div_.Tensor", div_);
}

}  // namespace paras_torch
