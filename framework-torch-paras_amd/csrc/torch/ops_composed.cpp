// aten::rms_norm and torch_paras::swiglu on the `paras` device: the two ops the
// reference builds by composing elementwise primitives, narrowing to the
// tensor dtype after each one (csrc/ops/rms_swiglu_ops.cpp:43-110).  Here each
// is one kernel that narrows at the same points.  torch_paras::swiglu is also
// registered for CPU tensors, as in the reference, with the plain composition.
#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

Tensor rms_norm(const Tensor& input, c10::IntArrayRef normalized_shape, const c10::optional<Tensor>& weight,
                c10::optional<double> eps) {
    const int64_t nd = static_cast<int64_t>(normalized_shape.size());
    TORCH_CHECK(nd >= 1, "paras rms_norm: normalized_shape must be non-empty");
    TORCH_CHECK(input.dim() >= nd, "paras rms_norm: input has fewer dims than normalized_shape");
    int64_t H = 1;
    for (int64_t i = 0; i < nd; ++i) {
        TORCH_CHECK(input.size(input.dim() - nd + i) == normalized_shape[i],
                    "paras rms_norm: normalized_shape does not match the trailing dims of input");
        H *= normalized_shape[i];
    }
    const bool has_w = weight.has_value() && weight->defined();
    require_same_device("paras rms_norm", input, {{"weight", has_w ? &*weight : nullptr}});
    if (has_w)
        TORCH_CHECK(weight->sizes().equals(normalized_shape), "paras rms_norm: weight shape must equal normalized_shape");
    Tensor in = input.contiguous();
    // A weight of another dtype: the reference's last step is `out * weight`, which promotes
    // (csrc/ops/rms_swiglu_ops.cpp:70-72), so the normalised tensor is formed in the input's dtype
    // and the product taken by the device's multiply in the promoted one.
    const bool fused_w = has_w && weight->scalar_type() == in.scalar_type();
    Tensor w;
    if (fused_w) w = weight->contiguous();
    Tensor out = at::empty_like(in);
    const int64_t rows = H > 0 ? in.numel() / H : 0;
    if (rows > 0 && H > 0)
        check(paras_rms_norm_composed_fwd(in.data_ptr(), fused_w ? w.data_ptr() : nullptr, out.data_ptr(), rows, H,
                                          eps.has_value() ? *eps : 1e-6, require_float_code(in, "paras rms_norm"),
                                          stream_for(in)));
    if (has_w && !fused_w) return at::mul(out, *weight);
    return out;
}

Tensor swiglu_device(const Tensor& x, const Tensor& gate) {
    TORCH_CHECK(x.scalar_type() == gate.scalar_type(), "paras swiglu: x and gate must have the same dtype");
    require_same_device("paras swiglu", x, {{"gate", &gate}});
    auto shape = at::infer_size(x.sizes(), gate.sizes());
    Tensor xe = x.expand(shape).contiguous(), ge = gate.expand(shape).contiguous();
    Tensor out = at::empty_like(xe);
    if (out.numel() == 0) return out;
    check(paras_swiglu_composed_fwd(xe.data_ptr(), ge.data_ptr(), out.data_ptr(), out.numel(),
                                    require_float_code(xe, "paras swiglu"), stream_for(xe)));
    return out;
}

Tensor swiglu_cpu(const Tensor& x, const Tensor& gate) { return x * at::silu(gate); }

}  // namespace
}  // namespace paras_torch

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) { m.impl("aten::rms_norm", &paras_torch::rms_norm); }

TORCH_LIBRARY_FRAGMENT(torch_paras, m) { m.def("swiglu(Tensor x, Tensor gate) -> Tensor"); }
TORCH_LIBRARY_IMPL(torch_paras, PrivateUse1, m) { m.impl("swiglu", &paras_torch::swiglu_device); }
TORCH_LIBRARY_IMPL(torch_paras, CPU, m) { m.impl("swiglu", &paras_torch::swiglu_cpu); }
