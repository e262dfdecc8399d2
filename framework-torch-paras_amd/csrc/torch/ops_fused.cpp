// The `paras::` op namespace: fused RMSNorm / SwiGLU / rotate_half with their
// explicit backward ops (same schemas as the reference, csrc/ops/fused_ops.cpp:
// 307-325), plus the MoE routing and grouped expert FFN ops this build adds.
// Each function validates like the reference op does and hands contiguous
// device pointers to libparas_hip.so.
#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

std::tuple<Tensor, Tensor> rms_norm(const Tensor& input, const Tensor& weight, double eps) {
    TORCH_CHECK(input.dim() <= 8, "paras rms_norm: rank exceeds kernel limit");
    TORCH_CHECK(input.dim() >= 1, "paras rms_norm: input must have rank >= 1");
    require_same_device("paras rms_norm", input, {{"weight", &weight}});
    Tensor in = input.contiguous();
    Tensor w = weight.contiguous();
    const int64_t H = in.size(-1);
    const int64_t rows = H > 0 ? in.numel() / H : 0;
    TORCH_CHECK(w.numel() == H, "paras rms_norm: weight size must match the last dimension");
    TORCH_CHECK(w.scalar_type() == in.scalar_type(), "paras rms_norm: weight dtype must match input dtype");
    Tensor out = at::empty_like(in);
    Tensor rstd = at::empty({rows}, in.options().dtype(c10::kFloat));
    if (rows == 0 || H == 0) return {out, rstd};
    check(paras_rms_norm_fwd(in.data_ptr(), w.data_ptr(), out.data_ptr(), rstd.data_ptr<float>(), rows, H, eps,
                             require_float_code(in, "paras rms_norm"), stream_for(in)));
    return {out, rstd};
}

std::tuple<Tensor, Tensor> rms_norm_backward(const Tensor& grad_out, const Tensor& input, const Tensor& weight,
                                             const Tensor& rstd) {
    require_same_device("paras rms_norm_backward", input, {{"grad_out", &grad_out}, {"weight", &weight}, {"rstd", &rstd}});
    require_same_dtype("paras rms_norm_backward", input, {{"grad_out", &grad_out}, {"weight", &weight}});
    Tensor go = grad_out.contiguous(), in = input.contiguous(), w = weight.contiguous();
    Tensor rs = rstd.contiguous();
    const int64_t H = in.size(-1);
    const int64_t rows = H > 0 ? in.numel() / H : 0;
    TORCH_CHECK(go.numel() == in.numel() && w.numel() == H && rs.numel() == rows && rs.scalar_type() == c10::kFloat,
                "paras rms_norm_backward: shape mismatch");
    Tensor grad_input = at::empty_like(in);
    Tensor grad_weight = at::zeros({H}, w.options());
    if (rows == 0 || H == 0) return {grad_input, grad_weight};
    Tensor ws = workspace(paras_rms_norm_bwd_workspace(rows, H), in.device());
    check(paras_rms_norm_bwd(go.data_ptr(), in.data_ptr(), w.data_ptr(), rs.data_ptr<float>(), grad_input.data_ptr(),
                             grad_weight.data_ptr(), ws.data_ptr(), rows, H, require_float_code(in, "paras rms_norm_backward"),
                             stream_for(in)));
    return {grad_input, grad_weight};
}

Tensor swiglu(const Tensor& gate, const Tensor& up) {
    TORCH_CHECK(gate.sizes() == up.sizes(), "paras swiglu: gate and up must have the same shape");
    TORCH_CHECK(gate.dim() <= 8, "paras swiglu: rank exceeds kernel limit");
    TORCH_CHECK(gate.scalar_type() == up.scalar_type(), "paras swiglu: gate and up must have the same dtype");
    require_same_device("paras swiglu", gate, {{"up", &up}});
    Tensor g = gate.contiguous(), u = up.contiguous();
    Tensor out = at::empty_like(g);
    if (out.numel() == 0) return out;
    check(paras_swiglu_fwd(g.data_ptr(), u.data_ptr(), out.data_ptr(), out.numel(), require_float_code(g, "paras swiglu"),
                           stream_for(g)));
    return out;
}

std::tuple<Tensor, Tensor> swiglu_backward(const Tensor& grad_out, const Tensor& gate, const Tensor& up) {
    require_same_device("paras swiglu_backward", grad_out, {{"gate", &gate}, {"up", &up}});
    require_same_dtype("paras swiglu_backward", grad_out, {{"gate", &gate}, {"up", &up}});
    Tensor go = grad_out.contiguous(), g = gate.contiguous(), u = up.contiguous();
    TORCH_CHECK(go.numel() == g.numel() && g.numel() == u.numel(), "paras swiglu_backward: shape mismatch");
    Tensor grad_gate = at::empty_like(g), grad_up = at::empty_like(u);
    if (go.numel() == 0) return {grad_gate, grad_up};
    check(paras_swiglu_bwd(go.data_ptr(), g.data_ptr(), u.data_ptr(), grad_gate.data_ptr(), grad_up.data_ptr(), go.numel(),
                           require_float_code(go, "paras swiglu_backward"), stream_for(go)));
    return {grad_gate, grad_up};
}

Tensor rotate_half_impl(const Tensor& x, bool backward, const char* name) {
    TORCH_CHECK(x.dim() >= 1, "paras ", name, ": input must have rank >= 1");
    require_same_device(name, x, {});
    TORCH_CHECK(x.dim() <= 8, "paras ", name, ": rank exceeds kernel limit");
    const int64_t D = x.size(-1);
    TORCH_CHECK(D % 2 == 0, "paras ", name, ": last dimension must be even");
    Tensor in = x.contiguous();
    Tensor out = at::empty_like(in);
    if (out.numel() == 0) return out;
    check(paras_rotate_half(in.data_ptr(), out.data_ptr(), in.numel() / D, D, backward ? 1 : 0,
                            require_float_code(in, name), stream_for(in)));
    return out;
}
Tensor rotate_half(const Tensor& x) { return rotate_half_impl(x, false, "rotate_half"); }
Tensor rotate_half_backward(const Tensor& g) { return rotate_half_impl(g, true, "rotate_half_backward"); }

// ---- MoE (no reference op; composition of reference primitives) -----------------
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor> moe_route(const Tensor& logits, int64_t k) {
    TORCH_CHECK(logits.dim() == 2, "paras moe_route: logits must be [tokens, experts]");
    require_same_device("paras moe_route", logits, {});
    Tensor lg = logits.contiguous();
    const int64_t T = lg.size(0), E = lg.size(1);
    TORCH_CHECK(E >= 1 && E <= 256, "paras moe_route: expert count must be in [1, 256]");
    TORCH_CHECK(k >= 1 && k <= E, "paras topk: k out of range");
    const auto i64 = lg.options().dtype(c10::kLong);
    Tensor topi = at::empty({T, k}, i64), topw = at::empty({T, k}, lg.options().dtype(c10::kFloat));
    Tensor order = at::empty({T * k}, i64), inv = at::empty({T * k}, i64);
    Tensor counts = at::empty({E}, i64), offsets = at::empty({E + 1}, i64);
    Tensor ws = workspace(paras_moe_route_workspace(T, E, k), lg.device());
    check(paras_moe_route(lg.data_ptr(), T, E, k, require_float_code(lg, "paras moe_route"), topi.data_ptr<int64_t>(),
                          topw.data_ptr<float>(), order.data_ptr<int64_t>(), inv.data_ptr<int64_t>(),
                          counts.data_ptr<int64_t>(), offsets.data_ptr<int64_t>(), ws.data_ptr(), stream_for(lg)));
    return {topi, topw, order, inv, counts, offsets};
}

Tensor moe_ffn(const Tensor& x, const Tensor& w_gate, const Tensor& w_up, const Tensor& w_down, const Tensor& topw,
               const Tensor& order, const Tensor& inv_order, const Tensor& offsets, int64_t k) {
    TORCH_CHECK(x.dim() == 2 && w_gate.dim() == 3 && w_up.dim() == 3 && w_down.dim() == 3,
                "paras moe_ffn: x [T,H], w_gate/w_up [E,I,H], w_down [E,H,I]");
    const int64_t T = x.size(0), H = x.size(1), E = w_gate.size(0), I = w_gate.size(1);
    TORCH_CHECK(w_gate.size(2) == H && w_up.sizes() == w_gate.sizes() && w_down.size(0) == E && w_down.size(1) == H &&
                    w_down.size(2) == I,
                "paras moe_ffn: weight shapes do not match");
    TORCH_CHECK(topw.numel() == T * k && order.numel() == T * k && inv_order.numel() == T * k && offsets.numel() == E + 1,
                "paras moe_ffn: routing tensors do not match T*k / E");
    TORCH_CHECK(x.scalar_type() == c10::kBFloat16 || x.scalar_type() == c10::kHalf,
                "paras moe_ffn: dtype must be bfloat16 or float16");
    require_same_device("paras moe_ffn", x, {{"w_gate", &w_gate}, {"w_up", &w_up}, {"w_down", &w_down}, {"topw", &topw},
                                             {"order", &order}, {"inv_order", &inv_order}, {"offsets", &offsets}});
    require_same_dtype("paras moe_ffn", x, {{"w_gate", &w_gate}, {"w_up", &w_up}, {"w_down", &w_down}});
    TORCH_CHECK(topw.scalar_type() == c10::kFloat, "paras moe_ffn: topw must be float32");
    TORCH_CHECK(order.scalar_type() == c10::kLong && inv_order.scalar_type() == c10::kLong && offsets.scalar_type() == c10::kLong,
                "paras moe_ffn: order, inv_order and offsets must be int64");
    // dense, and on a 16-byte boundary (a view at an odd storage offset is copied): what the MFMA tiles take
    auto dense16 = [](const Tensor& t) {
        Tensor c = t.contiguous();
        return (reinterpret_cast<uintptr_t>(c.data_ptr()) & 15) == 0 ? c : c.clone();
    };
    Tensor xc = dense16(x), wg = dense16(w_gate), wu = dense16(w_up), wd = dense16(w_down);
    Tensor tw = topw.contiguous(), od = order.contiguous(), iv = inv_order.contiguous(), of = offsets.contiguous();
    Tensor out = at::empty({T, H}, xc.options());
    if (T == 0) return out;
    const int dt = require_float_code(xc, "paras moe_ffn");
    Tensor ws = workspace(paras_moe_ffn_workspace(T, k, H, I, dt), xc.device());
    check(paras_moe_ffn(xc.data_ptr(), wg.data_ptr(), wu.data_ptr(), wd.data_ptr(), tw.data_ptr<float>(),
                        od.data_ptr<int64_t>(), iv.data_ptr<int64_t>(), of.data_ptr<int64_t>(), out.data_ptr(), ws.data_ptr(),
                        T, E, k, H, I, dt, stream_for(xc)));
    return out;
}

}  // namespace
}  // namespace paras_torch

TORCH_LIBRARY(paras, m) {
    m.def("rms_norm(Tensor input, Tensor weight, float eps) -> (Tensor, Tensor)");
    m.def("rms_norm_backward(Tensor grad_out, Tensor input, Tensor weight, Tensor rstd) -> (Tensor, Tensor)");
    m.def("swiglu(Tensor gate, Tensor up) -> Tensor");
    m.def("swiglu_backward(Tensor grad_out, Tensor gate, Tensor up) -> (Tensor, Tensor)");
    m.def("rotate_half(Tensor x) -> Tensor");
    m.def("rotate_half_backward(Tensor grad_out) -> Tensor");
    m.def("moe_route(Tensor logits, int k) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
    m.def("moe_ffn(Tensor x, Tensor w_gate, Tensor w_up, Tensor w_down, Tensor topw, Tensor order, "
          "Tensor inv_order, Tensor offsets, int k) -> Tensor");
}

TORCH_LIBRARY_IMPL(paras, PrivateUse1, m) {
    using namespace paras_torch;
    m.impl("rms_norm", &rms_norm);
    m.impl("rms_norm_backward", &rms_norm_backward);
    m.impl("swiglu", &swiglu);
    m.impl("swiglu_backward", &swiglu_backward);
    m.impl("rotate_half", &rotate_half);
    m.impl("rotate_half_backward", &rotate_half_backward);
    m.impl("moe_route", &moe_route);
    m.impl("moe_ffn", &moe_ffn);
}
