// Scaled-dot-product attention on the `paras` device.
//
//  * aten::_scaled_dot_product_attention_math -- the op the reference registers
//    (csrc/ops/attention_ops.cpp:71-151), with the same checks, the same
//    (output, weights) result, GQA by head mapping instead of
//    repeat_interleave.  Because the weights must be produced, it always runs
//    the math-semantics kernel, which narrows where the reference's composed
//    path does.
//  * aten::_scaled_dot_product_fused_attention_overrideable, chosen for
//    F.scaled_dot_product_attention through the PrivateUse1 entry of
//    _fused_sdp_choice: no weights are returned, so the MFMA flash / split-KV
//    decode kernels serve every shape they accept (anything else still goes to
//    the math-semantics kernel inside libparas_hip.so).
#include <ATen/native/DispatchStub.h>
#include <ATen/native/transformers/attention.h>
#include <ATen/native/transformers/sdp_utils_cpp.h>

#include <cmath>
#include <limits>

#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

struct Prepared {
    Tensor q, k, v, mask;  // 4-D views / copies that own the memory the call reads
    paras_sdpa_args a{};
    std::vector<int64_t> out_shape;
};

// Brings (..., H, L, E) operands to 4-D with a contiguous last dim and fills the
// C-ABI argument block.  K/V heads are mapped, never repeated.
void prepare(const Tensor& query, const Tensor& key, const Tensor& value, const c10::optional<Tensor>& attn_mask,
             bool is_causal, c10::optional<double> scale, bool enable_gqa, Prepared* p) {
    TORCH_CHECK(query.dim() >= 3 && key.dim() >= 3 && value.dim() >= 3,
                "paras sdpa: query/key/value must be at least 3-D (..., seq, head_dim)");
    const bool has_mask = attn_mask.has_value() && attn_mask->defined();
    require_same_device("paras sdpa", query, {{"key", &key}, {"value", &value}, {"attn_mask", has_mask ? &*attn_mask : nullptr}});
    TORCH_CHECK(!(is_causal && has_mask), "paras sdpa: is_causal and attn_mask are mutually exclusive");
    TORCH_CHECK(query.scalar_type() == key.scalar_type() && key.scalar_type() == value.scalar_type(),
                "paras sdpa: query, key and value must have the same dtype");
    TORCH_CHECK(query.size(-1) == key.size(-1), "paras sdpa: query and key head dims differ");
    TORCH_CHECK(key.size(-2) == value.size(-2), "paras sdpa: key and value lengths differ");
    const int64_t Hq = query.size(-3), Hk = key.size(-3);
    if (enable_gqa && Hk != Hq)
        TORCH_CHECK(Hk > 0 && Hq % Hk == 0,
                    "paras sdpa: query heads must be a multiple of key/value heads for enable_gqa");
    TORCH_CHECK(value.size(-3) == Hk, "paras sdpa: key and value head counts differ");

    // Leading (batch) dims: flatten query's; key/value broadcast over them.
    auto to4 = [](const Tensor& t, c10::IntArrayRef lead) {
        std::vector<int64_t> full(lead.begin(), lead.end());
        full.insert(full.end(), t.sizes().end() - 3, t.sizes().end());
        Tensor e = t.expand(full);
        int64_t batch = 1;                       // (spelled out: -1 cannot be inferred for an empty tensor)
        for (int64_t d : lead) batch *= d;
        return e.reshape({batch, t.size(-3), t.size(-2), t.size(-1)});
    };
    std::vector<int64_t> lead(query.sizes().begin(), query.sizes().end() - 3);
    {
        std::vector<int64_t> kl(key.sizes().begin(), key.sizes().end() - 3);
        auto b = at::infer_size(lead, kl);
        lead.assign(b.begin(), b.end());
    }
    p->q = to4(query, lead);
    p->k = to4(key, lead);
    p->v = to4(value, lead);
    if (!enable_gqa || Hk == Hq) {
        // Without GQA the head dims must agree or broadcast (Hk == 1), as matmul would.
        TORCH_CHECK(Hk == Hq || Hk == 1, "paras sdpa: key/value heads (", Hk, ") do not match query heads (", Hq, ")");
    }
    // A contiguous last dim is required; 16-bit operands are also moved onto what the MFMA kernels
    // take (a 16-byte boundary, strides that are multiples of 8 elements) when a view is not: the
    // copy costs far less than the general kernel such a view would otherwise run on.
    auto last_contig = [](Tensor t) {
        if (!(t.stride(-1) == 1 || t.size(-1) <= 1)) return t.contiguous();
        if (t.element_size() != 2 || t.numel() == 0 || t.size(-1) % 8 != 0) return t;   // (a dense copy would not help an odd head size)
        bool ok = (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15) == 0;
        for (int64_t d = 0; d < 3; ++d) ok = ok && (t.size(d) <= 1 || t.stride(d) % 8 == 0);
        return ok ? t : t.clone(c10::MemoryFormat::Contiguous);
    };
    p->q = last_contig(p->q);
    p->k = last_contig(p->k);
    p->v = last_contig(p->v);

    paras_sdpa_args& a = p->a;
    a.q = p->q.data_ptr();
    a.k = p->k.data_ptr();
    a.v = p->v.data_ptr();
    a.B = p->q.size(0);
    a.Hq = Hq;
    a.Hkv = Hk;
    a.Lq = p->q.size(2);
    a.Lk = p->k.size(2);
    a.D = p->q.size(3);
    a.Dv = p->v.size(3);
    for (int i = 0; i < 3; ++i) {
        a.q_strides[i] = p->q.stride(i);
        a.k_strides[i] = p->k.stride(i);
        a.v_strides[i] = p->v.stride(i);
    }
    a.dtype = require_float_code(query, "paras sdpa");
    a.is_causal = is_causal ? 1 : 0;
    // The reference multiplies the scores by a scalar narrowed to the tensor
    // dtype (mul.out through to_compute, csrc/ops/pointwise_ops.cpp:55-60).
    const double s = scale.has_value() ? *scale : 1.0 / std::sqrt(static_cast<double>(a.D));
    a.scale = narrow_scalar(s, query.scalar_type());
    a.mask_kind = 0;
    if (has_mask) {
        Tensor m = *attn_mask;
        TORCH_CHECK(is_paras(m), "paras sdpa: attn_mask must be on the same device");
        if (m.scalar_type() == c10::kBool) {
            a.mask_kind = 1;
        } else {
            a.mask_kind = 2;
            if (m.scalar_type() != query.scalar_type()) m = m.to(query.scalar_type());
        }
        std::vector<int64_t> target(lead.begin(), lead.end());
        target.push_back(Hq);
        target.push_back(a.Lq);
        target.push_back(a.Lk);
        m = m.expand(target);
        if (lead.size() != 1) m = m.reshape({a.B, Hq, a.Lq, a.Lk});   // a view unless batch dims must merge
        p->mask = m;
        a.mask = m.data_ptr();
        for (int i = 0; i < 4; ++i) a.mask_strides[i] = m.stride(i);
    }
    p->out_shape.assign(query.sizes().begin(), query.sizes().end());
    p->out_shape.back() = a.Dv;
}

void run(Prepared* p, Tensor* out, Tensor* attn, Tensor* lse) {
    paras_sdpa_args& a = p->a;
    *out = empty_paras({a.B, a.Hq, a.Lq, a.Dv}, p->q.scalar_type(), p->q.device());
    a.out = out->data_ptr();
    if (attn != nullptr) {
        *attn = empty_paras({a.B, a.Hq, a.Lq, a.Lk}, p->q.scalar_type(), p->q.device());
        a.attn = attn->data_ptr();
    }
    if (lse != nullptr) {
        *lse = empty_paras({a.B, a.Hq, a.Lq}, c10::kFloat, p->q.device());
        a.lse = lse->data_ptr<float>();
    }
    if (out->numel() == 0 && (attn == nullptr || attn->numel() == 0)) return;
    void* st = stream_for(p->q);
    const size_t nws = paras_sdpa_workspace(&a);
    Tensor ws;
    if (nws > 0) ws = workspace(nws, p->q.device());
    check(paras_sdpa_fwd(&a, nws > 0 ? ws.data_ptr() : nullptr, st));
}

std::tuple<Tensor, Tensor> sdpa_math(const Tensor& query, const Tensor& key, const Tensor& value,
                                     const c10::optional<Tensor>& attn_mask, double dropout_p, bool is_causal,
                                     const c10::optional<Tensor>& dropout_mask, c10::optional<double> scale,
                                     bool enable_gqa) {
    Prepared p;
    prepare(query, key, value, attn_mask, is_causal, scale, enable_gqa, &p);
    Tensor out, attn;
    run(&p, &out, &attn, nullptr);
    std::vector<int64_t> attn_shape(p.out_shape);
    attn_shape.back() = p.a.Lk;
    attn = attn.reshape(attn_shape);
    if (dropout_p > 0.0) {
        // Dropout changes the weights before the second product; that is the
        // composed path's business (csrc/ops/attention_ops.cpp:129-134).
        Tensor dropped = dropout_mask.has_value() && dropout_mask->defined()
                             ? attn * *dropout_mask / (1.0 - dropout_p)
                             : at::dropout(attn, dropout_p, /*train=*/true);
        Tensor v = value;
        if (enable_gqa && key.size(-3) != query.size(-3)) v = v.repeat_interleave(query.size(-3) / key.size(-3), -3);
        return {at::matmul(dropped, v), dropped};
    }
    return {out.reshape(p.out_shape), attn};
}

using OverrideableResult = std::tuple<Tensor, Tensor, Tensor, Tensor, c10::SymInt, c10::SymInt, Tensor, Tensor, Tensor>;

OverrideableResult sdpa_overrideable(const Tensor& query, const Tensor& key, const Tensor& value,
                                     const c10::optional<Tensor>& attn_bias, double dropout_p, bool is_causal,
                                     bool return_debug_mask, c10::optional<double> scale) {
    TORCH_CHECK(dropout_p == 0.0, "paras sdpa: the fused path has no dropout; use the math op");
    (void)return_debug_mask;
    Prepared p;
    prepare(query, key, value, attn_bias, is_causal, scale, /*enable_gqa=*/true, &p);
    // (16-bit head sizes below 256 other than 64, 128 and 256 run on the MFMA kernels too: the library
    // pads q, k and v with zero columns inside its workspace.)
    Tensor out, lse;
    run(&p, &out, nullptr, &lse);
    std::vector<int64_t> lse_shape(p.out_shape.begin(), p.out_shape.end() - 1);
    const auto opts = query.options();
    Tensor none = at::empty({0}, opts.dtype(c10::kLong));
    return {out.reshape(p.out_shape), lse.reshape(lse_shape), none, none, c10::SymInt(p.a.Lq), c10::SymInt(p.a.Lk),
            at::empty({0}, opts.dtype(c10::kLong)), at::empty({0}, opts.dtype(c10::kLong)), at::empty({0}, opts)};
}

// F.scaled_dot_product_attention asks this which backend to use for `paras`
// tensors.  No dropout -> the fused entry above; otherwise the math op.
int64_t fused_sdp_choice(const Tensor& query, const Tensor& key, const Tensor& value,
                         const c10::optional<Tensor>& attn_mask, double dropout_p, bool is_causal,
                         c10::optional<double> scale, bool enable_gqa) {
    (void)attn_mask; (void)is_causal; (void)scale;
    // The fused op maps query heads onto fewer key/value heads by itself; the reference only
    // does so under enable_gqa (csrc/ops/attention_ops.cpp:83-92) and otherwise fails in its
    // matmul.  Without the flag such shapes go to the math op, whose checks raise.  Inputs that
    // need gradients also go there: the fused forward has no backward op behind it.
    const bool heads_ok = query.dim() < 3 || key.dim() < 3 || enable_gqa || key.size(-3) == query.size(-3) || key.size(-3) == 1;
    const bool needs_grad = at::GradMode::is_enabled() && (query.requires_grad() || key.requires_grad() || value.requires_grad());
    const bool fused = dropout_p == 0.0 && float_code(query.scalar_type()) >= 0 && query.dim() >= 3 && heads_ok && !needs_grad;
    return static_cast<int64_t>(fused ? sdp::SDPBackend::overrideable : sdp::SDPBackend::math);
}

}  // namespace
}  // namespace paras_torch

namespace at::native {
REGISTER_PRIVATEUSE1_DISPATCH(_fused_sdp_choice_stub, &paras_torch::fused_sdp_choice)
}  // namespace at::native

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
    m.impl("aten::_scaled_dot_product_attention_math", &paras_torch::sdpa_math);
    m.impl("aten::_scaled_dot_product_fused_attention_overrideable", &paras_torch::sdpa_overrideable);
}
