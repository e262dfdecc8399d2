// C ABI entry points of scaled-dot-product attention: validation and kernel
// choice.  Checks mirror the reference op's (csrc/ops/attention_ops.cpp:77-90).
#include <hip/hip_runtime.h>

#include <cmath>

#include "core/device_context.h"
#include "core/status.h"
#include "kernels/sdpa_internal.h"
#include "paras_hip.h"

namespace paras {
namespace {

enum class SdpaKernel { Flash, Decode, Weights, Padded, Composed, Generic };

int validate(const paras_sdpa_args* a) {
    PARAS_REQUIRE(a != nullptr, "paras sdpa: null argument block");
    PARAS_REQUIRE(a->B >= 0 && a->Hq >= 0 && a->Hkv >= 0 && a->Lq >= 0 && a->Lk >= 0 && a->D >= 0 && a->Dv >= 0,
                  "paras sdpa: negative shape");
    PARAS_REQUIRE(!(a->is_causal && a->mask_kind != 0),
                  "paras sdpa: is_causal and attn_mask are mutually exclusive");
    PARAS_REQUIRE(a->mask_kind >= 0 && a->mask_kind <= 2, "paras sdpa: mask_kind must be 0, 1 or 2");
    PARAS_REQUIRE(a->mask_kind == 0 || a->mask != nullptr, "paras sdpa: mask_kind set but mask is null");
    PARAS_REQUIRE(a->dtype >= PARAS_F32 && a->dtype <= PARAS_F64, "paras sdpa: unknown dtype %d", a->dtype);
    if (a->Hq > 0)
        PARAS_REQUIRE(a->Hkv > 0 && a->Hq % a->Hkv == 0,
                      "paras sdpa: query heads must be a multiple of key/value heads for enable_gqa");
    return PARAS_OK;
}

bool empty_output(const paras_sdpa_args& a) { return a.B == 0 || a.Hq == 0 || a.Lq == 0 || a.Dv == 0; }

// 16-bit head sizes below 256 other than 64 and 128: the MFMA kernels exist for 64, 128 and 256, so q, k and v
// are copied into the workspace with zero columns appended (q.k and the first D output columns do
// not change; the scale is the caller's, i.e. that of the real head size) and the first D columns
// of the padded result are copied out -- instead of the general fp64 kernel, three orders of
// magnitude slower.
struct PaddedPlan {
    paras_sdpa_args inner;      // the padded problem; its pointers are offsets into the workspace until bound
    size_t q_off, k_off, v_off, out_off, inner_off, total;
};
size_t up256(size_t n) { return (n + 255) / 256 * 256; }

bool plan_padded(const paras_sdpa_args& a, PaddedPlan* plan) {
    if (a.dtype != PARAS_BF16 && a.dtype != PARAS_F16) return false;
    if (a.attn != nullptr || a.D != a.Dv || a.D < 1 || a.D >= 256 || a.D == 64 || a.D == 128) return false;
    if (a.Lq < 1 || a.Lk < 1) return false;
    const int64_t Dp = a.D < 64 ? 64 : a.D < 128 ? 128 : 256;
    PaddedPlan pl{};
    pl.inner = a;
    pl.inner.D = pl.inner.Dv = Dp;
    const int64_t qs[3] = {a.Hq * a.Lq * Dp, a.Lq * Dp, Dp}, ks[3] = {a.Hkv * a.Lk * Dp, a.Lk * Dp, Dp};
    for (int i = 0; i < 3; ++i) {
        pl.inner.q_strides[i] = qs[i];
        pl.inner.k_strides[i] = ks[i];
        pl.inner.v_strides[i] = ks[i];
    }
    size_t off = 0;
    pl.q_off = off;   off += up256(static_cast<size_t>(a.B * a.Hq * a.Lq * Dp) * 2);
    pl.k_off = off;   off += up256(static_cast<size_t>(a.B * a.Hkv * a.Lk * Dp) * 2);
    pl.v_off = off;   off += up256(static_cast<size_t>(a.B * a.Hkv * a.Lk * Dp) * 2);
    pl.out_off = off; off += up256(static_cast<size_t>(a.B * a.Hq * a.Lq * Dp) * 2);
    pl.inner_off = off;
    // the support checks look at pointer alignment: stand-ins with the alignment the bound ones will have
    char* const fake = reinterpret_cast<char*>(static_cast<uintptr_t>(256));
    pl.inner.q = fake; pl.inner.k = fake; pl.inner.v = fake; pl.inner.out = fake;
    size_t inner_ws = 0;
    if (decode_supported(pl.inner)) inner_ws = decode_workspace(pl.inner);
    else if (!flash_supported(pl.inner)) return false;
    pl.total = off + up256(inner_ws);
    if (plan) *plan = pl;
    return true;
}

SdpaKernel choose(const paras_sdpa_args& a) {
    if (decode_supported(a)) return SdpaKernel::Decode;
    if (flash_supported(a)) return SdpaKernel::Flash;
    if (weights_supported(a)) return SdpaKernel::Weights;
    if (plan_padded(a, nullptr)) return SdpaKernel::Padded;
    if (composed_supported(a)) return SdpaKernel::Composed;
    return SdpaKernel::Generic;
}

int launch_padded(const paras_sdpa_args& a, void* workspace, void* stream, hipStream_t s) {
    PaddedPlan pl;
    PARAS_REQUIRE(plan_padded(a, &pl), "paras sdpa: not a shape for the padded route");
    PARAS_REQUIRE(workspace != nullptr, "paras sdpa: workspace is null");
    PARAS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "paras sdpa: the workspace must be 256-byte aligned");
    char* ws = static_cast<char*>(workspace);
    paras_sdpa_args in = pl.inner;
    in.q = ws + pl.q_off; in.k = ws + pl.k_off; in.v = ws + pl.v_off; in.out = ws + pl.out_off;
    const int64_t Dp = in.D, one = 1;
    // zeros (a fill kernel: the caller may be capturing this stream), then the real columns
    const int64_t zero_elems = static_cast<int64_t>(pl.out_off / 2);      // q, k, v regions
    int rc = paras_fill_strided(ws, 1, &zero_elems, &one, 2, 0, stream);
    if (rc != PARAS_OK) return rc;
    auto copy_in = [&](const void* src, const int64_t (&st)[3], void* dst, int64_t H, int64_t L) {
        const int64_t sizes[4] = {a.B, H, L, a.D}, ss[4] = {st[0], st[1], st[2], 1}, ds[4] = {H * L * Dp, L * Dp, Dp, 1};
        return paras_copy_strided(src, dst, 4, sizes, ss, ds, 2, a.dtype, a.dtype, stream);
    };
    if ((rc = copy_in(a.q, a.q_strides, const_cast<void*>(in.q), a.Hq, a.Lq)) != PARAS_OK) return rc;
    if ((rc = copy_in(a.k, a.k_strides, const_cast<void*>(in.k), a.Hkv, a.Lk)) != PARAS_OK) return rc;
    if ((rc = copy_in(a.v, a.v_strides, const_cast<void*>(in.v), a.Hkv, a.Lk)) != PARAS_OK) return rc;
    if (decode_supported(in)) rc = launch_decode(in, ws + pl.inner_off, s);
    else                      rc = launch_flash(in, s);
    if (rc != PARAS_OK) return rc;
    const int64_t sizes[4] = {a.B, a.Hq, a.Lq, a.D}, ss[4] = {a.Hq * a.Lq * Dp, a.Lq * Dp, Dp, 1},
                  ds[4] = {a.Hq * a.Lq * a.D, a.Lq * a.D, a.D, 1};
    return paras_copy_strided(in.out, a.out, 4, sizes, ss, ds, 2, a.dtype, a.dtype, stream);
}

}  // namespace
}  // namespace paras

extern "C" {

const char* paras_sdpa_kernel_name(const paras_sdpa_args* args) {
    using namespace paras;
    if (validate(args) != PARAS_OK) return "invalid";
    switch (choose(*args)) {
        case SdpaKernel::Flash:  return flash_uses_wide(*args) ? "flash_mfma_wide" : "flash_mfma";
        case SdpaKernel::Decode: return "decode_split";
        case SdpaKernel::Weights: return "math_mfma";
        case SdpaKernel::Padded: return "padded_mfma";
        case SdpaKernel::Composed: return "composed";
        default:                 return "generic";
    }
}

size_t paras_sdpa_workspace(const paras_sdpa_args* args) {
    using namespace paras;
    if (validate(args) != PARAS_OK || empty_output(*args)) return 0;
    switch (choose(*args)) {
        case SdpaKernel::Decode:  return decode_workspace(*args);
        case SdpaKernel::Generic: return generic_workspace(*args);
        case SdpaKernel::Composed: return composed_workspace(*args);
        case SdpaKernel::Padded: {
            PaddedPlan pl;
            return plan_padded(*args, &pl) ? pl.total : 0;
        }
        default:                  return 0;
    }
}

int paras_sdpa_fwd(const paras_sdpa_args* args, void* workspace, void* stream) {
    using namespace paras;
    int rc = validate(args);
    if (rc != PARAS_OK) return rc;
    const paras_sdpa_args& a = *args;
    if (empty_output(a)) return PARAS_OK;
    PARAS_REQUIRE(a.out != nullptr, "paras sdpa: null output pointer");
    PARAS_REQUIRE(a.Lk == 0 || (a.q && a.k && a.v), "paras sdpa: null tensor pointer");   // (empty k / v have no storage)
    hipStream_t s = nullptr;
    rc = resolve_stream(stream, &s);
    if (rc != PARAS_OK) return rc;
    if (a.Lk == 0) {
        // softmax over nothing, then a product with an empty inner dim: zeros.
        // (a fill kernel rather than hipMemsetAsync: callers may be capturing this stream into a graph)
        const int esz = a.dtype == PARAS_F64 ? 8 : a.dtype == PARAS_F32 ? 4 : 2;
        const int64_t n = a.B * a.Hq * a.Lq * a.Dv, one = 1;
        return paras_fill_strided(a.out, 1, &n, &one, esz, 0, stream);
    }
    switch (choose(a)) {
        case SdpaKernel::Flash: return launch_flash(a, s);
        case SdpaKernel::Weights: return launch_weights(a, s);
        case SdpaKernel::Padded: return launch_padded(a, workspace, stream, s);
        case SdpaKernel::Composed: return launch_composed(a, workspace, stream, s);
        case SdpaKernel::Decode:
            PARAS_REQUIRE(workspace != nullptr || decode_workspace(a) == 0, "paras sdpa: workspace is null");
            return launch_decode(a, workspace, s);
        default: return launch_generic(a, workspace, s);
    }
}

}  // extern "C"
