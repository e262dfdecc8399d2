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

enum class SdpaKernel { Flash, Decode, Weights, Generic };

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

SdpaKernel choose(const paras_sdpa_args& a) {
    if (decode_supported(a)) return SdpaKernel::Decode;
    if (flash_supported(a)) return SdpaKernel::Flash;
    if (weights_supported(a)) return SdpaKernel::Weights;
    return SdpaKernel::Generic;
}

}  // namespace
}  // namespace paras

extern "C" {

const char* paras_sdpa_kernel_name(const paras_sdpa_args* args) {
    using namespace paras;
    if (validate(args) != PARAS_OK) return "invalid";
    switch (choose(*args)) {
        case SdpaKernel::Flash:  return "flash_mfma";
        case SdpaKernel::Decode: return "decode_split";
        case SdpaKernel::Weights: return "math_mfma";
        default:                 return "generic";
    }
}

size_t paras_sdpa_workspace(const paras_sdpa_args* args) {
    using namespace paras;
    if (validate(args) != PARAS_OK || empty_output(*args)) return 0;
    switch (choose(*args)) {
        case SdpaKernel::Decode:  return decode_workspace(*args);
        case SdpaKernel::Generic: return generic_workspace(*args);
        default:                  return 0;
    }
}

int paras_sdpa_fwd(const paras_sdpa_args* args, void* workspace, void* stream) {
    using namespace paras;
    int rc = validate(args);
    if (rc != PARAS_OK) return rc;
    const paras_sdpa_args& a = *args;
    if (empty_output(a)) return PARAS_OK;
    PARAS_REQUIRE(a.q && a.k && a.v && a.out, "paras sdpa: null tensor pointer");
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
        case SdpaKernel::Decode:
            PARAS_REQUIRE(workspace != nullptr || decode_workspace(a) == 0, "paras sdpa: workspace is null");
            return launch_decode(a, workspace, s);
        default: return launch_generic(a, workspace, s);
    }
}

}  // extern "C"
