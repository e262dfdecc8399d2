// Shared definitions of the PyTorch side of the `paras` device.
//
// This translation-unit group (compiled by g++, no HIP headers) owns the
// dispatcher registrations and tensor bookkeeping; everything that touches
// the GPU goes through the C ABI of libparas_hip.so (include/paras_hip.h).
#pragma once

#include <ATen/ATen.h>
#include <c10/core/Device.h>
#include <c10/util/Exception.h>
#include <torch/library.h>

#include <initializer_list>
#include <utility>

#include "paras_hip.h"

namespace paras_torch {

constexpr c10::DeviceType kParas = c10::DeviceType::PrivateUse1;

// Converts a C-ABI status into the reference's error convention: a c10::Error
// (RuntimeError in Python) carrying the library's message.
inline void check(int rc) {
    TORCH_CHECK(rc == PARAS_OK, paras_last_error());
}

inline bool is_paras(const at::Tensor& t) { return t.device().type() == kParas; }

// Every tensor argument of an op must live on the same `paras` device before any of its
// pointers reaches a kernel: the dispatcher picks the PrivateUse1 kernel as soon as ONE
// argument is on the device, and a host pointer handed to a HIP kernel is a GPU memory
// fault rather than an error.  Raises (RuntimeError in Python) on the host, before any launch.
inline void require_same_device(const char* op, const at::Tensor& ref, std::initializer_list<std::pair<const char*, const at::Tensor*>> others) {
    TORCH_CHECK(is_paras(ref), op, ": expected a tensor on a paras device, got ", ref.device());
    for (const auto& o : others) {
        if (o.second == nullptr || !o.second->defined()) continue;
        TORCH_CHECK(is_paras(*o.second) && o.second->device() == ref.device(), op, ": argument `", o.first, "` is on ",
                    o.second->device(), " but the op runs on ", ref.device(), "; move it with .to('", ref.device(), "') first");
    }
}
inline void require_same_dtype(const char* op, const at::Tensor& ref, std::initializer_list<std::pair<const char*, const at::Tensor*>> others) {
    for (const auto& o : others) {
        if (o.second == nullptr || !o.second->defined()) continue;
        TORCH_CHECK(o.second->scalar_type() == ref.scalar_type(), op, ": argument `", o.first, "` has dtype ", o.second->scalar_type(),
                    ", expected ", ref.scalar_type());
    }
}

// paras_dtype code of a floating tensor type, or -1.
inline int float_code(c10::ScalarType t) {
    switch (t) {
        case c10::kFloat:    return PARAS_F32;
        case c10::kHalf:     return PARAS_F16;
        case c10::kBFloat16: return PARAS_BF16;
        case c10::kDouble:   return PARAS_F64;
        default:             return -1;
    }
}

inline int require_float_code(const at::Tensor& t, const char* op) {
    const int c = float_code(t.scalar_type());
    TORCH_CHECK(c >= 0, op, ": unsupported dtype ", t.scalar_type());
    return c;
}

// Device numbering.  By default `paras:i` is HIP GPU i.  With PARAS_DEVICE_BASE=1 in the
// environment the package numbers devices as the reference does (csrc/compat/paras_compat.cpp:
// 87-97: device 0 is the host CPU engine, GPUs start at 1): `paras:i` is then HIP GPU i - 1 and
// `paras:0` raises, because this build has no host engine.  device_base() is 0 or 1;
// device_count_torch() is the number of `paras` indices (GPUs + base); hip_device() maps a
// `paras` index to the library's HIP index or raises.
int device_base();
int device_count_torch();
int hip_device(c10::DeviceIndex index);
inline int hip_device(const at::Tensor& t) { return hip_device(t.device().index()); }

// Makes `index` the calling thread's HIP device and returns the context
// stream every `paras` op of that device is queued on.
void* stream_for(c10::DeviceIndex index);
inline void* stream_for(const at::Tensor& t) { return stream_for(t.device().index()); }

// Thread-local current device index (the device guard's state).
c10::DeviceIndex current_device();

// Fresh tensor on the `paras` device.
at::Tensor empty_paras(c10::IntArrayRef sizes, c10::ScalarType dtype, c10::Device device);

// Device scratch memory for one op call (returned to the pool when it dies).
at::Tensor workspace(size_t nbytes, c10::Device device);

// Value of a double after one trip through `dtype` (double -> float -> T), the
// narrowing the reference applies to a wrapped scalar (to_compute,
// csrc/ops/pointwise_ops.cpp:55-60).
double narrow_scalar(double v, c10::ScalarType dtype);

}  // namespace paras_torch
