// Tensor lifecycle on the `paras` device: allocation, views, copies in every
// direction, fill, scalar read-back, and the boxed CPU fallback for every aten
// op this backend does not implement.
//
// Same contract as the reference's plumbing (csrc/ops/tensor_ops.cpp:36-69,
// 252-330, 971-1029), kept deliberately small: view ops that PyTorch already
// implements device-independently (permute, transpose, expand, slice, ...) are
// not re-registered.  Copies between the host and the device are blocking;
// device-side strided / converting copies run as kernels on the context stream.
#include <ATen/EmptyTensor.h>
#include <ATen/NativeFunctions.h>
#include <ATen/native/CPUFallback.h>
#include <ATen/native/Resize.h>
#include <c10/core/DeviceGuard.h>

#include <cstring>
#include <vector>

#include "paras_torch.h"

namespace paras_torch {
namespace {

using at::Tensor;

c10::Device resolve(c10::optional<c10::Device> device) {
    c10::Device d = device.value_or(c10::Device(kParas, current_device()));
    TORCH_CHECK(d.type() == kParas, "paras: expected a paras device, got ", d);
    if (!d.has_index()) d = c10::Device(kParas, current_device());
    (void)hip_device(d.index());       // raises for paras:0 under the reference's numbering and for indices out of range
    const int n = device_count_torch();
    TORCH_CHECK(d.index() >= 0 && d.index() < n, "paras: invalid device index ", static_cast<int>(d.index()),
                " (device count: ", n, ")");
    return d;
}

Tensor empty_memory_format(c10::IntArrayRef size, c10::optional<c10::ScalarType> dtype,
                           c10::optional<c10::Layout> layout, c10::optional<c10::Device> device,
                           c10::optional<bool> pin_memory, c10::optional<c10::MemoryFormat> memory_format) {
    TORCH_CHECK(!layout.has_value() || *layout == c10::kStrided, "paras: only strided tensors are supported");
    TORCH_CHECK(!pin_memory.value_or(false), "paras: pinned memory applies to host tensors only");
    const c10::Device d = resolve(device);
    const c10::DeviceGuard guard(d);
    constexpr c10::DispatchKeySet ks(c10::DispatchKey::PrivateUse1);
    return at::detail::empty_generic(size, c10::GetAllocator(kParas), ks, c10::dtype_or_default(dtype), memory_format);
}

Tensor empty_strided(c10::IntArrayRef size, c10::IntArrayRef stride, c10::optional<c10::ScalarType> dtype,
                     c10::optional<c10::Layout> layout, c10::optional<c10::Device> device,
                     c10::optional<bool> pin_memory) {
    TORCH_CHECK(!layout.has_value() || *layout == c10::kStrided, "paras: only strided tensors are supported");
    TORCH_CHECK(!pin_memory.value_or(false), "paras: pinned memory applies to host tensors only");
    const c10::Device d = resolve(device);
    const c10::DeviceGuard guard(d);
    constexpr c10::DispatchKeySet ks(c10::DispatchKey::PrivateUse1);
    return at::detail::empty_strided_generic(size, stride, c10::GetAllocator(kParas), ks, c10::dtype_or_default(dtype));
}

Tensor view(const Tensor& self, c10::IntArrayRef size) { return at::native::view(self, size); }

Tensor as_strided(const Tensor& self, c10::IntArrayRef size, c10::IntArrayRef stride,
                  c10::optional<int64_t> storage_offset) {
    return at::native::as_strided_tensorimpl(self, size, stride, storage_offset);
}

Tensor reshape_alias(const Tensor& self, c10::IntArrayRef size, c10::IntArrayRef stride) {
    return at::native::_reshape_alias(self, size, stride);
}

// ---- copies -----------------------------------------------------------------
bool dense_same_layout(const Tensor& a, const Tensor& b) {
    return a.is_contiguous() && b.is_contiguous() && a.sizes() == b.sizes();
}

// dst[...] = src[...] on one device, any strides; float<->float conversion on
// the device, other conversions through the host.
void device_copy(const Tensor& src, const Tensor& dst) {
    TORCH_CHECK(src.numel() == dst.numel() && src.sizes() == dst.sizes(),
                "paras copy_: element count mismatch (", src.sizes(), " vs ", dst.sizes(), ")");
    const bool same = src.scalar_type() == dst.scalar_type();
    const int sc = float_code(src.scalar_type()), dc = float_code(dst.scalar_type());
    if (!same && (sc < 0 || dc < 0)) {
        Tensor host = src.cpu().to(dst.scalar_type());
        const_cast<Tensor&>(dst).copy_(host);
        return;
    }
    TORCH_CHECK(src.dim() <= 8, "paras: tensor rank ", src.dim(), " exceeds kernel limit of 8");
    check(paras_copy_strided(src.data_ptr(), dst.data_ptr(), static_cast<int>(src.dim()), src.sizes().data(),
                             src.strides().data(), dst.strides().data(), static_cast<int>(src.element_size()),
                             same ? 0 : sc, same ? 0 : dc, stream_for(dst)));
}

Tensor copy_from(const Tensor& self, const Tensor& dst, bool non_blocking) {
    (void)non_blocking;  // host <-> device copies are blocking, as in the reference
    if (self.numel() == 0) return dst;
    const bool src_dev = is_paras(self), dst_dev = is_paras(dst);
    const size_t nbytes_dst = static_cast<size_t>(dst.numel()) * dst.element_size();

    if (src_dev && dst.device().is_cpu()) {
        const int dev = hip_device(self);
        Tensor staged = self;
        if (!self.is_contiguous() || self.scalar_type() != dst.scalar_type()) {
            const bool convertible = self.scalar_type() == dst.scalar_type() ||
                                     (float_code(self.scalar_type()) >= 0 && float_code(dst.scalar_type()) >= 0);
            staged = empty_paras(self.sizes(), convertible ? dst.scalar_type() : self.scalar_type(), self.device());
            device_copy(self, staged);
        }
        // copy_() reaches this function before any broadcasting: a source of fewer elements than
        // the destination takes the second branch, which copies staged.numel() elements and lets
        // the host copy expand them.
        if (staged.scalar_type() == dst.scalar_type() && dst.is_contiguous() && staged.sizes().equals(dst.sizes())) {
            check(paras_memcpy(dev, dst.data_ptr(), staged.data_ptr(), nbytes_dst, 1));
        } else {
            Tensor host = at::empty(staged.sizes(), staged.options().device(c10::kCPU));
            check(paras_memcpy(dev, host.data_ptr(), staged.data_ptr(),
                               static_cast<size_t>(staged.numel()) * staged.element_size(), 1));
            const_cast<Tensor&>(dst).copy_(host);
        }
        return dst;
    }
    if (self.device().is_cpu() && dst_dev) {
        const int dev = hip_device(dst);
        Tensor src_c = self.expand_as(dst);
        if (src_c.scalar_type() != dst.scalar_type()) src_c = src_c.to(dst.scalar_type());
        src_c = src_c.contiguous();
        if (dst.is_contiguous()) {
            check(paras_memcpy(dev, dst.data_ptr(), src_c.data_ptr(), nbytes_dst, 0));
        } else {
            Tensor staged = empty_paras(dst.sizes(), dst.scalar_type(), dst.device());
            check(paras_memcpy(dev, staged.data_ptr(), src_c.data_ptr(), nbytes_dst, 0));
            device_copy(staged, dst);
        }
        return dst;
    }
    if (src_dev && dst_dev) {
        if (self.device().index() != dst.device().index()) {
            Tensor host = at::empty(self.sizes(), self.options().device(c10::kCPU).dtype(dst.scalar_type()));
            copy_from(self, host, false);
            copy_from(host, dst, false);
            return dst;
        }
        if (dense_same_layout(self, dst) && self.scalar_type() == dst.scalar_type())
            check(paras_memcpy(hip_device(dst), dst.data_ptr(), self.data_ptr(), nbytes_dst, 2));
        else
            device_copy(self, dst);
        return dst;
    }
    TORCH_CHECK(false, "paras _copy_from: unsupported device pair ", self.device(), " -> ", dst.device());
}

Tensor copy_from_and_resize(const Tensor& self, const Tensor& dst) {
    if (dst.sizes() != self.sizes()) const_cast<Tensor&>(dst).resize_(self.sizes());
    return copy_from(self, dst, false);
}

// ---- fill / scalar ------------------------------------------------------------
Tensor& fill_scalar(Tensor& self, const c10::Scalar& value) {
    if (self.numel() == 0) return self;
    Tensor v = at::scalar_tensor(value, at::TensorOptions().dtype(self.scalar_type()).device(c10::kCPU));
    uint64_t bits = 0;
    std::memcpy(&bits, v.data_ptr(), self.element_size());
    TORCH_CHECK(self.dim() <= 8, "paras: tensor rank ", self.dim(), " exceeds kernel limit of 8");
    check(paras_fill_strided(self.data_ptr(), static_cast<int>(self.dim()), self.sizes().data(), self.strides().data(),
                             static_cast<int>(self.element_size()), bits, stream_for(self)));
    return self;
}

Tensor& zero_(Tensor& self) { return fill_scalar(self, 0); }

c10::Scalar local_scalar_dense(const Tensor& self) {
    TORCH_CHECK(self.numel() == 1, "paras: a tensor with ", self.numel(), " elements cannot be converted to a scalar");
    Tensor host = at::empty({}, self.options().device(c10::kCPU));
    check(paras_memcpy(hip_device(self), host.data_ptr(), self.data_ptr(), self.element_size(), 1));
    return at::_local_scalar_dense(host);
}

// ---- storage bookkeeping --------------------------------------------------------
Tensor& set_storage_offset_size(Tensor& self, at::Storage source, int64_t storage_offset, c10::IntArrayRef size,
                                c10::IntArrayRef stride) {
    auto* impl = self.unsafeGetTensorImpl();
    impl->set_storage_keep_dtype(std::move(source));
    impl->set_storage_offset(storage_offset);
    if (stride.data() != nullptr && stride.size() == size.size()) impl->set_sizes_and_strides(size, stride);
    else impl->set_sizes_contiguous(size);
    return self;
}

Tensor& set_storage(Tensor& self, at::Storage source) {
    const int64_t n = static_cast<int64_t>(source.nbytes() / self.dtype().itemsize());
    return set_storage_offset_size(self, std::move(source), 0, {n}, {});
}

const Tensor& resize_(const Tensor& self, c10::IntArrayRef size, c10::optional<c10::MemoryFormat> memory_format) {
    TORCH_CHECK(!memory_format.has_value() || *memory_format == c10::MemoryFormat::Contiguous,
                "paras resize_: only the contiguous memory format is supported");
    int64_t numel = 1;
    for (auto s : size) numel *= s;
    auto* impl = self.unsafeGetTensorImpl();
    const size_t need = static_cast<size_t>(numel + impl->storage_offset()) * self.element_size();
    if (need > self.storage().nbytes()) {
        const c10::DeviceGuard guard(self.device());
        c10::DataPtr fresh = c10::GetAllocator(kParas)->allocate(need);
        const size_t keep = self.storage().nbytes();
        if (keep > 0)
            check(paras_memcpy(hip_device(self), fresh.get(), self.storage().data(), keep, 2));
        check(paras_synchronize(hip_device(self)));
        self.storage().set_data_ptr_noswap(std::move(fresh));
        self.storage().set_nbytes(need);
    }
    impl->set_sizes_contiguous(size);
    return self;
}

bool has_compatible_shallow_copy_type(const Tensor& self, const Tensor& from) {
    return is_paras(self) == is_paras(from);
}

void cpu_fallback(const c10::OperatorHandle& op, torch::jit::Stack* stack) {
    static const bool verbose = [] {
        const char* v = std::getenv("PARAS_LOG");
        return v != nullptr && std::atoi(v) >= 1;
    }();
    if (verbose) std::fprintf(stderr, "[paras] falling back to CPU for %s\n", op.schema().operator_name().name.c_str());
    at::native::cpu_fallback(op, stack);
}

}  // namespace
}  // namespace paras_torch

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
    using namespace paras_torch;
    m.impl("aten::empty.memory_format", &empty_memory_format);
    m.impl("aten::empty_strided", &empty_strided);
    m.impl("aten::view", &view);
    m.impl("aten::as_strided", &as_strided);
    m.impl("aten::_reshape_alias", &reshape_alias);
    m.impl("aten::_copy_from", &copy_from);
    m.impl("aten::_copy_from_and_resize", &copy_from_and_resize);
    m.impl("aten::fill_.Scalar", &fill_scalar);
    m.impl("aten::zero_", &zero_);
    m.impl("aten::_local_scalar_dense", &local_scalar_dense);
    m.impl("aten::set_.source_Storage", &set_storage);
    m.impl("aten::set_.source_Storage_storage_offset", &set_storage_offset_size);
    m.impl("aten::resize_", &resize_);
    m.impl("aten::_has_compatible_shallow_copy_type", &has_compatible_shallow_copy_type);
}

TORCH_LIBRARY_IMPL(_, PrivateUse1, m) {
    m.fallback(torch::CppFunction::makeFromBoxedFunction<&paras_torch::cpu_fallback>());
}

TORCH_LIBRARY_IMPL(_, AutogradPrivateUse1, m) { m.fallback(torch::CppFunction::makeFallthrough()); }
