// `paras` as a PyTorch PrivateUse1 device: device guard, hooks and allocator.
//
// Mirrors the registration the reference performs (csrc/core/registration.cpp:
// 34-95, csrc/core/allocator.cpp:129-173) on top of the HIP-only context:
// device i is HIP device i, one context stream per device (stream id 0), the
// allocator hands out blocks of the binned HBM pool.
#include <ATen/detail/PrivateUse1HooksInterface.h>
#include <c10/core/Allocator.h>
#include <c10/core/impl/DeviceGuardImplInterface.h>
#include <torch/version.h>

#include <cstdlib>

#include "paras_torch.h"

#if TORCH_VERSION_MAJOR < 2 || (TORCH_VERSION_MAJOR == 2 && TORCH_VERSION_MINOR < 4)
#error "torch_paras requires PyTorch >= 2.4"
#endif

namespace paras_torch {
namespace {

int read_device_base() {
    const char* v = std::getenv("PARAS_DEVICE_BASE");
    return (v != nullptr && v[0] == '1' && v[1] == '\0') ? 1 : 0;
}
const int g_device_base = read_device_base();

// The thread's current device: the first GPU under either numbering.
thread_local c10::DeviceIndex tl_device = static_cast<c10::DeviceIndex>(g_device_base);

struct GuardImpl final : public c10::impl::DeviceGuardImplInterface {
    c10::DeviceType type() const override { return kParas; }
    c10::Device exchangeDevice(c10::Device d) const override {
        const c10::Device prev(kParas, tl_device);
        tl_device = d.index();
        return prev;
    }
    c10::Device getDevice() const override { return c10::Device(kParas, tl_device); }
    void setDevice(c10::Device d) const override { tl_device = d.index(); }
    void uncheckedSetDevice(c10::Device d) const noexcept override { tl_device = d.index(); }
    c10::Stream getStream(c10::Device d) const noexcept override { return c10::Stream(c10::Stream::UNSAFE, d, 0); }
    c10::Stream getDefaultStream(c10::Device d) const override { return getStream(d); }
    c10::Stream exchangeStream(c10::Stream) const noexcept override { return getStream(c10::Device(kParas, tl_device)); }
    c10::DeviceIndex deviceCount() const noexcept override { return static_cast<c10::DeviceIndex>(paras_device_count() + g_device_base); }
    bool queryStream(const c10::Stream&) const override { return true; }
    void synchronizeStream(const c10::Stream& s) const override { check(paras_synchronize(hip_device(s.device().index()))); }
    void synchronizeDevice(const c10::DeviceIndex index) const override { check(paras_synchronize(hip_device(index))); }
};

GuardImpl g_guard;
c10::impl::DeviceGuardImplRegistrar g_guard_registrar(kParas, &g_guard);

struct Hooks final : public at::PrivateUse1HooksInterface {
    bool hasPrimaryContext(c10::DeviceIndex index) const override {
        return index >= g_device_base && index < paras_device_count() + g_device_base;
    }
    bool isAvailable() const override { return paras_device_count() > 0; }
};

struct HooksRegistrar {
    Hooks hooks;
    HooksRegistrar() { at::RegisterPrivateUse1HooksInterface(&hooks); }
} g_hooks_registrar;

// DataPtr context: which pool (HIP device index) the block goes back to.
struct Block {
    void* ptr;
    int   device;
};

void release_block(void* opaque) {
    if (opaque == nullptr) return;
    auto* b = static_cast<Block*>(opaque);
    // A failure here (unknown pointer) cannot throw out of a deleter; the pool
    // keeps its message in paras_last_error().
    (void)paras_free(b->device, b->ptr);
    delete b;
}

struct Allocator final : public c10::Allocator {
    c10::DataPtr allocate(size_t nbytes) override {
        const c10::DeviceIndex index = tl_device;
        const int dev = hip_device(index);
        void* p = nullptr;
        if (nbytes > 0) check(paras_alloc(dev, nbytes, &p));
        auto* b = new Block{p, dev};
        return c10::DataPtr(p, b, &release_block, c10::Device(kParas, index));
    }
    c10::DeleterFnPtr raw_deleter() const override { return &release_block; }
    void copy_data(void* dest, const void* src, std::size_t count) const override {
        check(paras_memcpy(hip_device(tl_device), dest, src, count, 2));
        check(paras_synchronize(hip_device(tl_device)));
    }
};

Allocator g_allocator;
REGISTER_ALLOCATOR(kParas, &g_allocator);

}  // namespace

c10::DeviceIndex current_device() { return tl_device; }

int device_base() { return g_device_base; }
int device_count_torch() { return paras_device_count() + g_device_base; }

int hip_device(c10::DeviceIndex index) {
    TORCH_CHECK(!(g_device_base == 1 && index == 0),
                "paras:0 is the host CPU engine in the reference's numbering (PARAS_DEVICE_BASE=1); this build has no host "
                "engine: GPUs are paras:1 .. paras:", paras_device_count());
    const int hip = static_cast<int>(index) - g_device_base;
    TORCH_CHECK(hip >= 0 && hip < paras_device_count(), "paras: invalid device index ", static_cast<int>(index),
                " (device count: ", device_count_torch(), ")");
    return hip;
}

void* stream_for(c10::DeviceIndex index) {
    void* s = nullptr;
    check(paras_stream(hip_device(index), &s));
    return s;
}

at::Tensor empty_paras(c10::IntArrayRef sizes, c10::ScalarType dtype, c10::Device device) {
    return at::empty(sizes, at::TensorOptions().dtype(dtype).device(device));
}

at::Tensor workspace(size_t nbytes, c10::Device device) {
    return at::empty({static_cast<int64_t>(nbytes > 0 ? nbytes : 1)}, at::TensorOptions().dtype(c10::kByte).device(device));
}

double narrow_scalar(double v, c10::ScalarType dtype) {
    switch (dtype) {
        case c10::kFloat:    return static_cast<double>(static_cast<float>(v));
        case c10::kBFloat16: return static_cast<double>(static_cast<float>(c10::BFloat16(static_cast<float>(v))));
        case c10::kHalf:     return static_cast<double>(static_cast<float>(c10::Half(static_cast<float>(v))));
        default:             return v;
    }
}

}  // namespace paras_torch
