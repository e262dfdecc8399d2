#include "core/hbm_pool.h"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>

#include "core/status.h"

namespace paras {

namespace {

bool env_flag(const char* name) {
    const char* v = std::getenv(name);
    return v != nullptr && std::atoi(v) != 0;
}

constexpr int         kMinShift   = 8;                        // 256 B
constexpr int         kMaxShift   = 30;                       // 1 GiB
constexpr std::size_t kLargeAlign = std::size_t{256} << 20;   // 256 MiB

}  // namespace

HbmPool::HbmPool(int device)
    : device_(device), keep_idle_(!env_flag("PARAS_NO_CACHE")), trace_(env_flag("PARAS_DEBUG_ALLOC")) {}

HbmPool::~HbmPool() {
    // Process teardown: the HIP runtime may already be gone, so idle blocks are
    // left to the driver instead of calling hipFree from a static destructor.
}

std::size_t HbmPool::round_size(std::size_t nbytes) {
    if (nbytes <= (std::size_t{1} << kMinShift)) return std::size_t{1} << kMinShift;
    if (nbytes > (std::size_t{1} << kMaxShift)) return (nbytes + kLargeAlign - 1) / kLargeAlign * kLargeAlign;
    const int shift = 64 - __builtin_clzll(static_cast<unsigned long long>(nbytes - 1));
    return std::size_t{1} << shift;
}

int HbmPool::class_of(std::size_t rounded) {
    if (rounded > (std::size_t{1} << kMaxShift)) return kLargeClass;
    return __builtin_ctzll(static_cast<unsigned long long>(rounded)) - kMinShift;
}

void* HbmPool::take_idle(int cls, std::size_t rounded) {
    Bin& bin = bins_[cls];
    if (cls != kLargeClass) {
        if (bin.empty()) return nullptr;
        void* p = bin.back().ptr;
        bin.pop_back();
        return p;
    }
    // the large bin mixes sizes: most recently freed block of exactly this size
    for (std::size_t i = bin.size(); i-- > 0;)
        if (bin[i].bytes == rounded) {
            void* p = bin[i].ptr;
            bin.erase(bin.begin() + static_cast<std::ptrdiff_t>(i));
            return p;
        }
    return nullptr;
}

std::vector<HbmPool::Idle> HbmPool::detach_idle(std::size_t want) {
    std::vector<Idle> out;
    std::size_t got = 0;
    for (int cls = kLargeClass; cls >= 0 && (want == 0 || got < want); --cls) {
        Bin& bin = bins_[cls];
        while (!bin.empty() && (want == 0 || got < want)) {
            out.push_back(bin.back());
            got += bin.back().bytes;
            bin.pop_back();
        }
    }
    idle_ -= got;
    from_driver_ -= got;
    return out;
}

int HbmPool::free_detached(const std::vector<Idle>& blocks) {
    int status = PARAS_OK;
    if (!blocks.empty()) (void)hipSetDevice(device_);
    for (const Idle& b : blocks) {
        if (trace_) std::fprintf(stderr, "[paras] pool[%d] return %zu @%p\n", device_, b.bytes, b.ptr);
        if (hipFree(b.ptr) != hipSuccess) {
            (void)hipGetLastError();
            status = fail(PARAS_ERR_HIP, "hipFree failed while returning idle blocks of pool[%d]", device_);
        }
    }
    return status;
}

int HbmPool::acquire(std::size_t nbytes, void** out) {
    const std::size_t rounded = round_size(nbytes);
    const int cls = class_of(rounded);
    {
        std::lock_guard<std::mutex> g(lock_);
        if (void* p = take_idle(cls, rounded)) {
            idle_ -= rounded;
            in_use_.emplace(p, rounded);
            if (trace_) std::fprintf(stderr, "[paras] pool[%d] reuse %zu @%p\n", device_, rounded, p);
            *out = p;
            return PARAS_OK;
        }
    }
    PARAS_HIP_TRY(hipSetDevice(device_));
    void* p = nullptr;
    hipError_t err = hipMalloc(&p, rounded);
    // Out of memory: first give back as many idle bytes as the request needs (largest classes
    // first: fewest driver calls), then everything.
    for (int attempt = 0; err != hipSuccess && attempt < 2; ++attempt) {
        (void)hipGetLastError();
        std::vector<Idle> back;
        {
            std::lock_guard<std::mutex> g(lock_);
            if (idle_ == 0) break;
            back = detach_idle(attempt == 0 ? rounded : 0);
        }
        (void)hipDeviceSynchronize();    // nothing queued may still be using an idle block's memory
        (void)free_detached(back);
        err = hipMalloc(&p, rounded);
    }
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fail(PARAS_ERR_OOM, "hipMalloc of %zu bytes on device %d failed: %s", rounded, device_, hipGetErrorString(err));
    }
    {
        std::lock_guard<std::mutex> g(lock_);
        in_use_.emplace(p, rounded);
        from_driver_ += rounded;
    }
    if (trace_) std::fprintf(stderr, "[paras] pool[%d] alloc %zu @%p\n", device_, rounded, p);
    *out = p;
    return PARAS_OK;
}

int HbmPool::release(void* ptr) {
    if (ptr == nullptr) return PARAS_OK;
    std::size_t rounded = 0;
    {
        std::lock_guard<std::mutex> g(lock_);
        auto it = in_use_.find(ptr);
        if (it == in_use_.end()) return fail(PARAS_ERR_INVALID, "paras allocator: release of unknown pointer %p", ptr);
        rounded = it->second;
        in_use_.erase(it);
        if (keep_idle_) {
            bins_[class_of(rounded)].push_back(Idle{ptr, rounded});
            idle_ += rounded;
            if (trace_) std::fprintf(stderr, "[paras] pool[%d] keep %zu @%p\n", device_, rounded, ptr);
            return PARAS_OK;
        }
        from_driver_ -= rounded;
    }
    if (trace_) std::fprintf(stderr, "[paras] pool[%d] free %zu @%p\n", device_, rounded, ptr);
    PARAS_HIP_TRY(hipSetDevice(device_));
    // hipFree waits for the device, so work still reading the block finishes.
    PARAS_HIP_TRY(hipFree(ptr));
    return PARAS_OK;
}

int HbmPool::clear() {
    std::vector<Idle> back;
    {
        std::lock_guard<std::mutex> g(lock_);
        back = detach_idle(0);
    }
    return free_detached(back);
}

std::uint64_t HbmPool::allocated_bytes() const {
    std::lock_guard<std::mutex> g(lock_);
    return from_driver_;
}

std::uint64_t HbmPool::cached_bytes() const {
    std::lock_guard<std::mutex> g(lock_);
    return idle_;
}

}  // namespace paras
