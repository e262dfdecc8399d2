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

constexpr std::size_t kMinBlock   = 256;
constexpr std::size_t kPow2Limit  = std::size_t{1} << 30;  // 1 GiB
constexpr std::size_t kLargeAlign = std::size_t{256} << 20;  // 256 MiB

}  // namespace

HbmPool::HbmPool(int device)
    : device_(device),
      caching_(!env_flag("PARAS_NO_CACHE")),
      debug_(env_flag("PARAS_DEBUG_ALLOC")) {}

HbmPool::~HbmPool() {
    // Process teardown: the HIP runtime may already be gone, so cached blocks
    // are left to the driver instead of calling hipFree from a static
    // destructor.
}

std::size_t HbmPool::round_size(std::size_t nbytes) {
    if (nbytes <= kMinBlock) return kMinBlock;
    if (nbytes > kPow2Limit)
        return (nbytes + kLargeAlign - 1) / kLargeAlign * kLargeAlign;
    std::size_t r = kMinBlock;
    while (r < nbytes) r <<= 1;
    return r;
}

int HbmPool::acquire(std::size_t nbytes, void** out) {
    const std::size_t rounded = round_size(nbytes);
    {
        std::lock_guard<std::mutex> g(mutex_);
        auto it = free_lists_.find(rounded);
        if (it != free_lists_.end() && !it->second.empty()) {
            void* p = it->second.back();
            it->second.pop_back();
            cached_ -= rounded;
            live_[p] = rounded;
            if (debug_) std::fprintf(stderr, "[paras] pool[%d] reuse %zu @%p\n", device_, rounded, p);
            *out = p;
            return PARAS_OK;
        }
    }
    PARAS_HIP_TRY(hipSetDevice(device_));
    void* p = nullptr;
    hipError_t err = hipMalloc(&p, rounded);
    if (err != hipSuccess) {
        // One retry after handing cached blocks back to the driver.
        (void)hipGetLastError();
        (void)hipDeviceSynchronize();
        clear();
        err = hipMalloc(&p, rounded);
    }
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fail(PARAS_ERR_OOM, "hipMalloc of %zu bytes on device %d failed: %s", rounded,
                    device_, hipGetErrorString(err));
    }
    {
        std::lock_guard<std::mutex> g(mutex_);
        live_[p] = rounded;
        allocated_ += rounded;
    }
    if (debug_) std::fprintf(stderr, "[paras] pool[%d] alloc %zu @%p\n", device_, rounded, p);
    *out = p;
    return PARAS_OK;
}

int HbmPool::release(void* ptr) {
    if (ptr == nullptr) return PARAS_OK;
    std::size_t rounded = 0;
    {
        std::lock_guard<std::mutex> g(mutex_);
        auto it = live_.find(ptr);
        if (it == live_.end())
            return fail(PARAS_ERR_INVALID, "paras allocator: release of unknown pointer %p", ptr);
        rounded = it->second;
        live_.erase(it);
        if (caching_) {
            free_lists_[rounded].push_back(ptr);
            cached_ += rounded;
            if (debug_) std::fprintf(stderr, "[paras] pool[%d] cache %zu @%p\n", device_, rounded, ptr);
            return PARAS_OK;
        }
        allocated_ -= rounded;
    }
    if (debug_) std::fprintf(stderr, "[paras] pool[%d] free %zu @%p\n", device_, rounded, ptr);
    PARAS_HIP_TRY(hipSetDevice(device_));
    // hipFree waits for the device, so work still reading the block finishes.
    PARAS_HIP_TRY(hipFree(ptr));
    return PARAS_OK;
}

int HbmPool::clear() {
    std::map<std::size_t, std::vector<void*>> lists;
    {
        std::lock_guard<std::mutex> g(mutex_);
        lists.swap(free_lists_);
        for (auto& kv : lists) allocated_ -= kv.first * kv.second.size();
        cached_ = 0;
    }
    int status = PARAS_OK;
    if (!lists.empty()) (void)hipSetDevice(device_);
    for (auto& kv : lists)
        for (void* p : kv.second)
            if (hipFree(p) != hipSuccess) {
                (void)hipGetLastError();
                status = fail(PARAS_ERR_HIP, "hipFree failed while clearing pool[%d]", device_);
            }
    return status;
}

std::uint64_t HbmPool::allocated_bytes() const {
    std::lock_guard<std::mutex> g(mutex_);
    return allocated_;
}

std::uint64_t HbmPool::cached_bytes() const {
    std::lock_guard<std::mutex> g(mutex_);
    return cached_;
}

}  // namespace paras
