// Binned caching allocator over hipMalloc, one instance per device.
//
// Keeps the reference pool's contract (csrc/core/allocator.cpp:53-122):
// requests are rounded to a power of two of at least 256 bytes, a freed block
// goes to the free list of its size class and is handed out again for the
// next request of that class, `clear()` returns cached blocks to the driver.
// Differences, on purpose: the backing store is device HBM from hipMalloc
// (the reference's GPU flavor used managed memory), and size classes above
// 1 GiB round to a multiple of 256 MiB instead of the next power of two, so a
// 4.3 GB tensor does not pin 8 GiB of the 288 GB.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace paras {

class HbmPool {
public:
    explicit HbmPool(int device);
    ~HbmPool();

    static std::size_t round_size(std::size_t nbytes);

    // 0 on success; PARAS_ERR_OOM when hipMalloc fails even after the cache
    // has been flushed once.
    int acquire(std::size_t nbytes, void** out);
    // PARAS_ERR_INVALID for a pointer this pool did not hand out.
    int release(void* ptr);
    // hipFree()s every cached block.  The caller synchronizes first.
    int clear();

    std::uint64_t allocated_bytes() const;  // live + cached
    std::uint64_t cached_bytes() const;

private:
    int  device_;
    bool caching_;
    bool debug_;

    mutable std::mutex mutex_;
    std::map<std::size_t, std::vector<void*>> free_lists_;
    std::unordered_map<void*, std::size_t>    live_;
    std::uint64_t allocated_ = 0;
    std::uint64_t cached_    = 0;
};

}  // namespace paras
