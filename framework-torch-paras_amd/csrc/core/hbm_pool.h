// Caching allocator over hipMalloc, one instance per device.
//
// Contract (the reference pool's, csrc/core/allocator.cpp:53-122): a request is
// rounded up to a size class, a freed block is kept and handed out again for
// the next request of its class, `clear()` returns idle blocks to the driver.
//
// Built for a 288 GB part: classes are the powers of two from 256 B to 1 GiB,
// held in a fixed array indexed by the exponent (no tree walk under the lock);
// above 1 GiB a class is a multiple of 256 MiB, so a 4.3 GB tensor does not pin
// 8 GiB; the backing store is device HBM from hipMalloc (never managed memory);
// and when hipMalloc runs out the pool gives idle blocks back largest class
// first, only as many as the request needs, before it retries -- a full flush
// of a pool that holds tens of gigabytes of warm workspaces is the last resort,
// not the first.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace paras {

class HbmPool {
public:
    explicit HbmPool(int device);
    ~HbmPool();

    static std::size_t round_size(std::size_t nbytes);

    // 0 on success; PARAS_ERR_OOM when hipMalloc fails even after every idle
    // block has been given back.
    int acquire(std::size_t nbytes, void** out);
    // PARAS_ERR_INVALID for a pointer this pool did not hand out.
    int release(void* ptr);
    // hipFree()s every idle block.  The caller synchronizes first.
    int clear();

    std::uint64_t allocated_bytes() const;  // in use + idle
    std::uint64_t cached_bytes() const;     // idle

private:
    static constexpr int kPow2Classes = 23;            // 2^8 .. 2^30
    static constexpr int kLargeClass  = kPow2Classes;  // bin of everything above 1 GiB

    struct Idle {
        void*       ptr;
        std::size_t bytes;
    };
    using Bin = std::vector<Idle>;

    static int class_of(std::size_t rounded);
    // Pops an idle block of exactly `rounded` bytes, or returns nullptr.  Lock held.
    void* take_idle(int cls, std::size_t rounded);
    // Detaches idle blocks, largest class first, until `want` bytes are detached (all of them for
    // want == 0).  Lock held; the caller frees them without the lock.
    std::vector<Idle> detach_idle(std::size_t want);
    int free_detached(const std::vector<Idle>& blocks);

    const int  device_;
    const bool keep_idle_;
    const bool trace_;

    mutable std::mutex lock_;
    std::array<Bin, kPow2Classes + 1>     bins_;
    std::unordered_map<void*, std::size_t> in_use_;   // block -> class size
    std::uint64_t from_driver_ = 0;                    // bytes obtained from hipMalloc and not yet returned
    std::uint64_t idle_        = 0;                    // of those, bytes sitting in bins_
};

}  // namespace paras
