// HIP-only device context: one entry per visible HIP device, each with its
// own non-blocking stream (default priority) and its own binned HBM pool.
//
// Takes the place of the reference's dual-vendor compat::Queue plus Context
// (csrc/compat/paras_compat.h:143-218, csrc/core/context.h:43-74): no device
// enum, no managed memory, no host engine -- device i is HIP device i.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "core/hbm_pool.h"

namespace paras {

struct DeviceState {
    int           index = 0;
    std::string   name;
    std::string   arch;            // gcnArchName, e.g. "gfx950:sramecc+:xnack-"
    int           compute_units = 0;
    std::uint64_t hbm_bytes = 0;
    hipStream_t   stream = nullptr;  // created on first use, with device current
    std::once_flag stream_once;
    int           stream_status = 0;
    std::unique_ptr<HbmPool> pool;
};

class DeviceContext {
public:
    // Built on first use; never throws.  With no visible device the table is
    // empty and every per-device call fails with PARAS_ERR_NO_DEVICE.
    static DeviceContext& instance();

    int device_count() const { return static_cast<int>(devices_.size()); }

    // nullptr (and last error set) when index is out of range.
    DeviceState* device(int index);

    // Makes `index` the calling thread's HIP device and returns its stream.
    int stream(int index, hipStream_t* out);

    int synchronize(int index);

    // True in a process forked after the context was built: HIP state does not
    // survive fork (same poison flag as csrc/core/context.cpp:33-38).
    static bool bad_fork();

private:
    DeviceContext();
    std::vector<std::unique_ptr<DeviceState>> devices_;
};

// Resolves the stream argument of an ABI call.  The stream is used as given
// (NULL is HIP's null stream) on the calling thread's current HIP device;
// fails with PARAS_ERR_NO_DEVICE when no HIP device is visible.
int resolve_stream(void* stream_arg, hipStream_t* out);

}  // namespace paras
