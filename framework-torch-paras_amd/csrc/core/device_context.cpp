#include "core/device_context.h"

#include <pthread.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "core/status.h"

namespace paras {

namespace {

thread_local char tl_error[512] = {0};

bool g_bad_fork = false;
void forked_child() { g_bad_fork = true; }

int log_level() {
    static const int level = [] {
        const char* v = std::getenv("PARAS_LOG");
        return v ? std::atoi(v) : 0;
    }();
    return level;
}

}  // namespace

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
    va_end(ap);
    if (log_level() >= 1) std::fprintf(stderr, "[paras] error %d: %s\n", code, tl_error);
    return code;
}

void clear_error() { tl_error[0] = '\0'; }

const char* last_error_text() { return tl_error; }

DeviceContext::DeviceContext() {
    static std::once_flag fork_once;
    std::call_once(fork_once, [] { pthread_atfork(nullptr, nullptr, forked_child); });

    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        count = 0;
    }
    for (int i = 0; i < count; ++i) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, i) != hipSuccess) {
            (void)hipGetLastError();
            continue;
        }
        auto st = std::make_unique<DeviceState>();
        st->index         = static_cast<int>(devices_.size());
        st->name          = prop.name;
        st->arch          = prop.gcnArchName;
        st->compute_units = prop.multiProcessorCount;
        st->hbm_bytes     = prop.totalGlobalMem;
        st->pool          = std::make_unique<HbmPool>(i);
        if (log_level() >= 1)
            std::fprintf(stderr, "[paras] device %d: %s (%s, %d CUs, %.1f GB)\n", st->index,
                         st->name.c_str(), st->arch.c_str(), st->compute_units,
                         st->hbm_bytes / 1e9);
        devices_.push_back(std::move(st));
    }
}

DeviceContext& DeviceContext::instance() {
    static DeviceContext* ctx = new DeviceContext();  // never destroyed: outlives HIP teardown
    return *ctx;
}

DeviceState* DeviceContext::device(int index) {
    if (index < 0 || index >= device_count()) {
        fail(device_count() == 0 ? PARAS_ERR_NO_DEVICE : PARAS_ERR_INVALID,
             "paras: invalid device index %d (device count: %d)", index, device_count());
        return nullptr;
    }
    return devices_[index].get();
}

int DeviceContext::stream(int index, hipStream_t* out) {
    DeviceState* st = device(index);
    if (st == nullptr) return device_count() == 0 ? PARAS_ERR_NO_DEVICE : PARAS_ERR_INVALID;
    PARAS_HIP_TRY(hipSetDevice(index));
    std::call_once(st->stream_once, [st] {
        // Default priority on purpose: one stream per device, nothing to rank.
        hipError_t e = hipStreamCreateWithFlags(&st->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            st->stream_status = fail(PARAS_ERR_HIP, "hipStreamCreateWithFlags failed: %s",
                                     hipGetErrorString(e));
        }
    });
    if (st->stream_status != 0) return st->stream_status;
    *out = st->stream;
    return PARAS_OK;
}

int DeviceContext::synchronize(int index) {
    hipStream_t s = nullptr;
    int rc = stream(index, &s);
    if (rc != PARAS_OK) return rc;
    PARAS_HIP_TRY(hipStreamSynchronize(s));
    return PARAS_OK;
}

bool DeviceContext::bad_fork() {
    instance();
    return g_bad_fork;
}

int resolve_stream(void* stream_arg, hipStream_t* out) {
    if (DeviceContext::instance().device_count() == 0)
        return fail(PARAS_ERR_NO_DEVICE, "paras: no HIP device is visible");
    *out = static_cast<hipStream_t>(stream_arg);
    return PARAS_OK;
}

}  // namespace paras

// ---------------------------------------------------------------------------
// C ABI: library state, device context, allocator, copies
// ---------------------------------------------------------------------------
namespace paras { const char* last_error_text(); }

extern "C" {

const char* paras_last_error(void) { return paras::last_error_text(); }

int paras_abi_version(void) { return 1; }

int paras_device_count(void) { return paras::DeviceContext::instance().device_count(); }

int paras_is_bad_fork(void) { return paras::DeviceContext::bad_fork() ? 1 : 0; }

int paras_device_name(int device, char* buf, size_t buflen) {
    auto* st = paras::DeviceContext::instance().device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    PARAS_REQUIRE(buf != nullptr && buflen > 0, "paras_device_name: empty buffer");
    std::snprintf(buf, buflen, "%s", st->name.c_str());
    return PARAS_OK;
}

int paras_device_info(int device, int* compute_units, uint64_t* hbm_bytes) {
    auto* st = paras::DeviceContext::instance().device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    if (compute_units) *compute_units = st->compute_units;
    if (hbm_bytes) *hbm_bytes = st->hbm_bytes;
    return PARAS_OK;
}

int paras_stream(int device, void** stream_out) {
    PARAS_REQUIRE(stream_out != nullptr, "paras_stream: null output");
    hipStream_t s = nullptr;
    int rc = paras::DeviceContext::instance().stream(device, &s);
    if (rc == PARAS_OK) *stream_out = s;
    return rc;
}

int paras_synchronize(int device) { return paras::DeviceContext::instance().synchronize(device); }

int paras_alloc(int device, size_t nbytes, void** ptr_out) {
    PARAS_REQUIRE(ptr_out != nullptr, "paras_alloc: null output");
    auto* st = paras::DeviceContext::instance().device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    return st->pool->acquire(nbytes, ptr_out);
}

int paras_free(int device, void* ptr) {
    auto* st = paras::DeviceContext::instance().device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    return st->pool->release(ptr);
}

int paras_empty_cache(int device) {
    auto& ctx = paras::DeviceContext::instance();
    auto* st  = ctx.device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    int rc = ctx.synchronize(device);
    if (rc != PARAS_OK) return rc;
    return st->pool->clear();
}

int paras_memory_stats(int device, uint64_t* allocated, uint64_t* cached) {
    auto* st = paras::DeviceContext::instance().device(device);
    if (st == nullptr) return PARAS_ERR_INVALID;
    if (allocated) *allocated = st->pool->allocated_bytes();
    if (cached) *cached = st->pool->cached_bytes();
    return PARAS_OK;
}

size_t paras_round_size(size_t nbytes) { return paras::HbmPool::round_size(nbytes); }

int paras_memcpy(int device, void* dst, const void* src, size_t nbytes, int kind) {
    if (nbytes == 0) return PARAS_OK;
    PARAS_REQUIRE(dst != nullptr && src != nullptr, "paras_memcpy: null pointer");
    PARAS_REQUIRE(kind >= 0 && kind <= 2, "paras_memcpy: kind must be 0, 1 or 2");
    hipStream_t s = nullptr;
    int rc = paras::DeviceContext::instance().stream(device, &s);
    if (rc != PARAS_OK) return rc;
    const hipMemcpyKind k = kind == 0   ? hipMemcpyHostToDevice
                            : kind == 1 ? hipMemcpyDeviceToHost
                                        : hipMemcpyDeviceToDevice;
    PARAS_HIP_TRY(hipMemcpyAsync(dst, src, nbytes, k, s));
    if (kind != 2) PARAS_HIP_TRY(hipStreamSynchronize(s));
    return PARAS_OK;
}

int paras_memset(int device, void* dst, int value, size_t nbytes) {
    if (nbytes == 0) return PARAS_OK;
    PARAS_REQUIRE(dst != nullptr, "paras_memset: null pointer");
    hipStream_t s = nullptr;
    int rc = paras::DeviceContext::instance().stream(device, &s);
    if (rc != PARAS_OK) return rc;
    PARAS_HIP_TRY(hipMemsetAsync(dst, value, nbytes, s));
    return PARAS_OK;
}

}  // extern "C"
