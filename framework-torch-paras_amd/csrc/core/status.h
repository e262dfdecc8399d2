// Error plumbing shared by every translation unit of libparas_hip.so.
//
// The C ABI reports failures as negative status codes plus a thread-local
// message; nothing throws across it.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>

#include "paras_hip.h"

namespace paras {

// Stores a printf-formatted message as the calling thread's last error and
// returns `code`, so call sites read `return fail(PARAS_ERR_INVALID, "...")`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Clears the calling thread's last error.
void clear_error();

}  // namespace paras

// Returns PARAS_ERR_HIP from the enclosing function when a HIP call fails.
#define PARAS_HIP_TRY(expr)                                                          \
    do {                                                                             \
        hipError_t paras_hip_err_ = (expr);                                          \
        if (paras_hip_err_ != hipSuccess)                                            \
            return ::paras::fail(PARAS_ERR_HIP, "%s failed: %s (%s:%d)", #expr,      \
                                 hipGetErrorString(paras_hip_err_), __FILE__,        \
                                 __LINE__);                                          \
    } while (0)

// Argument check: returns PARAS_ERR_INVALID with a message when cond is false.
#define PARAS_REQUIRE(cond, ...)                                                     \
    do {                                                                             \
        if (!(cond)) return ::paras::fail(PARAS_ERR_INVALID, __VA_ARGS__);           \
    } while (0)
