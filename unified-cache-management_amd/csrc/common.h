// Shared host-side helpers of the HIP library: status codes, per-thread error text,
// HIP error translation.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ucm_hip.h"

namespace ucm {

// Stores a printf-formatted message for ucm_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline int hip_fail(hipError_t e, const char* what)
{
    // hipGetLastError() resets the sticky error so that a later, unrelated call does not
    // report this failure again.
    (void)hipGetLastError();
    return fail(e == hipErrorOutOfMemory ? UCM_EOOM : UCM_ERROR, "%s: %s", what,
                hipGetErrorString(e));
}

#define UCM_HIP_TRY(expr)                                          \
    do {                                                           \
        hipError_t e__ = (expr);                                   \
        if (e__ != hipSuccess) return ::ucm::hip_fail(e__, #expr); \
    } while (0)

#define UCM_REQUIRE(cond, ...)                                        \
    do {                                                              \
        if (!(cond)) return ::ucm::fail(UCM_EPARAM, __VA_ARGS__);     \
    } while (0)

inline int launch_status(const char* kernel)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(UCM_ERROR, "launch of %s failed: %s", kernel, hipGetErrorString(e));
    return UCM_OK;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace ucm
