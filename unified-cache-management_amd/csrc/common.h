// Shared host-side helpers of libucm_hip.so: error text, argument checks,
// launch checks.  Device code lives in the .hip files next to this header.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ucm_hip.h"

namespace ucm {

// thread-local text of the last failure, returned by ucm_last_error()
char* error_buffer();
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int check_hip(hipError_t e, const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline hipStream_t as_stream(ucm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace ucm

#define UCM_REQUIRE(cond, ...)                                   \
    do {                                                         \
        if (!(cond)) { return ucm::fail(UCM_EINVAL, __VA_ARGS__); } \
    } while (0)

#define UCM_SUPPORTED(cond, ...)                                  \
    do {                                                          \
        if (!(cond)) { return ucm::fail(UCM_ENOTSUP, __VA_ARGS__); } \
    } while (0)

// after a kernel launch: surfaces bad launch configurations right away
#define UCM_LAUNCH_CHECK(name) return ucm::check_hip(hipGetLastError(), name)
