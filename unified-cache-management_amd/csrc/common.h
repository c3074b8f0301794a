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

// Device-side accessors for pointers that were read from a pointer table in
// memory.  The compiler cannot tell that such a pointer is global memory and
// would emit flat loads, whose completion it can only wait for with the
// counters at zero: a prefetch issued before the wait then never overlaps
// anything.  Every pointer handed to this library is device-visible global
// memory (HBM or pinned host memory), so the cast is always valid.
namespace ucm {
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define UCM_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ u32x4 gload16(const void* p) { return *(const UCM_GLOBAL u32x4*)p; }
__device__ __forceinline__ u32x4 gload16_nt(const void* p)
{
    return __builtin_nontemporal_load((const UCM_GLOBAL u32x4*)p);
}
__device__ __forceinline__ void gstore16(void* p, const u32x4 v) { *(UCM_GLOBAL u32x4*)p = v; }
__device__ __forceinline__ void gstore16_nt(void* p, const u32x4 v)
{
    __builtin_nontemporal_store(v, (UCM_GLOBAL u32x4*)p);
}
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
