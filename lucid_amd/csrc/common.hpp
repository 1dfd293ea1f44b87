// Shared host-side plumbing for the gfx950 backend: status/last-error
// handling, the per-device workspace, and small launch helpers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/lucid_hip.h"

namespace lq {

// Thread-local message of the last failing call (Lucid surfaces typed
// exceptions, lucid/_C/core/Error.h; the C ABI returns a status + message).
std::string& last_error();
int fail(int status, const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define LQ_HIP(expr)                                        \
    do {                                                    \
        hipError_t _e = (expr);                             \
        if (_e != hipSuccess) return lq::hip_fail(_e, #expr); \
    } while (0)

#define LQ_REQUIRE(cond, status, ...)                     \
    do {                                                  \
        if (!(cond)) return lq::fail(status, __VA_ARGS__); \
    } while (0)

#define LQ_CHECK_LAUNCH(name)                                          \
    do {                                                               \
        hipError_t _e = hipGetLastError();                             \
        if (_e != hipSuccess) return lq::hip_fail(_e, "launch " name); \
    } while (0)

// Per-device scratch for reduction partials and split-K partial sums.
// Grown on demand; never shrunk.  Calls that overlap on one device race on it.
int workspace(size_t nbytes, void** ptr);

inline hipStream_t as_stream(lq_stream s) { return reinterpret_cast<hipStream_t>(s); }

__host__ __device__ inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace lq
