// Shared host-side plumbing for the gfx950 backend: status/last-error
// handling, the per-device workspace, and small launch helpers.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>
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

// Library-owned scratch for reduction partials, gathered matrices and split-K partial
// sums: one buffer per (device, stream, kind), grown on demand and never shrunk, so calls
// on different streams do not share scratch and calls on one stream are ordered by it.
// A buffer that is outgrown stays allocated while any captured graph exists (its address
// may be baked into the graph).  `fresh` reports that the buffer was (re)allocated by
// this request and holds no defined contents.
int stream_buffer(int kind, size_t nbytes, size_t min_bytes, hipStream_t stream, void** ptr, bool* fresh);
// kind 0: the general workspace (at least 4 MiB); 1 / 2: stream-K counters / slabs;
// 3: raw accumulators and operand sums of a layer with affine weights
int workspace(size_t nbytes, hipStream_t stream, void** ptr);
// Split-K scratch of one stream: arrival counters (zero between launches: the finisher of a
// tile resets its counter) and slabs for the partial results, whose layout the kernel defines.
struct SkScratch {
    int* counters = nullptr;
    int32_t* slabs = nullptr;
};
int sk_scratch(size_t counters, size_t slab_bytes, hipStream_t st, SkScratch* out);
// Resolves, for the current device, the address of the static scratch array that
// lq_minmax_noalloc uses (called by lq_init; the entry point does it on first use otherwise).
int minmax_noalloc_init();

// A launch site's once-per-device set-up (the dynamic LDS limit of a kernel is a per-device
// attribute of the function): one bit per device, taken under a mutex, so that the first calls
// of two threads, or on two devices, neither race nor skip it.
struct DeviceOnce {
    std::atomic<uint32_t> done{0};
    std::mutex mu;
};
template <class F>
int device_once(DeviceOnce& o, F&& setup) {
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < 32, LQ_ERR_DEVICE, "device index %d out of range", dev);
    const uint32_t bit = 1u << dev;
    if (o.done.load(std::memory_order_acquire) & bit) return LQ_OK;
    std::lock_guard<std::mutex> lock(o.mu);
    if (o.done.load(std::memory_order_relaxed) & bit) return LQ_OK;
    const int rc = setup();
    if (rc == LQ_OK) o.done.fetch_or(bit, std::memory_order_release);
    return rc;
}
// the common case: kernel `fn` may use up to `bytes` of dynamic LDS
inline int allow_dynamic_lds(DeviceOnce& o, const void* fn, int bytes) {
    return device_once(o, [&]() -> int {
        LQ_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        return LQ_OK;
    });
}

inline hipStream_t as_stream(lq_stream s) { return reinterpret_cast<hipStream_t>(s); }

__host__ __device__ inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// erf for the GELU kernels: Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7 (the rational
// term through v_rcp_f32, the Gaussian through v_exp_f32), 13 instructions where the
// library erff takes about 45 with both of its branches live in a wavefront.  The GELU
// it feeds, 0.5 x (1 + erf(x / sqrt 2)), is within 1e-6 of the exactly rounded one for
// every x (the error peaks for |x| < 4.2; beyond |x| = 5.6 the result is x or 0 exactly
// as with erff).  Not for erf on its own near 0: 1 - p e cancels there.
__device__ __forceinline__ float erf_as(float v) {
    const float z = __builtin_fabsf(v);
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.0f));
    float p = __builtin_fmaf(1.061405429f, t, -1.453152027f);
    p = __builtin_fmaf(p, t, 1.421413741f);
    p = __builtin_fmaf(p, t, -0.284496736f);
    p = __builtin_fmaf(p, t, 0.254829592f);
    p = p * t;
    const float e = __builtin_amdgcn_exp2f((z * z) * -1.4426950408889634f);
    return __builtin_copysignf(__builtin_fmaf(-p, e, 1.0f), v);
}

}  // namespace lq
