// Shared host/device helpers of libmi355_int8.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <utility>

#include "../../include/mi355_int8.h"

namespace mi {

extern thread_local int32_t g_last_hip_error;

inline int32_t hip_fail(hipError_t e)
{
    g_last_hip_error = (int32_t)e;
    return MI_EIO;
}

#define MI_HIP(expr)                                     \
    do {                                                 \
        hipError_t _e = (expr);                          \
        if (_e != hipSuccess) return ::mi::hip_fail(_e); \
    } while (0)

// every kernel launch is followed by this: reports a bad launch configuration
// as MI_EIO without synchronizing
inline int32_t launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? MI_OK : hip_fail(e);
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned4(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

int32_t compute_units();   // of the current device, cached
int32_t lds_limit();       // largest LDS allocation of one workgroup on the current device, cached

// A kernel's dynamic-LDS limit is a setting of the (kernel, device) pair: raised once for every device that the
// kernel is launched on, and refused where the device cannot give that much.  One LdsOptIn per kernel
// instantiation (a function-local static); a race between two first launches only repeats the call.
struct LdsOptIn {
    std::atomic<uint64_t> devices{0};
};
inline int32_t lds_opt_in(LdsOptIn &st, const void *kernel, int bytes)
{
    int dev = 0;
    MI_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return MI_EINVAL;
    const uint64_t bit = 1ull << dev;
    if (st.devices.load(std::memory_order_acquire) & bit) return MI_OK;
    if (bytes > lds_limit()) return MI_ENOSPC;
    MI_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    st.devices.fetch_or(bit, std::memory_order_release);
    return MI_OK;
}
#define MI_LDS_OPT_IN(kernel, bytes)                                                              \
    do {                                                                                          \
        static ::mi::LdsOptIn _st;                                                                \
        const int32_t _rc = ::mi::lds_opt_in(_st, reinterpret_cast<const void *>(kernel), bytes); \
        if (_rc != MI_OK) return _rc;                                                             \
    } while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{}): a loop whose index is a
// compile-time constant inside the body (register arrays indexed by it stay in registers)
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

}  // namespace mi
