// Shared host/device helpers of libmi355_int8.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

}  // namespace mi
