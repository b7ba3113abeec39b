// mxq_host.h — host-side plumbing shared by the C-ABI translation units:
// argument checks that run before any HIP call, launch-error capture.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mxq.h"

namespace mxq {

extern thread_local int g_last_hip_error;

inline hipStream_t as_stream(mx_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return MX_ERR_LAUNCH;
    }
    return MX_OK;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace mxq

#define MX_REQUIRE_PTR(p) \
    do {                  \
        if (!(p)) return MX_ERR_NULL; \
    } while (0)
#define MX_REQUIRE_SHAPE(c) \
    do {                    \
        if (!(c)) return MX_ERR_SHAPE; \
    } while (0)
#define MX_REQUIRE_ALIGN(p, a) \
    do {                       \
        if (!mxq::aligned((p), (a))) return MX_ERR_ALIGN; \
    } while (0)
