// mxq_host.h — host-side plumbing shared by the C-ABI translation units:
// argument checks that run before any HIP call, launch-error capture.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

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

// Partial-sum scratch of a split-K launch: either the library's own file-scope device array (resolved per device,
// see scratch_address) or a workspace the caller passed to a *_ws entry point.
struct SplitWs {
    float* ptr;        // device address
    uint64_t elems;    // capacity in floats
    bool caller;       // caller-owned: a launch that does not fit is an error instead of falling back to the unsplit kernel
};

// Device address of a file-scope __device__ array.  In host code the array's name is only a stand-in for the symbol:
// every device holds its own copy at its own address, which hipGetSymbolAddress returns for the CURRENT device.  The
// address is resolved once per device and kept in `slot` (one per array, indexed by device ordinal).
constexpr int kMaxDevices = 64;
template <class Sym>
inline int scratch_address(const Sym& symbol, std::atomic<void*> (&slot)[kMaxDevices], void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        g_last_hip_error = (int)(e != hipSuccess ? e : hipErrorInvalidDevice);
        return MX_ERR_LAUNCH;
    }
    void* p = slot[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, symbol);
        if (e != hipSuccess || !p) {
            g_last_hip_error = (int)(e != hipSuccess ? e : hipErrorInvalidSymbol);
            return MX_ERR_LAUNCH;
        }
        slot[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return MX_OK;
}

// gemv_q6_planes.hip: one token against one or two (gate and up) Q6_K plane sets; MX_ERR_UNSUPPORTED for a shape it
// does not take (K % 512, K > 16384, planes of 4 GB and more, misaligned scale planes)
int launch_gemv_q6_planes(hipStream_t st, int nseg, const void* x_q8, const uint8_t* const* lo, const uint8_t* const* hi, const int8_t* const* sc,
                          const uint16_t* const* d, uint16_t* const* y, uint32_t K, uint32_t N);

// per-device set-up of the translation units that own scratch arrays (mx_init)
int gemv_init_device();
int gemm_init_device();

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
