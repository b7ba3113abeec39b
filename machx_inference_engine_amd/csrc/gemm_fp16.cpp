// gemm_fp16.cpp — gemm_fp16_onednn: the reference's vendor-library matmul (oneDNN, src/ops/gemm_onednn.cpp:75-111;
// fp16 in and out, fp32 accumulate) maps onto the vendor library of this platform, rocBLAS' gemm_ex.  rocBLAS is loaded
// on first use, so the rest of the library carries no dependency on it.  (The reference's own tiled kernel, gemm_fp16
// with fp32 output, is the hand-written kernel in gemm_f16_tiled.hip.)
#include <dlfcn.h>
#include <rocblas/rocblas.h>

#include <mutex>

#include "mxq_host.h"

namespace {

struct RocblasApi {
    decltype(&rocblas_create_handle) create = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_gemm_ex) gemm_ex = nullptr;
    bool ok = false;
};

constexpr int kMaxDevices = 16;
std::mutex g_mu;
RocblasApi g_api;
bool g_tried = false;
rocblas_handle g_handle[kMaxDevices] = {};

bool load_api() {
    if (g_tried) return g_api.ok;
    g_tried = true;
    void* h = dlopen("librocblas.so", RTLD_NOW | RTLD_LOCAL);   // the unversioned name first, then the sonames ROCm 6 / 7 ship
    for (const char* name : {"librocblas.so.5", "librocblas.so.4"})
        if (!h) h = dlopen(name, RTLD_NOW | RTLD_LOCAL);
    if (!h) return false;
    g_api.create = reinterpret_cast<decltype(g_api.create)>(dlsym(h, "rocblas_create_handle"));
    g_api.set_stream = reinterpret_cast<decltype(g_api.set_stream)>(dlsym(h, "rocblas_set_stream"));
    g_api.gemm_ex = reinterpret_cast<decltype(g_api.gemm_ex)>(dlsym(h, "rocblas_gemm_ex"));
    g_api.ok = g_api.create && g_api.set_stream && g_api.gemm_ex;
    return g_api.ok;
}

// C[M,N] = A[M,K] . B[K,N], all row-major; column-major view: C^T[N,M] = B^T[N,K] . A^T[K,M].
int gemm_rowmajor(mx_stream_t s, const void* A, const void* B, void* C, rocblas_datatype c_type, uint32_t M, uint32_t N, uint32_t K) {
    MX_REQUIRE_PTR(A); MX_REQUIRE_PTR(B); MX_REQUIRE_PTR(C);
    MX_REQUIRE_SHAPE(M > 0 && N > 0 && K > 0 && M <= 0x7FFFFFFFu && N <= 0x7FFFFFFFu && K <= 0x7FFFFFFFu);
    MX_REQUIRE_ALIGN(A, 2); MX_REQUIRE_ALIGN(B, 2);
    std::lock_guard<std::mutex> lock(g_mu);
    if (!load_api()) return MX_ERR_UNSUPPORTED;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MX_ERR_LAUNCH;
    if (!g_handle[dev] && g_api.create(&g_handle[dev]) != rocblas_status_success) return MX_ERR_LAUNCH;
    if (g_api.set_stream(g_handle[dev], mxq::as_stream(s)) != rocblas_status_success) return MX_ERR_LAUNCH;
    const float alpha = 1.f, beta = 0.f;
    const rocblas_status st =
        g_api.gemm_ex(g_handle[dev], rocblas_operation_none, rocblas_operation_none, (rocblas_int)N, (rocblas_int)M, (rocblas_int)K, &alpha, B,
                      rocblas_datatype_f16_r, (rocblas_int)N, A, rocblas_datatype_f16_r, (rocblas_int)K, &beta, C, c_type, (rocblas_int)N, C, c_type,
                      (rocblas_int)N, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success) {
        mxq::g_last_hip_error = (int)st;
        return MX_ERR_LAUNCH;
    }
    return MX_OK;
}

}  // namespace

extern "C" {

int mx_gemm_fp16_onednn(mx_stream_t s, const uint16_t* A, const uint16_t* B, uint16_t* y, uint32_t M, uint32_t N, uint32_t K) {
    return gemm_rowmajor(s, A, B, y, rocblas_datatype_f16_r, M, N, K);
}

}  // extern "C"
