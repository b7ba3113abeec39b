// producers.hip — normalisation and gated-activation kernels that emit the block_q8_1x activation stream of the
// int-dot GEMVs together with their fp16 output, so that no separate quantize launch is needed
// (src/ops/elementwise.cpp:136-191, src/ops/deltanet.cpp:73-130).  The quantizer sees the
// ROUNDED fp16 outputs: the stream is bit-identical to quantize_q8_1 run on y afterwards.
#include "mxq_device.h"
#include "mxq_host.h"

namespace mxq {

constexpr int kNormThreads = 256;

// sum over the workgroup; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = group_sum<64>(v);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    if (lane == 63) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (uint32_t w = 0; w < (blockDim.x + 63) / 64; ++w) t += red[w];
    __syncthreads();
    return t;
}

// GATED = false: y = half((x * r) * w),            x fp16, w fp32      (rms_norm_f32w_q8)
// GATED = true : y = half((w * (x * r)) * silu(z)), x fp32, w, z fp16   (gated_rms_norm_q8)
// r = rsqrt(mean(x^2) + eps).  One workgroup per row; thread t of pass p owns the 4 elements
// 4 (256 p + t) .. +3, so 8 consecutive threads own one 32-element block.
template <bool GATED, class XT, class WT>
__global__ __launch_bounds__(kNormThreads) void norm_q8_kernel(const XT* x, const half_t* z, const WT* w, half_t* y, uint8_t* q8, uint32_t hidden, float eps) {
    __shared__ float red[kNormThreads / 64];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const XT* xr = x + (size_t)row * hidden;
    float sum = 0.f;
    for (uint32_t i = tid * 4; i < hidden; i += kNormThreads * 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float v = load_act(xr + i + j);
            sum += v * v;
        }
    }
    sum = block_sum(sum, red);
    const float r = rsqrtf(sum / (float)hidden + eps);
    half_t* yr = y + (size_t)row * hidden;
    uint8_t* qr = q8 + (size_t)row * (hidden / 32) * kQ81xBytes;
    const uint32_t n_pass = (hidden + kNormThreads * 4 - 1) / (kNormThreads * 4);
    for (uint32_t p = 0; p < n_pass; ++p) {
        const uint32_t i = (p * kNormThreads + tid) * 4;
        const bool live = i < hidden;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (live) {
            half_t h4[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float o;
                if (GATED) {
                    const float xn = load_act(xr + i + j) * r;
                    const float gz = (float)z[(size_t)row * hidden + i + j];
                    o = ((float)w[i + j] * xn) * (gz / (1.f + __expf(-gz)));
                } else {
                    o = (load_act(xr + i + j) * r) * (float)w[i + j];
                }
                h4[j] = (half_t)o;
                v[j] = (float)h4[j];
            }
            *reinterpret_cast<uint2*>(yr + i) = *reinterpret_cast<const uint2*>(h4);
        }
        emit_q8_1x(v, tid & 7u, live, qr + (size_t)(i / 32) * kQ81xBytes);
    }
}

// y = half(silu(gate) * up) (swiglu, src/ops/elementwise.cpp:449-467) or, OAI = true, the clamped
// gpt-oss form x = min(gate, limit), z = clamp(up, -limit, limit), y = half(x * sigmoid(alpha x) * (z + 1))
// (swiglu_oai, :469-492), written as fp16 (when y != NULL) and as the block_q8_1x stream of the rounded
// values: the down projection's int-dot input without a quantize launch.  Thread = 4 elements.
template <bool OAI>
__global__ __launch_bounds__(256) void act_q8_kernel(const half_t* gate, const half_t* up, half_t* y, uint8_t* q8, uint64_t n, float alpha, float limit) {
    const uint64_t i = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const bool live = i < n;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        half_t g4[4], u4[4], h4[4];
        *reinterpret_cast<uint2*>(g4) = *reinterpret_cast<const uint2*>(gate + i);
        *reinterpret_cast<uint2*>(u4) = *reinterpret_cast<const uint2*>(up + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float o;
            if (OAI) {
                const float x = fminf((float)g4[j], limit), z = fmaxf(fminf((float)u4[j], limit), -limit);
                o = (x / (1.f + __expf(alpha * (-x)))) * (z + 1.f);
            } else {
                const float g = (float)g4[j];
                o = (g / (1.f + __expf(-g))) * (float)u4[j];
            }
            h4[j] = (half_t)o;
            v[j] = (float)h4[j];
        }
        if (y) *reinterpret_cast<uint2*>(y + i) = *reinterpret_cast<const uint2*>(h4);
    }
    emit_q8_1x(v, threadIdx.x & 7u, live, q8 + (i / 32) * kQ81xBytes);
}

template <bool OAI>
static int act_q8(mx_stream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* y, void* q8_out, uint64_t n, float alpha, float limit) {
    MX_REQUIRE_PTR(gate); MX_REQUIRE_PTR(up); MX_REQUIRE_PTR(q8_out);
    MX_REQUIRE_SHAPE(n > 0 && n % 32 == 0 && (n / 4 + 255) / 256 <= 0x7FFFFFFFull);
    MX_REQUIRE_ALIGN(gate, 8); MX_REQUIRE_ALIGN(up, 8); MX_REQUIRE_ALIGN(y, 8); MX_REQUIRE_ALIGN(q8_out, 8);
    hipLaunchKernelGGL((act_q8_kernel<OAI>), dim3((uint32_t)((n / 4 + 255) / 256)), dim3(256), 0, as_stream(s), reinterpret_cast<const half_t*>(gate),
                       reinterpret_cast<const half_t*>(up), reinterpret_cast<half_t*>(y), static_cast<uint8_t*>(q8_out), n, alpha, limit);
    return launch_status();
}

static int check_norm(const void* x, const void* w, const void* y, const void* q8, uint32_t n_rows, uint32_t hidden) {
    MX_REQUIRE_PTR(x); MX_REQUIRE_PTR(w); MX_REQUIRE_PTR(y); MX_REQUIRE_PTR(q8);
    MX_REQUIRE_SHAPE(n_rows > 0 && hidden > 0 && hidden % 32 == 0);
    MX_REQUIRE_ALIGN(y, 8); MX_REQUIRE_ALIGN(q8, 8);
    return MX_OK;
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_rms_norm_f32w_q8(mx_stream_t s, const uint16_t* x, const float* w, uint16_t* y, void* q8_out, uint32_t n_rows, uint32_t hidden, float eps) {
    if (int rc = check_norm(x, w, y, q8_out, n_rows, hidden)) return rc;
    hipLaunchKernelGGL((norm_q8_kernel<false, half_t, float>), dim3(n_rows), dim3(kNormThreads), 0, as_stream(s), reinterpret_cast<const half_t*>(x),
                       (const half_t*)nullptr, w, reinterpret_cast<half_t*>(y), static_cast<uint8_t*>(q8_out), hidden, eps);
    return launch_status();
}

int mx_gated_rms_norm_q8(mx_stream_t s, const float* x, const uint16_t* z, const uint16_t* weight, uint16_t* y, void* q8_out, uint32_t n_rows,
                         uint32_t hidden, float eps) {
    if (int rc = check_norm(x, weight, y, q8_out, n_rows, hidden)) return rc;
    MX_REQUIRE_PTR(z);
    hipLaunchKernelGGL((norm_q8_kernel<true, float, half_t>), dim3(n_rows), dim3(kNormThreads), 0, as_stream(s), x, reinterpret_cast<const half_t*>(z),
                       reinterpret_cast<const half_t*>(weight), reinterpret_cast<half_t*>(y), static_cast<uint8_t*>(q8_out), hidden, eps);
    return launch_status();
}

int mx_swiglu_q8(mx_stream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* y, void* q8_out, uint64_t n) {
    return act_q8<false>(s, gate, up, y, q8_out, n, 0.f, 0.f);
}
int mx_swiglu_oai_q8(mx_stream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* y, void* q8_out, uint64_t n, float alpha, float limit) {
    return act_q8<true>(s, gate, up, y, q8_out, n, alpha, limit);
}

}  // extern "C"
