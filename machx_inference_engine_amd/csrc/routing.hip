// routing.hip — MoE routing and packing on the device, so that a layer never waits for the host
// between the router and the expert kernels:
//   router logits + softmax + top-k + renormalise + ascending-id order   src/ops/moe.cpp:22-216
//   softmax + top-k from logits already on the device                     src/ops/moe.cpp:366-412
//   packing arrays for one token                                          src/ops/moe.cpp:423-446
//   packing arrays for T tokens: stable counting sort by expert           src/model/qwen3moe_pack.cpp:5-31
#include "mxq_device.h"
#include "mxq_host.h"

namespace mxq {

// ---------------------------------------------------------------- router logits
// logit[t, e] = sum_h W_gate[e, h] * x[t, h]: one wave per (expert, token), fp32 weights,
// 4 elements per lane per step (16-byte weight loads).
__global__ __launch_bounds__(256) void router_logits_kernel(const half_t* x, const float* W, float* logits, uint32_t hidden, uint32_t E) {
    const uint32_t lane = threadIdx.x & 63u, e = blockIdx.x * 4u + (threadIdx.x >> 6), t = blockIdx.y;
    float acc = 0.f;
    if (e < E) {
        const float* wr = W + (size_t)e * hidden;
        const half_t* xr = x + (size_t)t * hidden;
        for (uint32_t i = lane * 4; i < hidden; i += 256) {
            const float4 w4 = *reinterpret_cast<const float4*>(wr + i);
            const uint2 xu = *reinterpret_cast<const uint2*>(xr + i);
            acc += w4.x * h2f(xu.x & 0xFFFFu) + w4.y * h2f(xu.x >> 16) + w4.z * h2f(xu.y & 0xFFFFu) + w4.w * h2f(xu.y >> 16);
        }
    }
    acc = group_sum<64>(acc);
    if (lane == 63 && e < E) logits[(size_t)t * E + e] = acc;
}

// ---------------------------------------------------------------- softmax + top-k
constexpr int kMaxTopK = 64;

__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
    return v;
}
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const unsigned long long o = __shfl_xor(v, d);
        v = o > v ? o : v;
    }
    return v;
}

// One workgroup per token, one thread per expert (E <= 1024).  p = softmax(logits); K rounds of
// a workgroup-wide maximum over the keys (bits(p) << 32 | e) — positive float bits are
// monotonic, an exact tie goes to the higher expert id — then thread 0 renormalises the K
// winners and orders them by ascending expert id.
template <class LogitT>
__global__ __launch_bounds__(1024) void topk_kernel(const LogitT* logits, int32_t* topk_idx, half_t* topk_w, uint32_t E, uint32_t K) {
    __shared__ float red_f[16];
    __shared__ unsigned long long red_k[16];
    __shared__ int32_t idx_s[kMaxTopK];
    __shared__ float w_s[kMaxTopK];
    const uint32_t e = threadIdx.x, t = blockIdx.x, lane = e & 63u, wave = e >> 6, n_waves = (blockDim.x + 63) / 64;
    const bool in = e < E;
    const float logit = in ? load_act(logits + (size_t)t * E + e) : -INFINITY;
    float m = wave_max_f(logit);
    if (lane == 0) red_f[wave] = m;
    __syncthreads();
    m = red_f[0];
    for (uint32_t w = 1; w < n_waves; ++w) m = fmaxf(m, red_f[w]);
    __syncthreads();
    const float ev = in ? __expf(logit - m) : 0.f;
    float s = group_sum<64>(ev);
    if (lane == 63) red_f[wave] = s;
    __syncthreads();
    s = 0.f;
    for (uint32_t w = 0; w < n_waves; ++w) s += red_f[w];
    const float p = ev / s;
    bool live = in;
    for (uint32_t kk = 0; kk < K; ++kk) {
        const unsigned long long key = live ? (((unsigned long long)f2u(p) << 32) | e) : 0ull;
        const unsigned long long wm = wave_max_u64(key);
        __syncthreads();
        if (lane == 0) red_k[wave] = wm;
        __syncthreads();
        unsigned long long win = red_k[0];
        for (uint32_t w = 1; w < n_waves; ++w) win = red_k[w] > win ? red_k[w] : win;
        if (live && e == (uint32_t)(win & 0xFFFFFFFFull)) {
            live = false;
            idx_s[kk] = (int32_t)e;
            w_s[kk] = u2f((uint32_t)(win >> 32));
        }
    }
    __syncthreads();
    if (e == 0) {
        float ren = 0.f;
        for (uint32_t kk = 0; kk < K; ++kk) ren += w_s[kk];
        const float inv = 1.0f / ren;
        for (uint32_t kk = 0; kk < K; ++kk) w_s[kk] *= inv;
        for (uint32_t i = 0; i + 1 < K; ++i)
            for (uint32_t j = 0; j + 1 + i < K; ++j)
                if (idx_s[j] > idx_s[j + 1]) {
                    const int32_t ti = idx_s[j]; idx_s[j] = idx_s[j + 1]; idx_s[j + 1] = ti;
                    const float tw = w_s[j]; w_s[j] = w_s[j + 1]; w_s[j + 1] = tw;
                }
    }
    __syncthreads();
    if (e < K) {
        topk_idx[(size_t)t * K + e] = idx_s[e];
        topk_w[(size_t)t * K + e] = (half_t)w_s[e];
    }
}

// ---------------------------------------------------------------- packing
// One token (src/ops/moe.cpp:423-446): offsets by counting, identity order.
__global__ void pack_decode_kernel(const int32_t* topk_idx, const half_t* topk_w, uint32_t* expert_offsets, int32_t* sorted_idx, int32_t* tk_to_packed,
                                   half_t* weights_packed, uint32_t E, uint32_t K) {
    // thread e counts the slots routed below e
    for (uint32_t e = threadIdx.x; e <= E; e += blockDim.x) {
        uint32_t below = 0;
        for (uint32_t kk = 0; kk < K; ++kk) below += ((uint32_t)topk_idx[kk] < e) ? 1u : 0u;
        expert_offsets[e] = below;
    }
    for (uint32_t kk = threadIdx.x; kk < K; kk += blockDim.x) {
        sorted_idx[kk] = 0;
        tk_to_packed[kk] = (int32_t)kk;
        weights_packed[kk] = topk_w[kk];
    }
}

// T tokens: stable counting sort of the T*K slots by expert id, in three launches.
//   count : workgroup e counts its slots                      -> expert_offsets[e + 1]
//   scan  : one workgroup turns the counts into offsets        (inclusive scan in place)
//   place : workgroup e walks the slots in order and writes its own, keeping slot order
__global__ __launch_bounds__(256) void pack_count_kernel(const int32_t* topk_idx, uint32_t n_slots, uint32_t* expert_offsets) {
    __shared__ uint32_t red[4];
    const uint32_t e = blockIdx.x;
    uint32_t c = 0;
    for (uint32_t i = threadIdx.x; i < n_slots; i += 256) c += ((uint32_t)topk_idx[i] == e) ? 1u : 0u;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) c += (uint32_t)__shfl_xor((int)c, d);
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        expert_offsets[e + 1] = red[0] + red[1] + red[2] + red[3];
        if (e == 0) expert_offsets[0] = 0;
    }
}
__global__ __launch_bounds__(64) void pack_scan_kernel(uint32_t* expert_offsets, uint32_t E) {
    // one wave: running inclusive scan over chunks of 64 counts
    const uint32_t lane = threadIdx.x;
    uint32_t base = 0;
    for (uint32_t e0 = 0; e0 < E; e0 += 64) {
        const uint32_t e = e0 + lane;
        uint32_t v = e < E ? expert_offsets[e + 1] : 0u;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = (uint32_t)__shfl_up((int)v, d);
            if (lane >= (uint32_t)d) v += o;
        }
        if (e < E) expert_offsets[e + 1] = base + v;
        base += (uint32_t)__shfl((int)v, 63);
    }
}
__global__ __launch_bounds__(256) void pack_place_kernel(const int32_t* topk_idx, const half_t* topk_w, uint32_t n_slots, uint32_t K,
                                                         const uint32_t* expert_offsets, int32_t* sorted_idx, half_t* weights_packed,
                                                         int32_t* tk_to_packed) {
    __shared__ uint32_t wave_cnt[4];
    const uint32_t e = blockIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t base = expert_offsets[e];
    if (expert_offsets[e + 1] == base) return;
    for (uint32_t i0 = 0; i0 < n_slots; i0 += 256) {
        const uint32_t i = i0 + threadIdx.x;
        const bool mine = i < n_slots && (uint32_t)topk_idx[i] == e;
        const unsigned long long mask = __ballot(mine);
        const uint32_t before = (uint32_t)__builtin_popcountll(mask & ((1ull << lane) - 1ull));
        __syncthreads();
        if (lane == 0) wave_cnt[wave] = (uint32_t)__builtin_popcountll(mask);
        __syncthreads();
        uint32_t wave_base = 0;
        for (uint32_t w = 0; w < wave; ++w) wave_base += wave_cnt[w];
        if (mine) {
            const uint32_t p = base + wave_base + before;
            sorted_idx[p] = (int32_t)(i / K);
            weights_packed[p] = topk_w[i];
            tk_to_packed[i] = (int32_t)p;
        }
        base += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    }
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_moe_topk_from_logits(mx_stream_t s, const uint16_t* logits, int32_t* topk_idx, uint16_t* topk_w, uint32_t E, uint32_t K, uint32_t n_tokens) {
    MX_REQUIRE_PTR(logits); MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w);
    MX_REQUIRE_SHAPE(E > 0 && E <= 1024 && K > 0 && K <= E && K <= (uint32_t)kMaxTopK && n_tokens > 0);
    hipLaunchKernelGGL((topk_kernel<half_t>), dim3(n_tokens), dim3((E + 63) / 64 * 64), 0, as_stream(s), reinterpret_cast<const half_t*>(logits), topk_idx,
                       reinterpret_cast<half_t*>(topk_w), E, K);
    return launch_status();
}

int mx_moe_router(mx_stream_t s, const uint16_t* x, const float* W_gate, int32_t* topk_idx, uint16_t* topk_w, uint32_t n_tokens, uint32_t hidden,
                  uint32_t n_experts, uint32_t k, float* logits_ws) {
    MX_REQUIRE_PTR(x); MX_REQUIRE_PTR(W_gate); MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w); MX_REQUIRE_PTR(logits_ws);
    MX_REQUIRE_SHAPE(n_tokens > 0 && n_tokens <= 65535 && hidden > 0 && hidden % 4 == 0 && n_experts > 0 && n_experts <= 1024 && k > 0 && k <= n_experts &&
                     k <= (uint32_t)kMaxTopK);
    MX_REQUIRE_ALIGN(x, 8); MX_REQUIRE_ALIGN(W_gate, 16);
    hipLaunchKernelGGL(router_logits_kernel, dim3((n_experts + 3) / 4, n_tokens), dim3(256), 0, as_stream(s), reinterpret_cast<const half_t*>(x), W_gate,
                       logits_ws, hidden, n_experts);
    if (int rc = launch_status()) return rc;
    hipLaunchKernelGGL((topk_kernel<float>), dim3(n_tokens), dim3((n_experts + 63) / 64 * 64), 0, as_stream(s), (const float*)logits_ws, topk_idx,
                       reinterpret_cast<half_t*>(topk_w), n_experts, k);
    return launch_status();
}

int mx_moe_build_pack_decode(mx_stream_t s, const int32_t* topk_idx, const uint16_t* topk_w, uint32_t* expert_offsets, int32_t* sorted_idx,
                             int32_t* tk_to_packed, uint16_t* weights_packed, uint32_t E, uint32_t K) {
    MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w); MX_REQUIRE_PTR(expert_offsets); MX_REQUIRE_PTR(sorted_idx); MX_REQUIRE_PTR(tk_to_packed);
    MX_REQUIRE_PTR(weights_packed);
    MX_REQUIRE_SHAPE(E > 0 && K > 0);
    hipLaunchKernelGGL(pack_decode_kernel, dim3(1), dim3(256), 0, as_stream(s), topk_idx, reinterpret_cast<const half_t*>(topk_w), expert_offsets, sorted_idx,
                       tk_to_packed, reinterpret_cast<half_t*>(weights_packed), E, K);
    return launch_status();
}

int mx_moe_build_packing_device(mx_stream_t s, const int32_t* topk_idx, const uint16_t* topk_w, uint32_t T, uint32_t K, uint32_t E, uint32_t* expert_offsets,
                                int32_t* sorted_idx, uint16_t* weights_packed, int32_t* tk_to_packed) {
    MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w); MX_REQUIRE_PTR(expert_offsets); MX_REQUIRE_PTR(sorted_idx); MX_REQUIRE_PTR(tk_to_packed);
    MX_REQUIRE_PTR(weights_packed);
    MX_REQUIRE_SHAPE(E > 0 && E <= 65535 && K > 0 && T > 0 && (uint64_t)T * K <= 0x7FFFFFFFull);
    const uint32_t n = T * K;
    hipStream_t st = as_stream(s);
    hipLaunchKernelGGL(pack_count_kernel, dim3(E), dim3(256), 0, st, topk_idx, n, expert_offsets);
    if (int rc = launch_status()) return rc;
    hipLaunchKernelGGL(pack_scan_kernel, dim3(1), dim3(64), 0, st, expert_offsets, E);
    if (int rc = launch_status()) return rc;
    hipLaunchKernelGGL(pack_place_kernel, dim3(E), dim3(256), 0, st, topk_idx, reinterpret_cast<const half_t*>(topk_w), n, K, (const uint32_t*)expert_offsets,
                       sorted_idx, reinterpret_cast<half_t*>(weights_packed), tk_to_packed);
    return launch_status();
}

}  // extern "C"
