// quant_dequant.hip — activation quantizers (fp16/fp32 -> block_q8_1x / block_q8_1s),
// flat block dequant (Q8_0 / Q4_K / Q6_K / MXFP4 -> fp16 / fp32) and the
// transposed whole-matrix dequant (-> fp16 Bt[K,N]).
#include "mxq_device.h"
#include "mxq_host.h"

namespace mxq {

// ---------------------------------------------------------------- q8_1 quantizers
// 8 lanes per 32-element block, 4 elements per lane: amax and the quant sums
// reduce over the 8-lane group with DPP.  d = amax/127, inv = 127/amax (0 for a
// zero block), q = round-half-away(v*inv), s = d*float(sum q)
// (src/ops/gemv_q8dot.cpp:94-124; split sums s0/s1: :57-91).
template <class ActT>
__device__ __forceinline__ void load4(const ActT* p, float (&v)[4]);
template <>
__device__ __forceinline__ void load4<half_t>(const half_t* p, float (&v)[4]) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    v[0] = h2f(u.x & 0xFFFFu); v[1] = h2f(u.x >> 16); v[2] = h2f(u.y & 0xFFFFu); v[3] = h2f(u.y >> 16);
}
template <>
__device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
    const float4 f = *reinterpret_cast<const float4*>(p);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
}

template <class ActT, bool SPLIT>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const ActT* x, uint8_t* out, uint64_t n_blocks) {
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t b = gid >> 3;
    const uint32_t l8 = (uint32_t)gid & 7u;
    const bool live = b < n_blocks;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) load4<ActT>(x + b * 32 + l8 * 4, v);
    const float amax = group_max8(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    const float d = amax / 127.0f, inv = amax > 0.f ? 127.0f / amax : 0.f;
    int q[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = (int)roundf(v[i] * inv);
        sum += q[i];
    }
    const uint32_t packed = (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) | ((uint32_t)(q[2] & 0xFF) << 16) | ((uint32_t)(q[3] & 0xFF) << 24);
    if (SPLIT) {
        const int lo = group_sum8_i(l8 < 4 ? sum : 0), hi = group_sum8_i(l8 < 4 ? 0 : sum);
        if (!live) return;
        uint8_t* blk = out + b * kQ81sBytes;
        reinterpret_cast<uint32_t*>(blk + 16)[l8] = packed;
        if (l8 == 0) *reinterpret_cast<float4*>(blk) = make_float4(d, d * (float)lo, d * (float)hi, 0.f);
    } else {
        const int tot = group_sum8_i(sum);
        if (!live) return;
        uint8_t* blk = out + b * kQ81xBytes;
        reinterpret_cast<uint32_t*>(blk + 8)[l8] = packed;
        if (l8 == 0) *reinterpret_cast<float2*>(blk) = make_float2(d, d * (float)tot);
    }
}

template <class ActT, bool SPLIT>
static int quantize_launch(mx_stream_t s, const ActT* x, void* out, uint64_t n) {
    MX_REQUIRE_PTR(x);
    MX_REQUIRE_PTR(out);
    MX_REQUIRE_SHAPE(n > 0 && n % 32 == 0);
    MX_REQUIRE_ALIGN(x, 8);
    MX_REQUIRE_ALIGN(out, SPLIT ? 16 : 8);
    const uint64_t nb = n / 32, threads = nb * 8;
    const uint64_t blocks = (threads + 255) / 256;
    MX_REQUIRE_SHAPE(blocks <= 0x7FFFFFFFull);
    hipLaunchKernelGGL((quantize_q8_1_kernel<ActT, SPLIT>), dim3((uint32_t)blocks), dim3(256), 0, as_stream(s), x, static_cast<uint8_t*>(out), nb);
    return launch_status();
}

// ---------------------------------------------------------------- element dequant
// One element of one block, written exactly as the reference evaluates it
// (include/ie/dequant_ref.hpp:32-96): the fp32 result is bit-identical for every
// association because each partial product is exact (11-bit d times <= 12-bit
// integer); only Q4_K's final subtraction rounds, once, fused or not.
enum { FMT_Q8_0 = 0, FMT_Q4_K = 1, FMT_Q6_K = 2, FMT_MXFP4 = 3, FMT_Q5_K = 4, FMT_Q4_0 = 5 };

template <int FMT>
struct BlockInfo;
template <>
struct BlockInfo<FMT_Q8_0> { static constexpr uint32_t elems = 32, bytes = kQ8_0Bytes; };
template <>
struct BlockInfo<FMT_Q4_K> { static constexpr uint32_t elems = 256, bytes = kQ4KBytes; };
template <>
struct BlockInfo<FMT_Q6_K> { static constexpr uint32_t elems = 256, bytes = kQ6KBytes; };
template <>
struct BlockInfo<FMT_MXFP4> { static constexpr uint32_t elems = 32, bytes = kMxfp4Bytes; };
template <>
struct BlockInfo<FMT_Q5_K> { static constexpr uint32_t elems = 256, bytes = 176; };
template <>
struct BlockInfo<FMT_Q4_0> { static constexpr uint32_t elems = 32, bytes = 18; };

__device__ __forceinline__ uint32_t ld16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

// Field-pointer forms of the Q4_K / Q6_K decoders: the same arithmetic whether the fields of a
// block sit together (AoS) or in per-field streams.
__device__ __forceinline__ void dequant8_q4k(const uint8_t* dm, const uint8_t* scales, const uint8_t* qs, uint32_t e0, float (&y)[8]) {
#pragma clang fp contract(off)
    const uint32_t g = e0 >> 6, hi = (e0 >> 5) & 1u, l = e0 & 31u;
    const uint32_t* sc32 = reinterpret_cast<const uint32_t*>(scales);
    uint32_t sc, mn;
    q4k_scale_pair(sc32[0], sc32[1], sc32[2], (int)g, sc, mn);
    const float d1 = h2f(ld16(dm)) * (float)((sc >> (8 * hi)) & 0xFFu);
    const float m1 = h2f(ld16(dm + 2)) * (float)((mn >> (8 * hi)) & 0xFFu);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t byte = qs[32 * g + l + i];
        y[i] = d1 * (float)(hi ? byte >> 4 : byte & 15u) - m1;
    }
}
__device__ __forceinline__ void dequant8_q6k(const uint8_t* ql, const uint8_t* qh, const uint8_t* scales, const uint8_t* dp, uint32_t e0, float (&y)[8]) {
#pragma clang fp contract(off)
    const uint32_t h = e0 >> 7, sub = (e0 >> 5) & 3u, l = e0 & 31u;
    const float d = h2f(ld16(dp));
    const float ds = d * (float)(int)(int8_t)scales[8 * h + 2 * sub + (l >> 4)];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t lb = ql[64 * h + 32 * (sub & 1u) + l + i];
        const uint32_t nib = (sub & 2u) ? lb >> 4 : lb & 15u;
        const uint32_t hi2 = (qh[32 * h + l + i] >> (2 * sub)) & 3u;
        y[i] = ds * (float)((int)(nib | (hi2 << 4)) - 32);
    }
}

// Dequantize the 8 consecutive elements [e0, e0+8) of block `b` (e0 % 8 == 0).
template <int FMT>
__device__ __forceinline__ void dequant8(const uint8_t* b, uint32_t e0, float (&y)[8]) {
    // No contraction: with fp16 output a fused multiply-add would round the exact
    // d1*q - m1 straight to fp16 (v_fma_mixlo_f16), skipping the fp32 rounding the
    // contract prescribes (fp32 value first, then one RNE conversion).
#pragma clang fp contract(off)
    if (FMT == FMT_Q8_0) {
        const float d = h2f(ld16(b));
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = d * (float)(int)(int8_t)b[2 + e0 + i];
    } else if (FMT == FMT_Q4_K) {
        dequant8_q4k(b, b + 4, b + 16, e0, y);
    } else if (FMT == FMT_Q5_K) {
        // {d, dmin, scales[12], qh[32], qs[128]} (include/ie/quant_blocks.hpp:79-85); Q4_K plus bit 2g+hi of qh[l]
        const uint32_t g = e0 >> 6, hi = (e0 >> 5) & 1u, l = e0 & 31u;
        const uint32_t* sc32 = reinterpret_cast<const uint32_t*>(b + 4);
        uint32_t sc, mn;
        q4k_scale_pair(sc32[0], sc32[1], sc32[2], (int)g, sc, mn);
        const float d1 = h2f(ld16(b)) * (float)((sc >> (8 * hi)) & 0xFFu);
        const float m1 = h2f(ld16(b + 2)) * (float)((mn >> (8 * hi)) & 0xFFu);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t byte = b[48 + 32 * g + l + i];
            const uint32_t q = (hi ? byte >> 4 : byte & 15u) + (((b[16 + l + i] >> (2 * g + hi)) & 1u) << 4);
            y[i] = d1 * (float)q - m1;
        }
    } else if (FMT == FMT_Q6_K) {
        dequant8_q6k(b, b + 128, b + 192, b + 208, e0, y);
    } else if (FMT == FMT_Q4_0) {
        // {fp16 d; u8 qs[16]}: element j in the low, j + 16 in the high nibble of qs[j]; w = d * (q - 8)
        // (include/ie/quant_blocks.hpp:32-43, src/ops/gemv_q4_0.cpp:3-8)
        const float d = h2f(ld16(b));
        const uint32_t hi = e0 >> 4, j0 = e0 & 15u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t byte = b[2 + j0 + i];
            y[i] = d * (float)((int)(hi ? byte >> 4 : byte & 15u) - 8);
        }
    } else {
        const float d = e8m0_half(b[0]);
        const uint32_t hi = e0 >> 4, j0 = e0 & 15u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t byte = b[1 + j0 + i];
            const uint32_t c = hi ? byte >> 4 : byte & 15u;
            const int mag = (int)((0x0C08060403020100ull >> (8 * (c & 7u))) & 0xFFu);
            y[i] = (float)((c & 8u) ? -mag : mag) * d;
        }
    }
}

__device__ __forceinline__ void store_exact(half_t* p, float v) { *p = f32_to_f16_rne(v); }
__device__ __forceinline__ void store_exact(float* p, float v) { *p = v; }

template <int FMT, class OutT>
__global__ __launch_bounds__(256) void dequant_flat_kernel(const uint8_t* packed, OutT* out, uint64_t n_groups) {
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n_groups) return;
    constexpr uint32_t gpb = BlockInfo<FMT>::elems / 8;
    const uint64_t blk = gid / gpb;
    const uint32_t e0 = (uint32_t)(gid % gpb) * 8u;
    float y[8];
    dequant8<FMT>(packed + blk * BlockInfo<FMT>::bytes, e0, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) store_exact(out + gid * 8 + i, y[i]);
}

// Bt[k*N + n] = half(W[n][k]).  Thread = (k-group of 8, n); n runs fastest
// across a wave so the eight row-strided stores are each coalesced.
template <int FMT>
__global__ __launch_bounds__(256) void dequant_bt_kernel(const uint8_t* W, half_t* Bt, uint32_t K, uint32_t N) {
    const uint32_t n = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t kg = blockIdx.y;
    if (n >= N) return;
    constexpr uint32_t gpb = BlockInfo<FMT>::elems / 8;
    const size_t row_bytes = (size_t)(K / BlockInfo<FMT>::elems) * BlockInfo<FMT>::bytes;
    float y[8];
    dequant8<FMT>(W + (size_t)n * row_bytes + (size_t)(kg / gpb) * BlockInfo<FMT>::bytes, (kg % gpb) * 8u, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) Bt[(size_t)(kg * 8u + i) * N + n] = f32_to_f16_rne(y[i]);
}

template <int FMT, class OutT>
static int dequant_flat(mx_stream_t s, const void* packed, OutT* out, uint64_t n) {
    MX_REQUIRE_PTR(packed);
    MX_REQUIRE_PTR(out);
    MX_REQUIRE_SHAPE(n > 0 && n % BlockInfo<FMT>::elems == 0);
    MX_REQUIRE_ALIGN(packed, (FMT == FMT_Q4_K || FMT == FMT_Q5_K) ? 4 : (FMT == FMT_MXFP4 ? 1 : 2));
    const uint64_t groups = n / 8, blocks = (groups + 255) / 256;
    MX_REQUIRE_SHAPE(blocks <= 0x7FFFFFFFull);
    hipLaunchKernelGGL((dequant_flat_kernel<FMT, OutT>), dim3((uint32_t)blocks), dim3(256), 0, as_stream(s), static_cast<const uint8_t*>(packed), out, groups);
    return launch_status();
}

template <int FMT>
static int dequant_bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_PTR(Bt);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && K % BlockInfo<FMT>::elems == 0 && K / 8 <= 65535);
    MX_REQUIRE_ALIGN(W, (FMT == FMT_Q4_K || FMT == FMT_Q5_K) ? 4 : (FMT == FMT_MXFP4 ? 1 : 2));
    hipLaunchKernelGGL((dequant_bt_kernel<FMT>), dim3((N + 255) / 256, K / 8), dim3(256), 0, as_stream(s), static_cast<const uint8_t*>(W), reinterpret_cast<half_t*>(Bt), K, N);
    return launch_status();
}

// ---------------------------------------------------------------- repacked layouts -> Bt
// Views give the 8 elements [8*kg, 8*kg+8) of row n.  Values are bit-identical to the AoS
// decoders above: the repacks move bits, they never change a value's representation.
struct Q4KStrView {     // qs[128] x nb | scales[12] x nb | {d,dmin}[4] x nb   (include/ie/quant_soa.hpp:33-41)
    const uint8_t* base; uint64_t nb; uint32_t bpr;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
        const uint64_t ib = (uint64_t)n * bpr + (kg >> 5);
        dequant8_q4k(base + nb * 140u + ib * 4u, base + nb * 128u + ib * 12u, base + ib * 128u, (kg & 31u) * 8u, y);
    }
};
struct Q6KStrView {     // ql[128] x nb | qh[64] x nb | scales[16] x nb | d[2] x nb   (include/ie/quant_soa.hpp:43-51)
    const uint8_t* base; uint64_t nb; uint32_t bpr;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
        const uint64_t ib = (uint64_t)n * bpr + (kg >> 5);
        dequant8_q6k(base + ib * 128u, base + nb * 128u + ib * 64u, base + nb * 192u + ib * 16u, base + nb * 208u + ib * 2u, (kg & 31u) * 8u, y);
    }
};
struct Q4KNatView {     // natural-order nibble plane + unpacked per-32 scale/min + per-256 d/dmin (src/ops/gemv_q4_soa.cpp:18-28)
    const uint8_t* q; const int8_t* sc; const int8_t* mn; const uint16_t* d; const uint16_t* dmin; uint32_t K;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
#pragma clang fp contract(off)
        const uint32_t k = kg * 8u;
        const uint32_t w = *reinterpret_cast<const uint32_t*>(q + (size_t)n * (K >> 1) + (k >> 1));
        const size_t sb = (size_t)n * (K >> 5) + (k >> 5), bb = (size_t)n * (K >> 8) + (k >> 8);
        const float d1 = h2f(d[bb]) * (float)(int)sc[sb];
        const float m1 = h2f(dmin[bb]) * (float)(int)mn[sb];
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = d1 * (float)((w >> (4 * i)) & 15u) - m1;
    }
};
struct Q6KNatView {     // natural-order 4-bit and 2-bit planes + per-16 int8 scale + per-256 d (src/ops/gemv_q6_soa.cpp:62-126)
    const uint8_t* lo; const uint8_t* hi; const int8_t* sc; const uint16_t* d; uint32_t K;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
#pragma clang fp contract(off)
        const uint32_t k = kg * 8u;
        const uint32_t wl = *reinterpret_cast<const uint32_t*>(lo + (size_t)n * (K >> 1) + (k >> 1));
        const uint32_t wh = *reinterpret_cast<const uint16_t*>(hi + (size_t)n * (K >> 2) + (k >> 2));
        const float ds = h2f(d[(size_t)n * (K >> 8) + (k >> 8)]) * (float)(int)sc[(size_t)n * (K >> 4) + (k >> 4)];
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = ds * (float)((int)(((wl >> (4 * i)) & 15u) | (((wh >> (2 * i)) & 3u) << 4)) - 32);
    }
};
struct Mxfp4SoaView {   // qs_plane[n*(K/2) + 16b + j], e_plane[n*(K/32) + b]   (src/ops/gemv_mxfp4.cpp:13-16,316-341)
    const uint8_t* qs; const uint8_t* e; uint32_t K;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
        const uint32_t b = kg >> 2, e0 = (kg & 3u) * 8u;
        const float d = e8m0_half(e[(size_t)n * (K >> 5) + b]);
        const uint8_t* p = qs + (size_t)n * (K >> 1) + 16u * b + (e0 & 15u);
        const uint32_t hi = e0 >> 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t c = hi ? p[i] >> 4 : p[i] & 15u;
            const int mag = (int)((0x0C08060403020100ull >> (8 * (c & 7u))) & 0xFFu);
            y[i] = (float)((c & 8u) ? -mag : mag) * d;
        }
    }
};

struct Q40SoaView {     // q4_qs[n*(K/2) + 16b + j], q4_d[n*(K/32) + b]   (src/ops/gemv_q4_0.cpp:179-192,455-477)
    const uint8_t* qs; const uint16_t* d; uint32_t K;
    __device__ __forceinline__ void get(uint32_t n, uint32_t kg, float (&y)[8]) const {
        const uint32_t b = kg >> 2, e0 = (kg & 3u) * 8u;
        const float dv = h2f(d[(size_t)n * (K >> 5) + b]);
        const uint8_t* p = qs + (size_t)n * (K >> 1) + 16u * b + (e0 & 15u);
        const uint32_t hi = e0 >> 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = dv * (float)((int)(hi ? p[i] >> 4 : p[i] & 15u) - 8);
    }
};

template <class V>
__global__ __launch_bounds__(256) void dequant_bt_view_kernel(V v, half_t* Bt, uint32_t N) {
    const uint32_t n = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t kg = blockIdx.y;
    if (n >= N) return;
    float y[8];
    v.get(n, kg, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) Bt[(size_t)(kg * 8u + i) * N + n] = f32_to_f16_rne(y[i]);
}

template <class V>
static int dequant_bt_view(mx_stream_t s, const V& v, uint16_t* Bt, uint32_t K, uint32_t N, uint32_t k_align) {
    MX_REQUIRE_PTR(Bt);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && K % k_align == 0 && K / 8 <= 65535);
    hipLaunchKernelGGL((dequant_bt_view_kernel<V>), dim3((N + 255) / 256, K / 8), dim3(256), 0, as_stream(s), v, reinterpret_cast<half_t*>(Bt), N);
    return launch_status();
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_quantize_q8_1(mx_stream_t s, const uint16_t* x, void* out, uint64_t n) {
    return quantize_launch<half_t, false>(s, reinterpret_cast<const half_t*>(x), out, n);
}
int mx_quantize_q8_1_f32(mx_stream_t s, const float* x, void* out, uint64_t n) {
    MX_REQUIRE_ALIGN(x, 16);
    return quantize_launch<float, false>(s, x, out, n);
}
int mx_quantize_q8_1s(mx_stream_t s, const uint16_t* x, void* out, uint64_t n) {
    return quantize_launch<half_t, true>(s, reinterpret_cast<const half_t*>(x), out, n);
}
int mx_quantize_q8_1s_f32(mx_stream_t s, const float* x, void* out, uint64_t n) {
    MX_REQUIRE_ALIGN(x, 16);
    return quantize_launch<float, true>(s, x, out, n);
}

#define MX_DEQ(name, FMT)                                                                                   \
    int mx_dequant_##name(mx_stream_t s, const void* p, uint16_t* out, uint64_t n) {                        \
        return dequant_flat<FMT, half_t>(s, p, reinterpret_cast<half_t*>(out), n);                          \
    }                                                                                                       \
    int mx_dequant_##name##_f32(mx_stream_t s, const void* p, float* out, uint64_t n) {                     \
        return dequant_flat<FMT, float>(s, p, out, n);                                                      \
    }                                                                                                       \
    int mx_dequant_##name##_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N) {     \
        return dequant_bt<FMT>(s, W, Bt, K, N);                                                             \
    }
MX_DEQ(q8_0, FMT_Q8_0)
MX_DEQ(q4_K, FMT_Q4_K)
MX_DEQ(q5_K, FMT_Q5_K)
MX_DEQ(q6_K, FMT_Q6_K)
MX_DEQ(mxfp4, FMT_MXFP4)
MX_DEQ(q4_0, FMT_Q4_0)
#undef MX_DEQ

// Transposed dequant of the repacked layouts.
int mx_dequant_q4_moe_soa_to_Bt(mx_stream_t s, const void* soa_region, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(soa_region);
    MX_REQUIRE_ALIGN(soa_region, 4);
    return dequant_bt_view(s, Q4KStrView{static_cast<const uint8_t*>(soa_region), (uint64_t)N * (K / 256), K / 256}, Bt, K, N, 256);
}
int mx_dequant_q6_K_soa_to_Bt(mx_stream_t s, const void* soa_region, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(soa_region);
    MX_REQUIRE_ALIGN(soa_region, 2);
    return dequant_bt_view(s, Q6KStrView{static_cast<const uint8_t*>(soa_region), (uint64_t)N * (K / 256), K / 256}, Bt, K, N, 256);
}
int mx_dequant_q4_soa_to_Bt(mx_stream_t s, const uint8_t* q4_q, const int8_t* q4_sc, const int8_t* q4_mn, const uint16_t* q4_d,
                            const uint16_t* q4_dmin, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(q4_q); MX_REQUIRE_PTR(q4_sc); MX_REQUIRE_PTR(q4_mn); MX_REQUIRE_PTR(q4_d); MX_REQUIRE_PTR(q4_dmin);
    MX_REQUIRE_ALIGN(q4_q, 4);
    return dequant_bt_view(s, Q4KNatView{q4_q, q4_sc, q4_mn, q4_d, q4_dmin, K}, Bt, K, N, 256);
}
int mx_dequant_q6_soa_to_Bt(mx_stream_t s, const uint8_t* q6_lo, const uint8_t* q6_hi, const int8_t* q6_sc, const uint16_t* q6_d, uint16_t* Bt,
                            uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(q6_lo); MX_REQUIRE_PTR(q6_hi); MX_REQUIRE_PTR(q6_sc); MX_REQUIRE_PTR(q6_d);
    MX_REQUIRE_ALIGN(q6_lo, 4); MX_REQUIRE_ALIGN(q6_hi, 2);
    return dequant_bt_view(s, Q6KNatView{q6_lo, q6_hi, q6_sc, q6_d, K}, Bt, K, N, 256);
}
int mx_dequant_q4_0_soa_to_Bt(mx_stream_t s, const uint8_t* soa_qs, const uint16_t* soa_d, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(soa_qs); MX_REQUIRE_PTR(soa_d);
    return dequant_bt_view(s, Q40SoaView{soa_qs, soa_d, K}, Bt, K, N, 32);
}
int mx_dequant_mxfp4_soa_to_Bt(mx_stream_t s, const uint8_t* qs_plane, const uint8_t* e_plane, uint16_t* Bt, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(qs_plane); MX_REQUIRE_PTR(e_plane);
    return dequant_bt_view(s, Mxfp4SoaView{qs_plane, e_plane, K}, Bt, K, N, 32);
}

}  // extern "C"
