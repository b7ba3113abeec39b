// gemm_f16_tiled.hip — the plain fp16 x fp16 -> fp32 GEMM as a hand-tiled kernel: the counterpart of the reference's
// in-house joint_matrix kernel (gemm_fp16, include/ie/ops.hpp:275-286, src/ops/gemm_fp16.cpp:46-178):
//     C[M, N] (fp32) = A[M, K] . B[K, N],   A and B fp16 row-major, fp32 accumulate.
// B is K-major ([K][N]), so unlike the quantized weights of gemm.hip it cannot feed the matrix cores from the lane's own
// global loads (an operand lane needs 8 consecutive k of one column): both tiles go through LDS, B transposed on the way.
//
// Workgroup = 4 waves = a 128 x 128 tile of C, K walked in steps of 32; wave (wm, wn) owns 64 x 64 = 2 x 2 tiles of
// v_mfma_f32_32x32x16_f16.  LDS: As[128][40] and Bs[128][40] halfs (row pitch 80 B: the 16 lanes of a ds_read_b128 pass
// fall on 16 different bank groups).  Ragged M, N and K are handled by guarded loads (zeros) and guarded stores, so C can
// be sized exactly (the reference stores whole tiles and asks for a padded C).
#include "mxq_formats.h"
#include "mxq_host.h"

namespace mxq {

typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kFBM = 128, kFBN = 128, kFBK = 32, kFPitch = kFBK + 8;

// 8 halfs at p[0..8) of a row holding `left` more elements; vector load when the address allows it
__device__ __forceinline__ uint4 load8h(const half_t* p, uint32_t left, bool row_ok) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (!row_ok || left == 0) return v;
    if (left >= 8 && (reinterpret_cast<uintptr_t>(p) & 15u) == 0) return *reinterpret_cast<const uint4*>(p);
    uint16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (uint32_t)i < left ? reinterpret_cast<const uint16_t*>(p)[i] : (uint16_t)0;
    v.x = h[0] | ((uint32_t)h[1] << 16); v.y = h[2] | ((uint32_t)h[3] << 16);
    v.z = h[4] | ((uint32_t)h[5] << 16); v.w = h[6] | ((uint32_t)h[7] << 16);
    return v;
}

__global__ __launch_bounds__(256) void gemm_f16_tiled_kernel(const half_t* __restrict__ A, const half_t* __restrict__ B, float* __restrict__ C, uint32_t M,
                                                              uint32_t N, uint32_t K) {
    __shared__ __align__(16) uint16_t As[kFBM * kFPitch];
    __shared__ __align__(16) uint16_t Bs[kFBN * kFPitch];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, j = lane & 31u, h = lane >> 5;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t m0 = blockIdx.y * kFBM, n0 = blockIdx.x * kFBN;
    f32x16_t acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    for (uint32_t k0 = 0; k0 < K; k0 += kFBK) {
        // ---- this step's tiles: requested before the barrier, written after it
        uint4 av[2], bv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t ia = tid + 256u * u, ra = ia >> 2, ca = (ia & 3u) * 8u;          // A: 128 rows x 4 chunks of 8 k
            const uint32_t ka = k0 + ca;
            av[u] = load8h(A + (size_t)(m0 + ra) * K + ka, ka < K ? K - ka : 0u, m0 + ra < M);
            const uint32_t ib = tid + 256u * u, kb = ib >> 4, cb = (ib & 15u) * 8u;         // B: 32 k rows x 16 chunks of 8 n
            const uint32_t nb = n0 + cb;
            bv[u] = load8h(B + (size_t)(k0 + kb) * N + nb, nb < N ? N - nb : 0u, k0 + kb < K);
        }
        __syncthreads();   // the previous step's fragments have been read
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t ia = tid + 256u * u, ra = ia >> 2, ca = (ia & 3u) * 8u;
            *reinterpret_cast<uint4*>(&As[ra * kFPitch + ca]) = av[u];
            const uint32_t ib = tid + 256u * u, kb = ib >> 4, cb = (ib & 15u) * 8u;
            const uint32_t w[4] = {bv[u].x, bv[u].y, bv[u].z, bv[u].w};
#pragma unroll
            for (int i = 0; i < 8; ++i) Bs[(cb + i) * kFPitch + kb] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));   // transposed: Bs[n][k]
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < kFBK / 16; ++ks) {
            f16x8_t af[2], bf[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
                af[mi] = *reinterpret_cast<const f16x8_t*>(&As[(wm * 64 + mi * 32 + j) * kFPitch + ks * 16 + 8 * h]);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                bf[ni] = *reinterpret_cast<const f16x8_t*>(&Bs[(wn * 64 + ni * 32 + j) * kFPitch + ks * 16 + 8 * h]);
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mi], bf[ni], acc[mi][ni], 0, 0, 0);
        }
    }
    // lane (j, h) holds column j and rows 8 (v / 4) + 4 h + v % 4 of each 32 x 32 tile
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const uint32_t col = n0 + wn * 64 + ni * 32 + j;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + wm * 64 + mi * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                if (row < M && col < N) C[(size_t)row * N + col] = acc[mi][ni][v];
            }
        }
}

}  // namespace mxq

extern "C" int mx_gemm_fp16(mx_stream_t s, const uint16_t* A, const uint16_t* B, float* C, uint32_t M, uint32_t N, uint32_t K) {
    using namespace mxq;
    MX_REQUIRE_PTR(A); MX_REQUIRE_PTR(B); MX_REQUIRE_PTR(C);
    MX_REQUIRE_SHAPE(M > 0 && N > 0 && K > 0);
    MX_REQUIRE_ALIGN(A, 2); MX_REQUIRE_ALIGN(B, 2); MX_REQUIRE_ALIGN(C, 4);
    const uint32_t gy = (M + kFBM - 1) / kFBM, gx = (N + kFBN - 1) / kFBN;
    if (gy > 65535u) return MX_ERR_SHAPE;
    hipLaunchKernelGGL(gemm_f16_tiled_kernel, dim3(gx, gy), dim3(256), 0, as_stream(s), reinterpret_cast<const half_t*>(A),
                       reinterpret_cast<const half_t*>(B), C, M, N, K);
    return launch_status();
}
