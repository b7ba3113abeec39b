// gemv_q6_planes.hip — one-token int-dot GEMV over the natural-order Q6_K planes of repack_q6_K_to_soa
// (src/ops/gemv_q6_soa.cpp:62-126: lo[n*(K/2) + k/2] nibble (k&1), hi[n*(K/4) + k/4] 2-bit field (k&3), per-16 int8
// scale, per-256 fp16 d), arithmetic of gemv_q6_soa_q8 (src/ops/gemv_q6_soa.cpp:208-251):
//     acc += (d * sc16) * d8 * (float)(idot - 32 * isum),  idot = sum(q6u * q8), q6u in 0..63.
//
// Two things make the plane form stream where the generic unit walk does not:
//   * interleaved units.  Eight lanes share a 512-element span of the row; lane m takes elements [32 m, 32 m + 32) of
//     both 256-element halves of it.  Every load instruction of the wave then reads whole cache lines (lo: 128
//     contiguous bytes per eight lanes, non-temporal; hi: 64) instead of one 16-byte piece per lane, which the memory
//     pipeline serves at a third of the rate;
//   * no code assembly.  The 6-bit code is lo + 16 hi, so idot = dot(lo, x) + 16 dot(hi, x).  The masked nibble words
//     hold elements (0 2 4 6 | 1 3 5 7) of eight and the shifted 2-bit words elements (k, k + 4, k + 8, k + 12) of
//     sixteen; instead of permuting every weight word into element order, the activation row is staged twice, once in
//     each of those two orders (a few byte permutes per 16 activations, once per workgroup), and the masked words go into
//     v_dot4_i32_i8 as they are.
// A wave owns whole rows (64 lanes x 64 elements per round, rows of any K % 512 == 0 take ceil(K / 4096) rounds); two
// register sets take turns so that the loads of one (row, round) item are in flight while the other is summed.
#include <atomic>

#include "mxq_gemv_core.h"
#include "mxq_host.h"

namespace mxq {

constexpr uint32_t kQ6pMaxLds = 40u * 1024u;   // 2.5 bytes of LDS per activation: K <= 16384

struct Q6pSeg {
    const uint8_t* lo;
    const uint8_t* hi;
    const uint8_t* sc;
    const uint8_t* d;
    half_t* y;
};

// chunk c (16 activations) of the staged row lives at c ^ ((c >> 5) & 1): the lanes of two neighbouring spans, which one
// ds_read_b128 pass serves together, then read the even and the odd 16-byte slots of a 256-byte window
__device__ __forceinline__ uint32_t q6p_slot(uint32_t c) { return c ^ ((c >> 5) & 1u); }

struct Q6pRaw {
    uint4 l0, l1;
    uint2 h0, h1;
    uint32_t s01, s23, d2;
};

struct Q6pTile {
    const uint4* x_lo;   // [K/16] chunks, elements (0 2 4 6 | 1 3 5 7 | 8 10 12 14 | 9 11 13 15)
    const uint4* x_hi;   // [K/16] chunks, elements (0 4 8 12 | 1 5 9 13 | 2 6 10 14 | 3 7 11 15)
    const uint2* x_hd;   // [K/16] {d8 bits, sum of the 16 q8}
};

// Stage the q8 row (block_q8_1x: {float d, float s, int8 qs[32]}, 40 bytes per 32 elements), one 16-chunk per thread and pass.
__device__ __forceinline__ Q6pTile q6p_stage(uint8_t* lds, const uint8_t* xq8, uint32_t K) {
    const uint32_t n_chunks = K / 16u;
    uint4* x_lo = reinterpret_cast<uint4*>(lds);
    uint4* x_hi = x_lo + n_chunks;
    uint2* x_hd = reinterpret_cast<uint2*>(x_hi + n_chunks);
    for (uint32_t c = threadIdx.x; c < n_chunks; c += kGemvThreads) {
        const uint8_t* blk = xq8 + (size_t)(c >> 1) * kQ81xBytes;
        const uint2* q = reinterpret_cast<const uint2*>(blk + 8 + (c & 1u) * 16u);
        const uint2 qa = q[0], qb = q[1];
        const uint32_t a = qa.x, b = qa.y, cc = qb.x, dd = qb.y;   // elements 0-3, 4-7, 8-11, 12-15
        const uint32_t d8 = *reinterpret_cast<const uint32_t*>(blk);
        int sum = dot4(0x01010101u, a, 0);
        sum = dot4(0x01010101u, b, sum);
        sum = dot4(0x01010101u, cc, sum);
        sum = dot4(0x01010101u, dd, sum);
        const uint32_t at = q6p_slot(c);
        x_lo[at] = make_uint4(__builtin_amdgcn_perm(b, a, 0x06040200u), __builtin_amdgcn_perm(b, a, 0x07050301u),
                              __builtin_amdgcn_perm(dd, cc, 0x06040200u), __builtin_amdgcn_perm(dd, cc, 0x07050301u));
        const uint32_t p0 = __builtin_amdgcn_perm(b, a, 0x05010400u), p1 = __builtin_amdgcn_perm(b, a, 0x07030602u);     // (a0 b0 a1 b1), (a2 b2 a3 b3)
        const uint32_t p2 = __builtin_amdgcn_perm(dd, cc, 0x05010400u), p3 = __builtin_amdgcn_perm(dd, cc, 0x07030602u);
        x_hi[at] = make_uint4(__builtin_amdgcn_perm(p2, p0, 0x05040100u), __builtin_amdgcn_perm(p2, p0, 0x07060302u),
                              __builtin_amdgcn_perm(p3, p1, 0x05040100u), __builtin_amdgcn_perm(p3, p1, 0x07060302u));
        x_hd[at] = make_uint2(d8, (uint32_t)sum);
    }
    return Q6pTile{x_lo, x_hi, x_hd};
}

// Unit u of row `row`: lane m = u & 7 of span u >> 3.
__device__ __forceinline__ void q6p_request(Q6pRaw& r, const Q6pSeg& seg, uint32_t row, uint32_t u, uint32_t K) {
    const uint32_t U = u >> 3, m = u & 7u;
    const uint8_t* lo = seg.lo + (size_t)row * (K >> 1) + U * 256u + m * 16u;
    const uint8_t* hi = seg.hi + (size_t)row * (K >> 2) + U * 128u + m * 8u;
    const uint8_t* sc = seg.sc + (size_t)row * (K >> 4) + U * 32u + m * 2u;
    r.l0 = load_u4_stream(lo);
    r.l1 = load_u4_stream(lo + 128);
    r.h0 = *reinterpret_cast<const uint2*>(hi);
    r.h1 = *reinterpret_cast<const uint2*>(hi + 64);
    r.s01 = *reinterpret_cast<const uint16_t*>(sc);
    r.s23 = *reinterpret_cast<const uint16_t*>(sc + 16);
    r.d2 = *reinterpret_cast<const uint32_t*>(seg.d + (size_t)row * ((K >> 8) * 2u) + U * 4u);
}

__device__ __forceinline__ float q6p_consume(const Q6pRaw& r, const Q6pTile& x, uint32_t u) {
    const uint32_t c0 = (u >> 3) * 32u + 2u * (u & 7u);   // first chunk of the lane's 32 elements in the span's first half
    const uint32_t lw[8] = {r.l0.x, r.l0.y, r.l0.z, r.l0.w, r.l1.x, r.l1.y, r.l1.z, r.l1.w};
    const uint32_t hw[4] = {r.h0.x, r.h0.y, r.h1.x, r.h1.y};
    const uint32_t sc[4] = {r.s01 & 0xFFu, r.s01 >> 8, r.s23 & 0xFFu, r.s23 >> 8};
    const float dsb[2] = {h2f(r.d2 & 0xFFFFu), h2f(r.d2 >> 16)};
    float acc = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t at = q6p_slot(c0 + (uint32_t)((g & 1) + (g >> 1) * 16));
        const uint4 xl = x.x_lo[at], xh = x.x_hi[at];
        const uint2 hd = x.x_hd[at];
        const uint32_t w0 = lw[2 * g], w1 = lw[2 * g + 1], h = hw[g];
        int ih = dot4(h & 0x03030303u, xh.x, 0);
        ih = dot4((h >> 2) & 0x03030303u, xh.y, ih);
        ih = dot4((h >> 4) & 0x03030303u, xh.z, ih);
        ih = dot4((h >> 6) & 0x03030303u, xh.w, ih);
        int il = dot4(w0 & 0x0F0F0F0Fu, xl.x, ih * 16 - 32 * (int)hd.y);
        il = dot4((w0 >> 4) & 0x0F0F0F0Fu, xl.y, il);
        il = dot4(w1 & 0x0F0F0F0Fu, xl.z, il);
        il = dot4((w1 >> 4) & 0x0F0F0F0Fu, xl.w, il);
        acc += (dsb[g >> 1] * (float)(int)(int8_t)sc[g]) * (u2f(hd.x) * (float)il);
    }
    return acc;
}

__global__ __launch_bounds__(kGemvThreads, 4) void gemv_q6_planes_kernel(Q6pSeg seg0, Q6pSeg seg1, const uint8_t* xq8, uint32_t K, uint32_t N) {
    extern __shared__ __align__(16) uint8_t lds[];
    const Q6pSeg& seg = blockIdx.y ? seg1 : seg0;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const Q6pTile xt = q6p_stage(lds, xq8, K);

    // ---- rows of this wave, rounds of 64 units per row
    const uint32_t n_units = K / 64u, rounds = (n_units + 63u) / 64u;
    const uint32_t wave_id = blockIdx.x * kGemvWaves + (tid >> 6), n_waves = gridDim.x * kGemvWaves;
    auto request = [&](Q6pRaw& r, uint32_t row, uint32_t round) {
        const uint32_t u = round * 64u + lane;
        if (row < N && u < n_units) q6p_request(r, seg, row, u, K);
    };
    auto consume = [&](const Q6pRaw& r, uint32_t row, uint32_t round, float& acc) {
        const uint32_t u = round * 64u + lane;
        if (row < N && u < n_units) acc += q6p_consume(r, xt, u);
    };
    auto finish = [&](uint32_t row, float acc) {
        const float v = group_sum<64>(acc);
        if (lane == 63u && row < N) seg.y[row] = (half_t)v;
    };

    // item = (row, round).  Two register sets take turns (the loop is unrolled over them, so no set is ever copied: a
    // copy would wait for its load): one item is in flight while the other is summed.  Four sets, three items in flight,
    // measured slower (4096 -> 14336: 12.0 -> 13.8 us), and so did a workgroup-wide walk of long rows (thread t takes unit t,
    // one round per row: 14336 -> 4096 13.6 us either way).  The first item is requested before the barrier behind the staging.
    struct Item {
        uint32_t row, round;
    };
    auto next = [&](Item it) {
        it.round += 1u;
        if (it.round == rounds) {
            it.round = 0;
            it.row += n_waves;
        }
        return it;
    };
    Q6pRaw r0, r1;
    Item head{wave_id, 0u}, cur = head;   // next item to request, next item to sum
    request(r0, head.row, head.round);
    head = next(head);
    __syncthreads();
    float acc = 0.f;
#define Q6P_STEP(rq, rc)                                       \
    request(rq, head.row, head.round);                          \
    head = next(head);                                          \
    __builtin_amdgcn_sched_barrier(0);                          \
    if (cur.row < N) {                                          \
        consume(rc, cur.row, cur.round, acc);                   \
        if (cur.round + 1u == rounds) {                         \
            finish(cur.row, acc);                               \
            acc = 0.f;                                          \
        }                                                       \
    }                                                           \
    cur = next(cur);
    while (cur.row < N) {
        Q6P_STEP(r1, r0)
        Q6P_STEP(r0, r1)
    }
#undef Q6P_STEP
}

static int q6p_cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    }
    return n;
}

// One (nseg = 1) or two (gate and up: nseg = 2) matrices against one q8 row.  Returns MX_ERR_UNSUPPORTED for shapes this
// kernel does not take (the caller then runs the generic unit walk).
int launch_gemv_q6_planes(hipStream_t st, int nseg, const void* x_q8, const uint8_t* const* lo, const uint8_t* const* hi, const int8_t* const* sc,
                          const uint16_t* const* d, uint16_t* const* y, uint32_t K, uint32_t N) {
    const uint32_t lds = K * 2u + K / 2u;
    if (K % 512u != 0 || lds > kQ6pMaxLds || (uint64_t)N * (K >> 1) >= (1ull << 32)) return MX_ERR_UNSUPPORTED;
    Q6pSeg s[2];
    for (int i = 0; i < nseg; ++i) {
        if ((reinterpret_cast<uintptr_t>(d[i]) & 3u) || (reinterpret_cast<uintptr_t>(sc[i]) & 1u)) return MX_ERR_UNSUPPORTED;
        s[i] = Q6pSeg{lo[i], hi[i], reinterpret_cast<const uint8_t*>(sc[i]), reinterpret_cast<const uint8_t*>(d[i]), reinterpret_cast<half_t*>(y[i])};
    }
    if (nseg == 1) s[1] = s[0];
    // persistent waves: as many workgroups as are resident (four per CU when the activation tile allows), at most one row per wave and pass
    static std::atomic<int> fit[11];   // by LDS size in 4 KB steps, asked once each
    const uint32_t cls = (lds + 4095u) / 4096u;
    int per_cu = fit[cls].load(std::memory_order_relaxed);
    if (!per_cu) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(&gemv_q6_planes_kernel), kGemvThreads, cls * 4096u) != hipSuccess || per_cu < 1) per_cu = 1;
        if (per_cu > 4) per_cu = 4;
        fit[cls].store(per_cu, std::memory_order_relaxed);
    }
    uint32_t grid = (uint32_t)q6p_cu_count() * (uint32_t)per_cu / (uint32_t)nseg;
    const uint32_t need = (N + kGemvWaves - 1) / kGemvWaves;
    if (grid > need) grid = need;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(gemv_q6_planes_kernel, dim3(grid, nseg), dim3(kGemvThreads), lds, st, s[0], s[1], static_cast<const uint8_t*>(x_q8), K, N);
    return launch_status();
}

}  // namespace mxq
