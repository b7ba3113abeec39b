// gemv.hip — dense decode GEMV entry points (T = 1 and batched T <= 16) for
// Q4_K / Q6_K / Q8_0 / MXFP4 weights: int-dot on q8 activations and the
// float-activation variants.  Kernel structure: mxq_gemv_core.h.
#include "mxq_gemv_core.h"
#include "mxq_mmq.h"
#include <stdlib.h>

#include <type_traits>

#include "mxq_host.h"

namespace mxq {

// One launch can carry two independent (weights, output, bias) segments that
// share the activation (the fused gate/up form); blockIdx.y picks the segment.
template <class F, class OutT>
struct GemvSeg {
    typename F::W w;
    OutT* y;
    const float* bias;
};

// Formats whose T = 1 kernels hold a second set of units in registers (requested ahead of the row group being
// summed, or ahead of the activation staging): the ones where that was measured to pay and that stay within the
// 128 VGPRs the four-workgroups-per-CU launch wants.  Q6_K gains nothing from it with four workgroups per CU (12.1 ->
// 12.2 us on 4096 -> 14336, 95.8 -> 98.5 us on the 151936-row output projection) and a tenth with two (launch_q8_tg).
template <class F>
constexpr bool kPrefetchAcrossRows = std::is_same<F, FmtQ8Soa>::value || std::is_same<F, FmtQ8SoaW>::value || std::is_same<F, FmtQ4K>::value || std::is_same<F, FmtQ8Aos>::value || std::is_same<F, FmtQ6K>::value;

// Persistent workgroups: each stages the activation tile(s) and then streams
// its share of row groups.  With a single K-tile (every decode shape at T <= 2)
// the activation is staged once per workgroup.  The single-token instances are compiled
// for the four workgroups per CU they are launched with (128 registers): left alone the
// compiler takes a few more for some formats and a workgroup per CU is lost (Q6_K planes,
// 4096 -> 14336: 15.5 -> 13.5 us with three registers spilled; no other format changes).
template <class F, int T, int R, int G, int U, class OutT>
__global__ __launch_bounds__(kGemvThreads, (T == 1 ? 4 : 1)) void gemv_q8_kernel(GemvSeg<F, OutT> seg0, GemvSeg<F, OutT> seg1, const uint8_t* xq8,
                                                                uint32_t K, uint32_t N, uint32_t KT, uint32_t T_real, uint32_t q8_split) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS * R;
    const GemvSeg<F, OutT>& seg = blockIdx.y ? seg1 : seg0;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    const size_t q8_row_bytes = (size_t)(K / 32) * (q8_split ? kQ81sBytes : kQ81xBytes);
    auto xrow = [&](uint32_t t) { return xq8 + (size_t)(t < T_real ? t : T_real - 1) * q8_row_bytes; };
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_tiles = (K + KT - 1) / KT;
    ActTile act;
    bool staged = false;
    if (T <= 2 && kPrefetchAcrossRows<F> && K == 64u * G && n_tiles == 1) {
        // One unit per lane and row (K = 4096 with 64 lanes per row, ...): a row is a single round of loads, so the
        // loads of the next row group are issued before the dot products and the lane-group sum of this one;
        // otherwise every wave would sit with nothing in flight from its last load's arrival to its store.
        // Measured on 4096 -> 14336: Q8_0 planes 13.2 -> 12.4 us (T = 2: 14.2 -> 13.0), Q4_K 8.6 -> 8.4 us (T = 2:
        // 10.2 -> 9.2).  Batches of four and more lose (the second set of units costs occupancy next to R x T sums).
        // The first row group's weights are requested before the activation row is staged: they do not depend on it.
        // Two register sets take turns (never copied: a copy would wait for the load), so the loads of one row group are
        // in flight while the other one is summed; a slot past the last row group reads one broadcast line.  The first
        // row group's weights are requested between the activation loads and their LDS writes.
        typename F::Cursor ca[R], cb[R];
        typename F::Raw ra[R], rb[R];
        const uint32_t stride = gridDim.x;
        auto request = [&](uint32_t rgq, typename F::Cursor (&c)[R], typename F::Raw (&w)[R]) {
            const bool live = rgq < n_rg;
            const uint32_t row0 = rgq * ROWS_PER_WG + (wave * GROUPS + grp) * R;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                c[r] = F::cursor(seg.w, live ? ((row0 + r < N) ? row0 + r : N - 1) : 0u, live ? gl : 0u);
                w[r] = load_unit<F, G>(c[r], 0, false);
            }
        };
        auto finish = [&](uint32_t rgq, const typename F::Cursor (&c)[R], const typename F::Raw (&w)[R]) {
            const uint32_t row0 = rgq * ROWS_PER_WG + (wave * GROUPS + grp) * R;
            float acc[R][T];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < T; ++t) acc[r][t] = 0.f;
            gemv_step<F, T, R>(w, c, gl, act, acc);
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    float v = group_sum<G>(acc[r][t]);
                    if (lane == (uint32_t)group_sum_lane<G>(lane) && row0 + r < N && (uint32_t)t < T_real) {
                        if (seg.bias) v += seg.bias[row0 + r];
                        store_out(seg.y + (size_t)t * N + row0 + r, v);
                    }
                }
        };
        uint32_t rg = blockIdx.x;
        act = stage_act<F::SUM_GRAN, T>(lds, xrow, 0, K, KT, q8_split != 0, [&]() { request(rg, ca, ra); });
        __syncthreads();
        for (; rg < n_rg; rg += 2 * stride) {
            request(rg + stride, cb, rb);
            __builtin_amdgcn_sched_barrier(0);
            finish(rg, ca, ra);
            request(rg + 2 * stride, ca, ra);
            __builtin_amdgcn_sched_barrier(0);
            if (rg + stride < n_rg) finish(rg + stride, cb, rb);
        }
        return;
    }
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x) {
        const uint32_t row0 = rg * ROWS_PER_WG + (wave * GROUPS + grp) * R;
        float acc[R][T];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < T; ++t) acc[r][t] = 0.f;
        for (uint32_t tile = 0; tile < n_tiles; ++tile) {
            const uint32_t k0 = tile * KT, kt = (K - k0 < KT) ? K - k0 : KT;
            typename F::Cursor cu[R];
#pragma unroll
            for (int r = 0; r < R; ++r) cu[r] = F::cursor(seg.w, (row0 + r < N) ? row0 + r : N - 1, k0 / 64 + gl);
            const uint32_t n_units = (kt + 63) / 64;
            const bool half_tail = (kt & 63u) != 0;
            if (T == 1 && kPrefetchAcrossRows<F> && n_tiles == 1 && !staged && (half_tail ? n_units - 1 : n_units) / G >= (uint32_t)U) {
                // first row group of a single-tile launch: the first round of weights is requested before the
                // activation row is staged (a long row stages for a microsecond or two before its first load otherwise)
                typename F::Raw pre[U][R];
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int r = 0; r < R; ++r) pre[u][r] = load_unit<F, G>(cu[r], u, false);
                act = stage_act<F::SUM_GRAN, T>(lds, xrow, k0, kt, KT, q8_split != 0);
                __syncthreads();
                staged = true;
                gemv_rows<F, T, R, G, U>(cu, n_units, half_tail, gl, act, acc, pre);
                continue;
            }
            if (n_tiles > 1 || !staged) {
                __syncthreads();
                act = stage_act<F::SUM_GRAN, T>(lds, xrow, k0, kt, KT, q8_split != 0);
                __syncthreads();
                staged = true;
            }
            gemv_rows<F, T, R, G, U>(cu, n_units, half_tail, gl, act, acc);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < T; ++t) {
                float v = group_sum<G>(acc[r][t]);
                if (lane == (uint32_t)group_sum_lane<G>(lane) && row0 + r < N && (uint32_t)t < T_real) {
                    if (seg.bias) v += seg.bias[row0 + r];
                    store_out(seg.y + (size_t)t * N + row0 + r, v);
                }
            }
    }
}

// Long rows with few of them, one token (the 14336 -> 4096 down projections): a launch with at most two workgroups per
// CU, where a lane group walks its row in several rounds.  The plain walk loads a round, waits, sums, loads the next:
// every wave has nothing in flight while it sums.  Here two rounds of U units rotate through two register sets
// (never copied), so one round is always in flight while the other is summed, and both are requested before the
// activation row is staged.  Twice the registers for units, which a launch this sparse can afford.
template <class F, int G, class OutT>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_deep_kernel(GemvSeg<F, OutT> seg, const uint8_t* xq8, uint32_t K, uint32_t N, uint32_t KT,
                                                                     uint32_t q8_split) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G, U = 2, R = 1, T = 1;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    auto xrow = [&](uint32_t) { return xq8; };
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_units = (K + 63) / 64;
    const bool half_tail = (K & 63u) != 0;
    const uint32_t n_whole = half_tail ? n_units - 1 : n_units;
    const uint32_t nb = n_whole / G / U;   // full rounds of U units per lane
    ActTile act;
    bool staged = false;
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x) {
        const uint32_t row = rg * ROWS_PER_WG + wave * GROUPS + grp;
        typename F::Cursor cu[R];
        cu[0] = F::cursor(seg.w, row < N ? row : N - 1, gl);
        typename F::Raw a[U][R], b[U][R];
        auto fetch = [&](typename F::Raw (&dst)[U][R], uint32_t round) {
#pragma unroll
            for (int u = 0; u < U; ++u) dst[u][0] = load_unit<F, G>(cu[0], round * U + u, false);
        };
        auto sum = [&](const typename F::Raw (&src)[U][R], uint32_t round, float (&acc)[R][T]) {
#pragma unroll
            for (int u = 0; u < U; ++u) gemv_step<F, T, R>(src[u], cu, gl + (round * U + u) * G, act, acc);
        };
        if (nb >= 1) fetch(a, 0);
        if (nb >= 2) fetch(b, 1);
        if (!staged) {
            act = stage_act<F::SUM_GRAN, T>(lds, xrow, 0, K, KT, q8_split != 0);
            __syncthreads();
            staged = true;
        }
        float acc[R][T] = {{0.f}};
        uint32_t k = 0;
        for (; k + 2 <= nb; k += 2) {
            sum(a, k, acc);
            if (k + 2 < nb) fetch(a, k + 2);
            sum(b, k + 1, acc);
            if (k + 3 < nb) fetch(b, k + 3);
        }
        if (k < nb) sum(a, k, acc);
        for (uint32_t it = nb * U; it * G + gl < n_units; ++it) {   // the ragged rest, predicated
            typename F::Raw raw[R];
            raw[0] = load_unit<F, G>(cu[0], it, half_tail && (it * G + gl == n_units - 1));
            gemv_step<F, T, R>(raw, cu, gl + it * G, act, acc);
        }
        float v = group_sum<G>(acc[0][0]);
        if (lane == (uint32_t)group_sum_lane<G>(lane) && row < N) {
            if (seg.bias) v += seg.bias[row];
            store_out(seg.y + row, v);
        }
    }
}

// Rows much longer than a wave can cover in one step (K >= 8192) with few of them (N = 4096: the down
// projections): the whole workgroup walks R rows at a time, thread t of 256 taking units t, t + 256, ...,
// and the four wave sums meet in LDS.  One memory round trip per row instead of K / 64 / G of them, and
// G / 256 times fewer rows per workgroup, so that a short matrix still fills every CU.  Single K tile only.
template <class F, int T, int R, class OutT>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_wide_kernel(GemvSeg<F, OutT> seg0, GemvSeg<F, OutT> seg1, const uint8_t* xq8, uint32_t K,
                                                                     uint32_t N, uint32_t KT, uint32_t T_real, uint32_t q8_split) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ float red[2][kGemvWaves][R][T];
    const GemvSeg<F, OutT>& seg = blockIdx.y ? seg1 : seg0;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const size_t q8_row_bytes = (size_t)(K / 32) * (q8_split ? kQ81sBytes : kQ81xBytes);
    auto xrow = [&](uint32_t t) { return xq8 + (size_t)(t < T_real ? t : T_real - 1) * q8_row_bytes; };
    // q8_split == 2: `xq8` is one fp16 row, quantized while it is staged (T = 1; the same tile as staging quantize_q8_1's output)
    ActTile act;
    if (T == 1 && q8_split == 2u) {
        auto hrow = [&](uint32_t) { return reinterpret_cast<const half_t*>(xq8); };
        act = stage_act_f16<F::SUM_GRAN, T>(lds, hrow, 0, K, KT);
    } else {
        act = stage_act<F::SUM_GRAN, T>(lds, xrow, 0, K, KT, q8_split != 0);
    }
    __syncthreads();
    const uint32_t n_units = (K + 63) / 64, n_rg = (N + R - 1) / R;
    const bool half_tail = (K & 63u) != 0;
    uint32_t par = 0;
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x, par ^= 1u) {
        const uint32_t row0 = rg * R;
        float acc[R][T];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < T; ++t) acc[r][t] = 0.f;
        typename F::Cursor cu[R];
#pragma unroll
        for (int r = 0; r < R; ++r) cu[r] = F::cursor(seg.w, (row0 + r < N) ? row0 + r : N - 1, tid);
        gemv_rows<F, T, R, kGemvThreads, 1>(cu, n_units, half_tail, tid, act, acc);
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float v = group_sum<64>(acc[r][t]);
                if (lane == (uint32_t)group_sum_lane<64>(lane)) red[par][wave][r][t] = v;
            }
        __syncthreads();   // one barrier per row group: the sums alternate between two buffers
        if (tid < R * T) {
            const uint32_t r = tid / T, t = tid % T;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kGemvWaves; ++w) v += red[par][w][r][t];
            if (row0 + r < N && t < T_real) {
                if (seg.bias) v += seg.bias[row0 + r];
                store_out(seg.y + (size_t)t * N + row0 + r, v);
            }
        }
    }
}

// The workgroup-wide walk when a row's units fill a whole number of half waves but fewer than four waves (K = 14336:
// 224 units, three and a half waves, so one lane in eight of gemv_q8_wide_kernel idles): a workgroup of 2 * units threads takes
// two rows at a time, thread t unit t % units of row t / units; the middle wave holds the end of one row in its first
// 32 lanes and the start of the other in the rest.  Every wave sums its two halves separately; after the barrier one
// thread per row adds that row's half-wave sums in order.  Measured against gemv_q8_wide_kernel at 14336 -> 4096, three
// workgroups per CU: Q6_K 13.2 -> 12.2 us, Q8_0 planes 12.2 -> 12.05; both down projections inside the decode step
// 65.3 -> 63.3 us (two workgroups per CU: 12.5 / 12.1 us, one: 17.0 / 14.7, four: the step 66.9).
// q8_split == 2: `xq8` is one fp16 row, quantized while it is staged.
template <class F, class OutT>
__global__ __launch_bounds__(512) void gemv_q8_wide_pair_kernel(GemvSeg<F, OutT> seg, const uint8_t* xq8, uint32_t K, uint32_t N, uint32_t KT,
                                                                 uint32_t q8_split) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ float red[2][16];   // [buffer][half wave]
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n_units = K / 64, halves_per_row = n_units / 32;
    const uint32_t slot = tid >= n_units ? 1u : 0u, unit = tid - slot * n_units;
    auto xrow = [&](uint32_t) { return xq8; };
    ActTile act;
    if (q8_split == 2u) {
        auto hrow = [&](uint32_t) { return reinterpret_cast<const half_t*>(xq8); };
        act = stage_act_f16<F::SUM_GRAN, 1>(lds, hrow, 0, K, KT);
    } else {
        act = stage_act<F::SUM_GRAN, 1>(lds, xrow, 0, K, KT, q8_split != 0);
    }
    __syncthreads();
    const uint32_t n_rg = (N + 1) / 2;
    uint32_t par = 0;
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x, par ^= 1u) {
        const uint32_t row = 2 * rg + slot;
        typename F::Cursor cu[1];
        typename F::Raw raw[1];
        cu[0] = F::cursor(seg.w, row < N ? row : N - 1, unit);
        raw[0] = load_unit<F, kGemvThreads>(cu[0], 0, false);
        float acc[1][1] = {{0.f}};
        gemv_step<F, 1, 1>(raw, cu, unit, act, acc);
        const float v = group_sum<32>(acc[0][0]);
        if ((lane & 31u) == 31u) red[par][2 * wave + (lane >> 5)] = v;
        __syncthreads();   // one barrier per row pair: the sums alternate between two buffers
        if (tid < 2 && 2 * rg + tid < N) {
            float r = 0.f;
            for (uint32_t hw = tid * halves_per_row; hw < (tid + 1) * halves_per_row; ++hw) r += red[par][hw];
            if (seg.bias) r += seg.bias[2 * rg + tid];
            store_out(seg.y + 2 * rg + tid, r);
        }
    }
}

// true if the launch was made: one matrix, one token, a whole number of half waves per row and fewer than four waves
// (K = 8192, Q8_0 planes: 9.45 -> 8.35 us; K = 12288: 11.1 -> 10.9; with 256 units gemv_q8_wide_kernel has no idle lane)
static int cu_count();
constexpr uint32_t kWidePairWgsPerCu = 3;
template <class F, class OutT>
static bool launch_wide_pair(hipStream_t st, const GemvSeg<F, OutT>& g, const uint8_t* x, uint32_t K, uint32_t N, uint32_t KT, uint32_t q8_split) {
    const uint32_t units = K / 64;
    if (K % 64 != 0 || units % 32 != 0 || units >= 256) return false;
    const uint32_t cap = (uint32_t)cu_count() * kWidePairWgsPerCu, n_rg = (N + 1) / 2;
    hipLaunchKernelGGL((gemv_q8_wide_pair_kernel<F, OutT>), dim3(n_rg < cap ? n_rg : cap), dim3(2 * units), act_tile_bytes(1, KT, F::SUM_GRAN), st, g, x, K, N, KT, q8_split);
    return true;
}

// Batched launches with long rows and few of them (T >= 2, K >= 8192: the down projections in a speculative-verify
// batch): the row-group grid alone leaves CUs idle and every workgroup restages several activation tiles.  Here
// the grid is (row groups, K slices): a workgroup stages one slice once and writes its partial sums to a scratch
// plane, part[(slice * T + t) * N + row]; a second, tiny launch adds the slices in slice order and writes y.  (A
// single launch with a last-arriver reduction needs device-scope fences, which on this part write back the XCD's
// L2: measured five times slower than the two launches.)
// The scratch is either a workspace the caller passes (the *_ws entry points) or the file-scope device array below,
// which the library owns: no entry point allocates.  The array exists once per device and keeps the last call's
// contents; every element a reduction reads was written by the split launch in front of it, so nothing needs
// clearing, but two calls that overlap on one device (different streams, graph branches) would race on it, as calls
// sharing the reference's static per-device scratch buffers do (src/model/dense_dispatch.hpp:547-560).
constexpr uint32_t kSplitMaxSlices = 4;
constexpr uint64_t kSplitElems = 4ull * 8 * 16384;   // 2 MB: four slices of eight tokens of 16384 rows
static __device__ __align__(256) float g_splitk_part[kSplitElems];
static std::atomic<void*> g_splitk_addr[kMaxDevices];

int gemv_init_device() {
    void* p = nullptr;
    return scratch_address(HIP_SYMBOL(g_splitk_part), g_splitk_addr, &p);
}

// the library-owned scratch of the current device as a SplitWs
static int static_split_ws(SplitWs* ws) {
    void* p = nullptr;
    if (int rc = scratch_address(HIP_SYMBOL(g_splitk_part), g_splitk_addr, &p)) return rc;
    *ws = SplitWs{static_cast<float*>(p), kSplitElems, false};
    return MX_OK;
}

template <class F, int T, int R, int G>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_splitk_kernel(typename F::W w, const uint8_t* xq8, float* part, uint32_t K, uint32_t N,
                                                                       uint32_t KS, uint32_t T_real, uint32_t q8_split) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS * R;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    const uint32_t rg = blockIdx.x, ks = blockIdx.y;
    const uint32_t k0 = ks * KS, kt = (K - k0 < KS) ? K - k0 : KS;
    const size_t q8_row_bytes = (size_t)(K / 32) * (q8_split ? kQ81sBytes : kQ81xBytes);
    auto xrow = [&](uint32_t t) { return xq8 + (size_t)(t < T_real ? t : T_real - 1) * q8_row_bytes; };
    const ActTile act = stage_act<F::SUM_GRAN, T>(lds, xrow, k0, kt, KS, q8_split != 0);
    __syncthreads();
    const uint32_t row0 = rg * ROWS_PER_WG + (wave * GROUPS + grp) * R;
    float acc[R][T];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < T; ++t) acc[r][t] = 0.f;
    typename F::Cursor cu[R];
#pragma unroll
    for (int r = 0; r < R; ++r) cu[r] = F::cursor(w, (row0 + r < N) ? row0 + r : N - 1, k0 / 64 + gl);
    gemv_rows<F, T, R, G, 1>(cu, (kt + 63) / 64, (kt & 63u) != 0, gl, act, acc);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float v = group_sum<G>(acc[r][t]);
            if (lane == (uint32_t)group_sum_lane<G>(lane) && row0 + r < N && (uint32_t)t < T_real)
                part[((size_t)ks * T_real + t) * N + row0 + r] = v;
        }
}

template <class OutT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(OutT* y, const float* bias, const float* part, uint32_t N, uint32_t T_real, uint32_t n_split) {
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (row >= N || t >= T_real) return;
    float v = 0.f;
    for (uint32_t k = 0; k < n_split; ++k) v += part[((size_t)k * T_real + t) * N + row];
    if (bias) v += bias[row];
    store_out(y + (size_t)t * N + row, v);
}

// Up to three matrices of different N that share one quantized activation row, in one launch: the
// workgroups tile the concatenated row space, so small projections (GQA k / v) ride a full grid
// (gemv_q4_0_soa_q8_multi, include/ie/ops.hpp:577-592).  T = 1.
template <class F>
struct GemvBanks {
    typename F::W w[3];
    half_t* y[3];
    uint32_t rg_end[3];   // cumulative row-group counts
    uint32_t n[3];
};
template <class F, int G>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_multi_kernel(GemvBanks<F> bk, const uint8_t* xq8, uint32_t K, uint32_t KT, int n_banks) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G, U = 2;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    auto xrow = [&](uint32_t) { return xq8; };
    const uint32_t n_tiles = (K + KT - 1) / KT;
    const uint32_t total_rg = bk.rg_end[n_banks - 1];
    ActTile act;
    bool staged = false;
    for (uint32_t rg = blockIdx.x; rg < total_rg; rg += gridDim.x) {
        const int b = (rg < bk.rg_end[0]) ? 0 : (rg < bk.rg_end[1] ? 1 : 2);
        const uint32_t N = bk.n[b];
        const uint32_t row = (rg - (b ? bk.rg_end[b - 1] : 0u)) * ROWS_PER_WG + wave * GROUPS + grp;
        float acc[1][1] = {{0.f}};
        for (uint32_t tile = 0; tile < n_tiles; ++tile) {
            const uint32_t k0 = tile * KT, kt = (K - k0 < KT) ? K - k0 : KT;
            typename F::Cursor cu[1] = {F::cursor(bk.w[b], row < N ? row : N - 1, k0 / 64 + gl)};
            if (n_tiles > 1 || !staged) {
                __syncthreads();
                act = stage_act<F::SUM_GRAN, 1>(lds, xrow, k0, kt, KT, false);
                __syncthreads();
                staged = true;
            }
            gemv_rows<F, 1, 1, G, U>(cu, (kt + 63) / 64, (kt & 63u) != 0, gl, act, acc);
        }
        const float v = group_sum<G>(acc[0][0]);
        if (lane == (uint32_t)group_sum_lane<G>(lane) && row < N) store_out(bk.y[b] + row, v);
    }
}

// ---------------------------------------------------------------- float activations (T = 1)
// Same unit walk; activations staged as fp32 plus per-16 sums; the fold is the
// reference's acc += (d*sc) * sum(a*q) - (dmin*m) * sum(a)  (src/ops/gemv_q4k.cpp:119-146).
// blockIdx.y selects one of two weight matrices that share the activation (gemv_q4_K_dual,
// src/ops/gemv_q4k.cpp:170-275); accum_scale != NULL turns the store into the scaled
// accumulate y = half(float(y) + float(accum_scale[0]) * acc) (gemv_q4_K_down_accum, :398-472).
// Epilogues of the float-activation kernel.  FACT_STORE: plain / dual (grid.y picks the matrix) /
// scaled accumulate.  The pair modes walk the same row of two matrices in one lane group:
// FACT_SILU_PAIR writes y0[n] = half(silu(g) * u) and one extra workgroup writes the shared-expert
// gate scalar sigmoid(W_shg . A) (gemv_q4_K_shexp_gate_up, src/ops/gemv_q4k.cpp:288-395);
// FACT_GBETA rounds both sums through fp16 and writes g = A_log[n] * softplus(a + dt_bias[n]),
// beta = sigmoid(b) (gemv_q4_K_dual_ssm_gbeta, src/ops/gemv_q4k.cpp:480-590).
enum { FACT_STORE = 0, FACT_SILU_PAIR = 1, FACT_GBETA = 2 };
struct FactTail {
    const float* p0;   // SILU_PAIR: W_shg [K];   GBETA: A_log [N]
    const float* p1;   //                         GBETA: dt_bias [N]
    void* o0;          // SILU_PAIR: sh_g_out (fp16 scalar);  GBETA: g_out (fp32 [N])
    void* o1;          //                                     GBETA: beta_out (fp32 [N])
};

template <class F, int R, int G, class ActT, class OutT, int EPI>
__global__ __launch_bounds__(kGemvThreads) void gemv_fact_kernel(typename F::W w0, typename F::W w1, const ActT* A, OutT* y0, OutT* y1,
                                                                  const half_t* accum_scale, FactTail tail, uint32_t K, uint32_t N, uint32_t KT) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr bool PAIR = EPI != FACT_STORE;
    static_assert(!PAIR || R == 2, "pair modes keep one row of each matrix per lane group");
    const typename F::W& w = (!PAIR && blockIdx.y) ? w1 : w0;
    OutT* y = (!PAIR && blockIdx.y) ? y1 : y0;
    float* xa = reinterpret_cast<float*>(lds);          // [KT]
    float* s16 = xa + KT;                                // [KT/16]
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS * (PAIR ? 1 : R);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_tiles = (K + KT - 1) / KT;
    uint32_t n_wg = gridDim.x;
    if constexpr (EPI == FACT_SILU_PAIR) {
        // last workgroup: the gate scalar, a plain fp32 dot over the whole workgroup
        n_wg -= 1;
        if (blockIdx.x == n_wg) {
            float part = 0.f;
            for (uint32_t i = threadIdx.x; i < K; i += blockDim.x) part += load_act(A + i) * tail.p0[i];
            part = group_sum<64>(part);
            if (lane == (uint32_t)group_sum_lane<64>(lane)) xa[wave] = part;
            __syncthreads();
            if (threadIdx.x == 0) {
                float dot = 0.f;
                for (int i = 0; i < kGemvWaves; ++i) dot += xa[i];
                static_cast<half_t*>(tail.o0)[0] = (half_t)(1.0f / (1.0f + __expf(-dot)));
            }
            return;
        }
    }
    bool staged = false;
    // One K tile that one staging round covers (16 floats per thread): request the activation chunk, then the first row
    // group's weight units, and only then touch the activations.  Loads return in order, so the wait for the chunk
    // leaves the younger weight requests in flight while the row is written to LDS.
    typename F::Raw pre[R];
    const bool lead = n_tiles == 1 && K <= 16u * kGemvThreads && blockIdx.x < n_rg;
    const bool pre_live = lead && gl < (K + 63) / 64 && (K & 63u) == 0;
    if (lead) {
        float v[16];
        const uint32_t i = threadIdx.x;
        const bool live = i < (K + 63) / 64 * 4;
        if (live && i * 16 < K) {
            load16(A + i * 16, v);
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) v[j] = 0.f;
        }
        if (pre_live) {
            const uint32_t prow0 = blockIdx.x * ROWS_PER_WG + (wave * GROUPS + grp) * (PAIR ? 1 : R);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t row = PAIR ? prow0 : prow0 + r;
                const typename F::Cursor c = F::cursor((PAIR && r) ? w1 : w, row < N ? row : N - 1, gl);
                pre[r] = load_unit<F, G>(c, 0, false);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (live) {
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) sum += v[j];
#pragma unroll
            for (int j = 0; j < 4; ++j) reinterpret_cast<float4*>(xa)[fact_slot(i * 4 + j)] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
            s16[i] = sum;
        }
        __syncthreads();
        staged = true;
    }
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += n_wg) {
        const uint32_t row0 = rg * ROWS_PER_WG + (wave * GROUPS + grp) * (PAIR ? 1 : R);
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = 0.f;
        for (uint32_t tile = 0; tile < n_tiles; ++tile) {
            const uint32_t k0 = tile * KT, kt = (K - k0 < KT) ? K - k0 : KT;
            if (n_tiles > 1 || !staged) {
                __syncthreads();
                stage_fact(xa, s16, A + k0, kt);
                __syncthreads();
                staged = true;
            }
            const uint32_t n_units = (kt + 63) / 64;
            const bool half_tail = (kt & 63u) != 0;
            typename F::Cursor cu[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t row = PAIR ? row0 : row0 + r;
                cu[r] = F::cursor((PAIR && r) ? w1 : w, row < N ? row : N - 1, k0 / 64 + gl);
            }
            for (uint32_t it = 0; it * G + gl < n_units; ++it) {
                const uint32_t ul = it * G + gl, e0 = F::elem_off(ul);
                typename F::Raw raw[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (pre_live && it == 0 && rg == blockIdx.x) raw[r] = pre[r];
                    else raw[r] = load_unit<F, G>(cu[r], it, half_tail && ul == n_units - 1);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    acc[r] += fact_unit<F>(raw[r], cu[r], xa, s16, e0);
                }
            }
        }
        float v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = group_sum<G>(acc[r]);
        const bool writer = lane == (uint32_t)group_sum_lane<G>(lane);
        if constexpr (EPI == FACT_STORE) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (writer && row0 + r < N) {
                    if (accum_scale) store_out(y + row0 + r, load_act(y + row0 + r) + (float)accum_scale[0] * v[r]);
                    else store_out(y + row0 + r, v[r]);
                }
            }
        } else if constexpr (EPI == FACT_SILU_PAIR) {
            if (writer && row0 < N) store_out(y + row0, v[0] / (1.0f + __expf(-v[0])) * v[1]);
        } else {
            if (writer && row0 < N) {
                const float a_h = (float)(half_t)v[0] + tail.p1[row0];
                const float sp = fmaxf(a_h, 0.f) + log1pf(__expf(-fabsf(a_h)));
                static_cast<float*>(tail.o0)[row0] = tail.p0[row0] * sp;
                static_cast<float*>(tail.o1)[row0] = 1.0f / (1.0f + __expf(-(float)(half_t)v[1]));
            }
        }
    }
}

// ---------------------------------------------------------------- host dispatch
static int cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    }
    return n;
}

constexpr uint32_t kLdsBudget = 48 * 1024;
// Workgroups of `kernel` that fit one CU at once (registers and `lds` bytes of dynamic LDS), asked once per kernel and
// LDS size class (4 KB steps: the activation tile runs from a few KB to 48 KB with K and T, and the answer changes with
// it).  Persistent grids are sized with it: a workgroup that does not fit next to the others would run alone after them.
static uint32_t resident_wgs(const void* kernel, uint32_t lds) {
    constexpr int kSlots = 1024;   // a fixed table (nothing is allocated): entries beyond it are asked about every time
    static std::atomic<uintptr_t> key[kSlots];
    static std::atomic<uint32_t> val[kSlots];
    const uint32_t cls = (lds + 4095u) / 4096u;                                  // 0 .. 40
    const uintptr_t want = reinterpret_cast<uintptr_t>(kernel) * 64u + cls;     // user-space addresses leave the top bits free
    for (int i = 0; i < kSlots; ++i) {
        const uintptr_t k = key[i].load(std::memory_order_acquire);
        if (k == want) {
            const uint32_t v = val[i].load(std::memory_order_acquire);
            if (v) return v;
            break;   // another thread is filling the slot: ask as well
        }
        if (!k) break;
    }
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, (int)kGemvThreads, cls * 4096u) != hipSuccess || n < 1) n = 1;
    for (int i = 0; i < kSlots; ++i) {
        uintptr_t expected = 0;
        if (key[i].compare_exchange_strong(expected, want, std::memory_order_acq_rel) || expected == want) {
            val[i].store((uint32_t)n, std::memory_order_release);
            break;
        }
    }
    return (uint32_t)n;
}
constexpr int kRows = 2;             // rows per lane group, float-activation kernels
constexpr uint32_t kWgsPerCu = 4;    // persistent grid: workgroups per CU
constexpr uint32_t kWideF16WgsPerCu = 3;   // the workgroup-wide walk on an fp16 row: every workgroup quantizes the whole row while staging it
// rows per lane group / unroll of the unit walk: one row and two units in flight for a single
// token; batched, two rows share each activation read once the per-token work dominates
// (T > 4, or T > 2 for the formats whose fold carries a min term), one row below that
template <int T, int SUM_GRAN> struct GemvShape {
    static constexpr int R = (T <= 2 || (T <= 4 && (SUM_GRAN == 0 || SUM_GRAN == 2))) ? 1 : 2, U = (T == 1) ? 2 : 1;
};

// Q8_0 planes, one token: rows that a wave covers in one round of loads (K <= 4096, whole 512-element spans) take the
// interleaved unit walk (FmtQ8SoaW).  Longer rows keep the plain units in the lane-group kernels: those hold several
// rounds of units in registers, and the interleaved form's cross-lane scale exchange costs them a workgroup per CU
// (14336 -> 4096: 13.4 us plain, 15.7 - 18.4 us interleaved); long rows of a short matrix take the interleaved units
// in the workgroup-wide walk instead (gemv_q8_0_soa_batched).
static bool q8_soa_interleaved(uint32_t K) { return K % FmtQ8SoaW::K_ALIGN == 0 && K <= 4096u; }

// long rows of a short matrix (one round of the whole workgroup per row): see gemv_q8_0_soa_batched
static bool q8_soa_wide(uint32_t K, uint32_t N) {
    return K % FmtQ8SoaW::K_ALIGN == 0 && K >= 8192u && K <= 64u * (uint32_t)kGemvThreads && N <= 16u * (uint32_t)cu_count();
}

// lanes per row: the G in {16, 32, 64} that wastes the fewest lane slots, larger on ties
static uint32_t pick_group(uint32_t units) {
    uint32_t best = 64, waste = (units + 63) / 64 * 64 - units;
    for (uint32_t g : {32u, 16u}) {
        const uint32_t w = (units + g - 1) / g * g - units;
        if (w < waste) { best = g; waste = w; }
    }
    return best;
}

template <class F, int T, int G, class OutT>
static int launch_q8_tg(hipStream_t st, const GemvSeg<F, OutT>& s0, const GemvSeg<F, OutT>& s1, int nseg, const uint8_t* xq8,
                        uint32_t K, uint32_t N, uint32_t T_real, bool split, const SplitWs& ws) {
    // GGUF Q8_0 blocks are 17 dword loads per unit: one unit in flight (measured at T = 1 against two: K = 4096,
    // N = 14336 18.1 -> 15.8 us; K = 14336, N = 4096 18.1 -> 16.6 us)
    constexpr int R = GemvShape<T, F::SUM_GRAN>::R, U = std::is_same<F, FmtQ8Aos>::value ? 1 : GemvShape<T, F::SUM_GRAN>::U;
    constexpr uint32_t rows_per_wg = kGemvWaves * (64 / G) * R;
    const uint32_t per_elem_x32 = qs_bytes_per32(F::SUM_GRAN) + hdr_bytes_per32(F::SUM_GRAN);   // LDS bytes per 32 activation elements
    const uint32_t KT_max = (kLdsBudget / (per_elem_x32 * T)) * 32 / 256 * 256;
    if (KT_max == 0) return MX_ERR_SHAPE;
    const uint32_t K256 = (K + 255) / 256, n_tiles = (K256 * 256 + KT_max - 1) / KT_max;
    const uint32_t KT = (K256 + n_tiles - 1) / n_tiles * 256;   // balanced tiles
    const uint32_t n_rg = (N + rows_per_wg - 1) / rows_per_wg;
    if constexpr (T == 1 && (F::SUM_GRAN == 16 || std::is_same<F, FmtQ4K>::value || std::is_same<F, FmtQ8Aos>::value)) {
        // long rows, too few of them to give every CU its workgroups: the workgroup-wide row walk.  Measured at
        // K = 14336, N = 4096: Q6_K 14.4 -> 12.7 us, 12.2 with paired rows; Q4_K gains nothing from the 256-thread walk
        // and 9.65 -> 8.8 us from the paired rows; no gain for T = 2.
        // (mx_gemv_q6_K_f16q8 / mx_gemv_q4_K_f16q8 take the same launch under the same condition, so that both forms give the same bits.)
        if (n_tiles == 1 && K >= 8192 && n_rg <= 2u * (uint32_t)cu_count()) {
            if (nseg == 1 && launch_wide_pair<F, OutT>(st, s0, xq8, K, N, KT, split ? 1u : 0u)) return launch_status();
            if constexpr (F::SUM_GRAN == 16) {
                const uint32_t capw = (uint32_t)cu_count() * kWgsPerCu / nseg;
                dim3 gridw(N < capw ? N : capw, nseg);
                hipLaunchKernelGGL((gemv_q8_wide_kernel<F, 1, 1, OutT>), gridw, dim3(kGemvThreads), act_tile_bytes(1, KT, F::SUM_GRAN), st, s0, s1, xq8, K, N, KT,
                                   T_real, split ? 1u : 0u);
                return launch_status();
            }
        }
    }
    if constexpr (T >= 2) {
        const uint32_t cus = (uint32_t)cu_count();
        if (nseg == 1 && K >= 8192 && (n_tiles > 1 || n_rg < 2u * cus)) {
            uint32_t n_split = (4u * cus + n_rg - 1) / n_rg;   // about four workgroups per CU
            if (n_split < n_tiles) n_split = n_tiles;
            if (n_split > kSplitMaxSlices) n_split = kSplitMaxSlices;
            const uint32_t KS = (K256 + n_split - 1) / n_split * 256;
            n_split = (K + KS - 1) / KS;
            if (n_split >= 2 && KS <= KT_max) {
                const bool fits = ws.ptr && (uint64_t)n_split * T_real * N <= ws.elems;
                if (!fits && ws.caller) return MX_ERR_WORKSPACE;   // a caller's workspace is never silently bypassed
                if (fits) {
                    hipLaunchKernelGGL((gemv_q8_splitk_kernel<F, T, R, G>), dim3(n_rg, n_split), dim3(kGemvThreads), act_tile_bytes(T, KS, F::SUM_GRAN),
                                       st, s0.w, xq8, ws.ptr, K, N, KS, T_real, split ? 1u : 0u);
                    hipLaunchKernelGGL((splitk_reduce_kernel<OutT>), dim3((N + 255) / 256, T_real), dim3(256), 0, st, s0.y, s0.bias, ws.ptr, N, T_real,
                                       n_split);
                    return launch_status();
                }
            }
        }
    }
    if constexpr (T == 1 && kPrefetchAcrossRows<F>) {
        // long rows, at most two workgroups per CU, at least two full rounds per lane: the two-round rotation
        if (nseg == 1 && n_tiles == 1 && n_rg <= 2u * (uint32_t)cu_count() && ((K & 63u) ? (K + 63) / 64 - 1 : (K + 63) / 64) / G >= 4u) {
            hipLaunchKernelGGL((gemv_q8_deep_kernel<F, G, OutT>), dim3(n_rg), dim3(kGemvThreads), act_tile_bytes(1, KT, F::SUM_GRAN), st, s0, xq8, K, N, KT,
                               split ? 1u : 0u);
            return launch_status();
        }
    }
    // A CU streams at a fixed rate (its waves' loads in flight over the memory latency), so the
    // launch is balanced per CU, not per workgroup: with a whole number of workgroups per CU
    // the dispatcher gives every CU the same number of them, and the strided row-group loop
    // hands each CU the same number of row groups to within one per workgroup.
    // The persistent grid holds as many workgroups per CU as are resident at once, at most kWgsPerCu: the batched
    // instances of some formats need more than 128 registers (Q6_K with three or four rows: 148 - 151), so only three
    // fit, and a fourth per CU would run alone after the others.
    const uint32_t lds = act_tile_bytes(T, KT, F::SUM_GRAN);
    uint32_t per_cu = resident_wgs(reinterpret_cast<const void*>(&gemv_q8_kernel<F, T, R, G, U, OutT>), lds);
    if (per_cu > kWgsPerCu) per_cu = kWgsPerCu;
    {
        // More waves than the memory system can serve only lengthen its queues; measured per format (K = 4096, us with
        // four workgroups per CU -> with the number chosen here).  Q8_0 planes, interleaved units (two rows per wave in
        // flight): fused gate + up 20.8 -> 20.45 and 128256 rows 88.3 -> 85.2 with two, 14336 rows 12.0 with two, three
        // or four.  GGUF Q8_0 blocks: one token 16.4 -> 14.9 and two 17.6 -> 16.0 with two, four tokens 19.1 -> 18.8
        // with three.  Q4_K, one token: 8.3 -> 8.0 with three (4096 rows: 4.37 -> 4.09).  Q6_K, one or two
        // tokens, with the two register sets of the one-unit-per-lane path (the same bytes in flight per CU as four
        // workgroups with one set, half the waves competing for the vector pipe): fused gate + up 19.7 -> 17.6 with two
        // (21.9 with one, 19.4 with three), 14336 rows 12.45 -> 11.3, 151936 rows 94.2 -> 88.5, 4096 rows 6.4 -> 5.1, two
        // tokens 14.5 -> 13.3; K = 8192: 16.1 -> 13.9 with three.
        const uint64_t rows = (uint64_t)nseg * N;
        uint32_t fewer = kWgsPerCu;
        if constexpr (T == 1 && std::is_same<F, FmtQ8SoaW>::value) fewer = rows >= 24576u ? 2u : 3u;
        else if constexpr (std::is_same<F, FmtQ8Aos>::value) fewer = T <= 2 ? 2u : (T <= 4 ? 3u : kWgsPerCu);
        else if constexpr (T == 1 && std::is_same<F, FmtQ4K>::value) fewer = 3u;
        else if constexpr (T <= 2 && std::is_same<F, FmtQ6K>::value) fewer = K <= 4096u ? 2u : 3u;
        if (per_cu > fewer) per_cu = fewer;
    }
    const uint32_t cap = (uint32_t)cu_count() * per_cu / nseg;
    dim3 grid(n_rg < cap ? n_rg : (cap ? cap : 1u), nseg);
    hipLaunchKernelGGL((gemv_q8_kernel<F, T, R, G, U, OutT>), grid, dim3(kGemvThreads), lds, st, s0, s1, xq8, K, N, KT, T_real, split ? 1u : 0u);
    return launch_status();
}

template <class F, int G, class OutT>
static int launch_q8_g(hipStream_t st, const GemvSeg<F, OutT>& s0, const GemvSeg<F, OutT>& s1, int nseg, const uint8_t* xq8, uint32_t K,
                       uint32_t N, uint32_t T, bool split, const SplitWs& ws) {
    switch (T) {
        case 1: return launch_q8_tg<F, 1, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
        case 2: return launch_q8_tg<F, 2, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
        case 3: return launch_q8_tg<F, 3, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
        case 4: return launch_q8_tg<F, 4, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
        case 5:
        case 6: return launch_q8_tg<F, 6, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
        case 7:
        case 8: return launch_q8_tg<F, 8, G, OutT>(st, s0, s1, nseg, xq8, K, N, T, split, ws);
    }
    return MX_ERR_SHAPE;
}

// ---------------------------------------------------------------- batches on the matrix cores (mxq_mmq.h)
// Formats with an int8 operand producer run every batch of two and more rows there: the weight stream is the same,
// the per-token dot products become one matrix instruction per block and 32 rows.
template <class F> struct MmqOf { using type = void; };
template <> struct MmqOf<FmtQ8Soa> { using type = MmqQ8Soa; };
template <> struct MmqOf<FmtQ8Aos> { using type = MmqQ8Aos; };
template <> struct MmqOf<FmtQ4K> { using type = MmqQ4K; };
template <> struct MmqOf<FmtQ6K> { using type = MmqQ6K; };
template <> struct MmqOf<FmtMxfp4Soa> { using type = MmqMxfp4Soa; };

static typename FmtQ8Soa::Bank mmq_bank(const FmtQ8Soa::W& w) { return {w.qs, w.d, 0, 0, w.K}; }
static typename FmtQ4K::Bank mmq_bank(const FmtQ4K::W& w) { return {w.base, 0, w.row_bytes}; }
static MmqQ8Aos::Bank mmq_bank(const FmtQ8Aos::W& w) { return {w.base, 0, w.row_bytes}; }
static typename FmtQ6K::Bank mmq_bank(const FmtQ6K::W& w) { return {w.base, 0, w.row_bytes}; }
static typename FmtMxfp4Soa::Bank mmq_bank(const FmtMxfp4Soa::W& w) { return {w.qs, w.e, 0, 0, w.K}; }

constexpr uint32_t kMmqLdsBudget = 48 * 1024;
constexpr uint32_t kMmqMaxRanges = 16;   // K ranges across workgroups of one dense launch

// staged k range per pass: the largest multiple of `gran` elements whose LDS image fits the budget
static uint32_t mmq_pass_range(uint32_t T, int TV, bool has_min, uint32_t gran) {
    const uint32_t per256 = T * 256u + 8u * (uint32_t)(2 * TV) * 4u * (has_min ? 2u : 1u);
    const uint32_t n256 = (kMmqLdsBudget - 32u * T) / per256;
    const uint32_t kr = n256 * 256u / gran * gran;
    return kr ? kr : gran;
}

// K ranges across workgroups of a dense launch when the row blocks alone leave CUs idle: about two workgroups per CU,
// every wave keeping at least two groups
static uint32_t mmq_dense_ranges(uint32_t K, uint32_t N, uint32_t WR, uint32_t WK) {
    const uint32_t cus = (uint32_t)cu_count();
    const uint32_t n_groups = (K / 32u + 7u) / 8u, rgs = (N + 32u * WR - 1u) / (32u * WR);
    uint32_t Z = 1;
    if (2u * rgs < 3u * cus) Z = (2u * cus + rgs - 1u) / rgs;
    if (Z > n_groups / (2u * WK)) Z = n_groups / (2u * WK);
    if (Z > kMmqMaxRanges) Z = kMmqMaxRanges;
    return Z < 1 ? 1 : Z;
}

template <class P, int TV, int WR, int WK>
static int launch_mmq_dense_cfg(hipStream_t st, const typename P::Bank& bank, const uint8_t* xq8, half_t* y, uint32_t K, uint32_t N, uint32_t T,
                                bool split, const SplitWs& ws) {
    const uint32_t nb = K / 32u, n_groups = (nb + 7u) / 8u;
    const uint32_t rgs = (N + 32u * WR - 1u) / (32u * WR);
    uint32_t Z = mmq_dense_ranges(K, N, WR, WK);   // the partial sums have to fit the scratch
    if (Z > 1 && (!ws.ptr || (uint64_t)Z * T * N > ws.elems)) {
        if (ws.caller) return MX_ERR_WORKSPACE;
        while (Z > 1 && (uint64_t)Z * T * N > ws.elems) --Z;
    }
    const uint32_t gz = (n_groups + Z - 1u) / Z;
    Z = (n_groups + gz - 1u) / gz;
    uint32_t kr = mmq_pass_range(T, TV, P::HAS_MIN, 256u * WK);
    const uint32_t need = (gz + WK - 1u) / WK * WK * 256u;
    if (kr > need) kr = need;
    MmqArgs<P> a{};
    a.bank0 = bank; a.bank1 = bank; a.xq8 = xq8; a.out = y; a.part = Z > 1 ? ws.ptr : nullptr;
    a.M = T; a.K = K; a.N = N; a.E = 1; a.q8_split = split ? 1u : 0u; a.kr = kr;
    const uint32_t red = (uint32_t)(WR * WK) * TV * 64u * 4u;
    a.red_off = (mmq_lds_bytes(T, kr, TV, P::HAS_MIN) + 15u) & ~15u;
    const uint32_t lds = a.red_off + red;
    hipLaunchKernelGGL((mmq_kernel<P, TV, 1, WR, WK, MMQ_STORE>), dim3(rgs, 1, Z), dim3(64 * WR * WK), lds, st, a);
    if (Z > 1) {
        const uint32_t mn = T * N;
        hipLaunchKernelGGL(mmq_reduce_kernel, dim3((mn + 255u) / 256u), dim3(256), 0, st, y, ws.ptr, mn, Z);
    }
    return launch_status();
}

template <class P>
static int launch_mmq_dense(hipStream_t st, const typename P::Bank& bank, const uint8_t* xq8, half_t* y, uint32_t K, uint32_t N, uint32_t T, bool split,
                            const SplitWs& ws) {
    if (T <= 8) return launch_mmq_dense_cfg<P, 4, 1, 4>(st, bank, xq8, y, K, N, T, split, ws);
    return launch_mmq_dense_cfg<P, 8, 2, 2>(st, bank, xq8, y, K, N, T, split, ws);
}

// T up to 16: passes of at most 8 tokens.
template <class F, class OutT>
static int launch_q8(mx_stream_t s, GemvSeg<F, OutT> s0, GemvSeg<F, OutT> s1, int nseg, const void* xq8, uint32_t K, uint32_t N, uint32_t T,
                     bool split = false, const SplitWs* caller_ws = nullptr) {
    const uint8_t* x = static_cast<const uint8_t*>(xq8);
    const uint32_t G = pick_group((K + 63) / 64);
    SplitWs ws{nullptr, 0, false};
    if (caller_ws) ws = *caller_ws;
    else if (T >= 2 && nseg == 1)   // the only launches that may split K
        if (int rc = static_split_ws(&ws)) return rc;
    using P = typename MmqOf<F>::type;
    if constexpr (!std::is_void<P>::value && std::is_same<OutT, half_t>::value) {
        // measured crossover against the vector-ALU batch kernels (4096 -> 14336, us): Q8_0 planes T = 4: 15.4 vs 16.1,
        // T = 8: 20.4 vs 17.6; Q6_K T = 8: 26.2 vs 22.0; batches of 9 .. 16 take one pass here instead of two there
        // (GGUF Q8_0 blocks: the 2-byte aligned block walk loses below a full second pass, 24.4 vs 30.9 us at T = 8)
        constexpr uint32_t kMmqFromT = std::is_same<F, FmtQ8Aos>::value ? 9u : 5u;
        // long rows (14336 -> 4096): batches of four cross over one row earlier for Q8_0 planes (19.6 vs 18.9 us) and Q6_K
        // (24.1 vs 22.7 us); Q4_K does not (15.4 vs 15.5 us)
        constexpr bool kEarlier = std::is_same<F, FmtQ8Soa>::value || std::is_same<F, FmtQ6K>::value;
        const uint32_t from = (kEarlier && K >= 8192u) ? kMmqFromT - 1u : kMmqFromT;
        if (T >= from && nseg == 1 && !s0.bias) return launch_mmq_dense<P>(as_stream(s), mmq_bank(s0.w), x, s0.y, K, N, T, split, ws);
    }
    for (uint32_t t0 = 0; t0 < T; t0 += 8) {
        const uint32_t tn = (T - t0 < 8) ? T - t0 : 8;
        GemvSeg<F, OutT> a = s0, b = s1;
        a.y = s0.y + (size_t)t0 * N;
        if (nseg > 1) b.y = s1.y + (size_t)t0 * N;
        const uint8_t* xt = x + (size_t)t0 * (K / 32) * (split ? kQ81sBytes : kQ81xBytes);
        const int rc = (G == 16)   ? launch_q8_g<F, 16, OutT>(as_stream(s), a, b, nseg, xt, K, N, tn, split, ws)
                       : (G == 32) ? launch_q8_g<F, 32, OutT>(as_stream(s), a, b, nseg, xt, K, N, tn, split, ws)
                                   : launch_q8_g<F, 64, OutT>(as_stream(s), a, b, nseg, xt, K, N, tn, split, ws);
        if (rc != MX_OK) return rc;
    }
    return MX_OK;
}

static int check_common(const void* x, const void* y, uint32_t K, uint32_t N, uint32_t T, uint32_t k_align) {
    MX_REQUIRE_PTR(x);
    MX_REQUIRE_PTR(y);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && K % k_align == 0);
    MX_REQUIRE_SHAPE(T >= 1 && T <= 16);
    return MX_OK;
}

template <class OutT>
static int gemv_aos_q8(int fmt, mx_stream_t s, const void* xq8, const void* W, OutT* y, uint32_t K, uint32_t N, uint32_t T, bool split = false,
                       const SplitWs* ws = nullptr) {
    const uint32_t k_align = fmt == 0 ? 32 : 256;
    if (int rc = check_common(xq8, y, K, N, T, k_align)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(xq8, split ? 16 : 8);
    MX_REQUIRE_ALIGN(W, fmt == 1 ? 16 : 2);
    const uint8_t* base = static_cast<const uint8_t*>(W);
    if (fmt == 1) {
        GemvSeg<FmtQ4K, OutT> g{{base, K / 256 * (uint32_t)kQ4KBytes}, y, nullptr};
        return launch_q8<FmtQ4K, OutT>(s, g, g, 1, xq8, K, N, T, split, ws);
    }
    if (fmt == 2) {
        GemvSeg<FmtQ6K, OutT> g{{base, K / 256 * (uint32_t)kQ6KBytes}, y, nullptr};
        return launch_q8<FmtQ6K, OutT>(s, g, g, 1, xq8, K, N, T, split, ws);
    }
    GemvSeg<FmtQ8Aos, OutT> g{{base, K / 32 * (uint32_t)kQ8_0Bytes}, y, nullptr};
    return launch_q8<FmtQ8Aos, OutT>(s, g, g, 1, xq8, K, N, T, split, ws);
}

template <class F, class ActT, class OutT, int EPI = FACT_STORE>
static int launch_fact(mx_stream_t s, const typename F::W& w, const ActT* A, OutT* y, uint32_t K, uint32_t N, const typename F::W* w_b = nullptr,
                       OutT* y_b = nullptr, const half_t* accum_scale = nullptr, FactTail tail = FactTail{}) {
    constexpr bool PAIR = EPI != FACT_STORE;
    const uint32_t nseg = (w_b && !PAIR) ? 2u : 1u;
    const typename F::W w1 = w_b ? *w_b : w;
    uint32_t KT = 8192;
    if (KT > K) KT = (K + 255) / 256 * 256;
    const uint32_t lds = KT * 4 + KT / 16 * 4;
    const uint32_t G = pick_group((K + 63) / 64);
    const uint32_t rows_per_wg = kGemvWaves * (64 / G) * (PAIR ? 1 : kRows);
    const uint32_t n_rg = (N + rows_per_wg - 1) / rows_per_wg;
    const void* kernel = G == 16   ? reinterpret_cast<const void*>(&gemv_fact_kernel<F, kRows, 16, ActT, OutT, EPI>)
                         : G == 32 ? reinterpret_cast<const void*>(&gemv_fact_kernel<F, kRows, 32, ActT, OutT, EPI>)
                                   : reinterpret_cast<const void*>(&gemv_fact_kernel<F, kRows, 64, ActT, OutT, EPI>);
    uint32_t per_cu = resident_wgs(kernel, lds);   // these kernels take 177 - 211 registers: two workgroups per CU
    if (per_cu > kWgsPerCu) per_cu = kWgsPerCu;
    uint32_t cap = (uint32_t)cu_count() * per_cu / nseg;   // persistent and CU-balanced, as the int-dot launch
    if (!cap) cap = 1;
    dim3 grid((n_rg < cap ? n_rg : cap) + (EPI == FACT_SILU_PAIR ? 1 : 0), nseg);
    if (G == 16)
        hipLaunchKernelGGL((gemv_fact_kernel<F, kRows, 16, ActT, OutT, EPI>), grid, dim3(kGemvThreads), lds, as_stream(s), w, w1, A, y, y_b, accum_scale, tail, K, N, KT);
    else if (G == 32)
        hipLaunchKernelGGL((gemv_fact_kernel<F, kRows, 32, ActT, OutT, EPI>), grid, dim3(kGemvThreads), lds, as_stream(s), w, w1, A, y, y_b, accum_scale, tail, K, N, KT);
    else
        hipLaunchKernelGGL((gemv_fact_kernel<F, kRows, 64, ActT, OutT, EPI>), grid, dim3(kGemvThreads), lds, as_stream(s), w, w1, A, y, y_b, accum_scale, tail, K, N, KT);
    return launch_status();
}

template <class ActT, class OutT>
static int gemv_aos_fact(int fmt, mx_stream_t s, const ActT* A, const void* W, OutT* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y, K, N, 1, fmt == 0 ? 32 : 256)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(W, fmt == 1 ? 16 : 2);
    const uint8_t* base = static_cast<const uint8_t*>(W);
    if (fmt == 1) return launch_fact<FmtQ4K>(s, FmtQ4K::W{base, K / 256 * (uint32_t)kQ4KBytes}, A, y, K, N);
    if (fmt == 2) return launch_fact<FmtQ6K>(s, FmtQ6K::W{base, K / 256 * (uint32_t)kQ6KBytes}, A, y, K, N);
    return launch_fact<FmtQ8Aos>(s, FmtQ8Aos::W{base, K / 32 * (uint32_t)kQ8_0Bytes}, A, y, K, N);
}

// Fused gate + up for the other int-dot formats: two matrices of the same shape against one q8 row, one
// launch (the shape of gemv_mxfp4_soa_q8_x2 above and of gemv_q4_K_dual_ffn; blockIdx.y picks the matrix).
template <class F>
static int gemv_x2(mx_stream_t s, const void* x, const typename F::W& wa, const typename F::W& wb, uint16_t* ya, uint16_t* yb, uint32_t K, uint32_t N) {
    GemvSeg<F, half_t> a{wa, reinterpret_cast<half_t*>(ya), nullptr}, b{wb, reinterpret_cast<half_t*>(yb), nullptr};
    return launch_q8<F, half_t>(s, a, b, 2, x, K, N, 1);
}
// Decode FFN forms (T = 1, one K tile): NW = 2 walks row n of the gate and of the up matrix together and writes
// h[n] = half(silu(half(g)) * half(u)), the rounding points of the three-launch chain gemv, gemv, swiglu
// (src/ops/elementwise.cpp:449-466 on fp16 g and u); NW = 1 is the plain GEMV.  XF16: the activation row arrives
// as fp16 and is quantized to q8 while it is staged (the same values as quantize_q8_1, so the same output bits),
// which removes the quantize launch in front of the GEMV.
template <class F, int NW, int G, int U, bool XF16>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_ffn_kernel(typename F::W w0, typename F::W w1, const void* x, half_t* y, uint32_t K, uint32_t N,
                                                                    uint32_t KT) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    ActTile act;
    if (XF16) {
        auto hrow = [&](uint32_t) { return static_cast<const half_t*>(x); };
        act = stage_act_f16<F::SUM_GRAN, 1>(lds, hrow, 0, K, KT);
    } else {
        auto xrow = [&](uint32_t) { return static_cast<const uint8_t*>(x); };
        act = stage_act<F::SUM_GRAN, 1>(lds, xrow, 0, K, KT, false);
    }
    __syncthreads();
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_units = (K + 63) / 64;
    const bool half_tail = (K & 63u) != 0;
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x) {
        const uint32_t n = rg * ROWS_PER_WG + wave * GROUPS + grp;
        const uint32_t nc = n < N ? n : N - 1;
        typename F::Cursor cu[NW];
        cu[0] = F::cursor(w0, nc, gl);
        if (NW == 2) cu[NW - 1] = F::cursor(w1, nc, gl);
        float acc[NW][1];
#pragma unroll
        for (int r = 0; r < NW; ++r) acc[r][0] = 0.f;
        gemv_rows<F, 1, NW, G, U>(cu, n_units, half_tail, gl, act, acc);
        const float v0 = group_sum<G>(acc[0][0]);
        const float v1 = (NW == 2) ? group_sum<G>(acc[NW - 1][0]) : 0.f;
        if (lane == (uint32_t)group_sum_lane<G>(lane) && n < N) {
            if (NW == 2) {
                const float g = (float)(half_t)v0, u = (float)(half_t)v1;
                y[n] = (half_t)((g / (1.f + __expf(-g))) * u);
            } else {
                y[n] = (half_t)v0;
            }
        }
    }
}

template <class F, int NW, bool XF16>
static int launch_ffn(mx_stream_t s, const typename F::W& w0, const typename F::W& w1, const void* x, uint16_t* y, uint32_t K, uint32_t N) {
    const uint32_t per_elem_x32 = qs_bytes_per32(F::SUM_GRAN) + hdr_bytes_per32(F::SUM_GRAN);
    const uint32_t KT = (K + 255) / 256 * 256;
    if ((uint64_t)KT / 32 * per_elem_x32 > kLdsBudget) return MX_ERR_SHAPE;   // the activation row has to fit one LDS tile
    const uint32_t G = pick_group((K + 63) / 64);
    const uint32_t rows_per_wg = kGemvWaves * (64 / G);
    const uint32_t n_rg = (N + rows_per_wg - 1) / rows_per_wg, cap = (uint32_t)cu_count() * kWgsPerCu;
    const dim3 grid(n_rg < cap ? n_rg : cap), block(kGemvThreads);
    const uint32_t lds = act_tile_bytes(1, KT, F::SUM_GRAN);
    half_t* yh = reinterpret_cast<half_t*>(y);
    constexpr int U = std::is_same<F, FmtQ8Aos>::value ? 1 : 2;
    if (G == 16) hipLaunchKernelGGL((gemv_q8_ffn_kernel<F, NW, 16, U, XF16>), grid, block, lds, as_stream(s), w0, w1, x, yh, K, N, KT);
    else if (G == 32) hipLaunchKernelGGL((gemv_q8_ffn_kernel<F, NW, 32, U, XF16>), grid, block, lds, as_stream(s), w0, w1, x, yh, K, N, KT);
    else hipLaunchKernelGGL((gemv_q8_ffn_kernel<F, NW, 64, U, XF16>), grid, block, lds, as_stream(s), w0, w1, x, yh, K, N, KT);
    return launch_status();
}
template <class F, int NW>
static int launch_ffn_x(mx_stream_t s, const typename F::W& w0, const typename F::W& w1, const void* x, int x_is_f16, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(x, y, K, N, 1, F::K_ALIGN)) return rc;
    MX_REQUIRE_ALIGN(x, x_is_f16 ? 16 : 8);
    return x_is_f16 ? launch_ffn<F, NW, true>(s, w0, w1, x, y, K, N) : launch_ffn<F, NW, false>(s, w0, w1, x, y, K, N);
}

// Streaming-read yardstick: the same persistent launch geometry as the decode GEMV (workgroups per CU x CUs,
// 256 threads, 16-byte loads, four in flight per thread) with no arithmetic, so that a GEMV launch can be
// priced against what a pure read of the same bytes achieves on the same device.
__global__ __launch_bounds__(kGemvThreads) void stream_read_kernel(const uint4* __restrict__ src, uint64_t n16, uint32_t* sink) {
    uint4 a = {0u, 0u, 0u, 0u};
    const uint64_t step = (uint64_t)gridDim.x * (kGemvThreads * 4u);
    for (uint64_t base = (uint64_t)blockIdx.x * (kGemvThreads * 4u) + threadIdx.x; base < n16; base += step) {
        uint4 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint64_t idx = base + (uint64_t)i * kGemvThreads;
            v[i] = idx < n16 ? src[idx] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a.x ^= v[i].x; a.y ^= v[i].y; a.z ^= v[i].z; a.w ^= v[i].w;
        }
    }
    const uint32_t r = a.x ^ a.y ^ a.z ^ a.w;
    if (r == 0x9E3779B9u && sink) sink[0] = r;   // keeps the loads; the value is of no interest
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_gemv_q4_K_q8(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<half_t>(1, s, x, W, reinterpret_cast<half_t*>(y), K, N, 1);
}
int mx_gemv_q6_K_q8(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<half_t>(2, s, x, W, reinterpret_cast<half_t*>(y), K, N, 1);
}
int mx_gemv_q8_0_q8(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<half_t>(0, s, x, W, reinterpret_cast<half_t*>(y), K, N, 1);
}
int mx_gemv_q4_K_q8_batched(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    return gemv_aos_q8<half_t>(1, s, x, W, reinterpret_cast<half_t*>(y), K, N, T);
}
int mx_gemv_q4_K_q8s_batched(mx_stream_t s, const void* x_q8s, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    return gemv_aos_q8<half_t>(1, s, x_q8s, W, reinterpret_cast<half_t*>(y), K, N, T, true);
}
int mx_gemv_q6_K_q8s_batched(mx_stream_t s, const void* x_q8s, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    return gemv_aos_q8<half_t>(2, s, x_q8s, W, reinterpret_cast<half_t*>(y), K, N, T, true);
}
int mx_gemv_q6_K_q8_batched(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    return gemv_aos_q8<half_t>(2, s, x, W, reinterpret_cast<half_t*>(y), K, N, T);
}
int mx_gemv_q8_0_q8_batched(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    return gemv_aos_q8<half_t>(0, s, x, W, reinterpret_cast<half_t*>(y), K, N, T);
}
int mx_gemv_q4_K_q8_f32(mx_stream_t s, const void* x, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<float>(1, s, x, W, y, K, N, 1);
}
int mx_gemv_q6_K_q8_f32(mx_stream_t s, const void* x, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<float>(2, s, x, W, y, K, N, 1);
}
int mx_gemv_q8_0_q8_f32(mx_stream_t s, const void* x, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_q8<float>(0, s, x, W, y, K, N, 1);
}

static int gemv_q8_0_soa_batched(mx_stream_t s, const void* x, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t K, uint32_t N,
                                 uint32_t T, const SplitWs* ws) {
    if (int rc = check_common(x, y, K, N, T, 32)) return rc;
    MX_REQUIRE_PTR(qs_W);
    MX_REQUIRE_PTR(d_W);
    MX_REQUIRE_ALIGN(x, 8);
    MX_REQUIRE_ALIGN(qs_W, 16);
    MX_REQUIRE_ALIGN(d_W, 2);
    if (T <= 2 && q8_soa_wide(K, N)) {
        // Long rows, few of them (the 14336 -> 4096 down projections): the workgroup-wide row walk with interleaved units.
        // A row is one round of whole-line nontemporal loads of the whole workgroup (224 of 256 threads at K = 14336) and
        // one round trip, and a short matrix still gives every CU its workgroups.  Measured against the two-round
        // rotation of the plain units (gemv_q8_deep_kernel): 13.9 -> 12.1 us (two rows per pass: 12.2 - 12.9 us); two
        // tokens against the lane-group walk: 15.7 -> 13.9 us.
        GemvSeg<FmtQ8SoaW, half_t> g{{qs_W, d_W, K}, reinterpret_cast<half_t*>(y), nullptr};
        // three workgroups per CU (one token: 12.5 us with four, 12.1 with three, 13.1 with two)
        const uint32_t KT = (K + 255) / 256 * 256, capw = (uint32_t)cu_count() * 3u;
        const dim3 gridw(N < capw ? N : capw, 1);
        const uint8_t* xq = static_cast<const uint8_t*>(x);
        if (T == 1 && launch_wide_pair<FmtQ8SoaW, half_t>(as_stream(s), g, xq, K, N, KT, 0u)) return launch_status();
        if (T == 1)
            hipLaunchKernelGGL((gemv_q8_wide_kernel<FmtQ8SoaW, 1, 1, half_t>), gridw, dim3(kGemvThreads), act_tile_bytes(1, KT, FmtQ8SoaW::SUM_GRAN),
                               as_stream(s), g, g, xq, K, N, KT, 1u, 0u);
        else
            hipLaunchKernelGGL((gemv_q8_wide_kernel<FmtQ8SoaW, 2, 1, half_t>), gridw, dim3(kGemvThreads), act_tile_bytes(2, KT, FmtQ8SoaW::SUM_GRAN),
                               as_stream(s), g, g, xq, K, N, KT, 2u, 0u);
        return launch_status();
    }
    if (T <= 4 && q8_soa_interleaved(K)) {   // whole cache lines per load
        GemvSeg<FmtQ8SoaW, half_t> g{{qs_W, d_W, K}, reinterpret_cast<half_t*>(y), nullptr};
        return launch_q8<FmtQ8SoaW, half_t>(s, g, g, 1, x, K, N, T, false, ws);
    }
    GemvSeg<FmtQ8Soa, half_t> g{{qs_W, d_W, K}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ8Soa, half_t>(s, g, g, 1, x, K, N, T, false, ws);
}
int mx_gemv_q8_0_soa_q8_batched(mx_stream_t s, const void* x, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t K,
                                uint32_t N, uint32_t T) {
    return gemv_q8_0_soa_batched(s, x, qs_W, d_W, y, K, N, T, nullptr);
}

// ---- caller-workspace forms of the batched GEMVs: the split-K partial sums go to `ws` instead of the library's
// per-device scratch, so calls on different streams can overlap.  ws_bytes below mx_gemv_batched_ws_bytes(K, N, T)
// is MX_ERR_WORKSPACE; a shape that never splits K (the query returns 0) ignores the workspace.
static int check_ws(const void* ws, uint64_t ws_bytes, uint32_t K, uint32_t N, uint32_t T, SplitWs* out) {
    uint64_t need = 0;
    if (int rc = mx_gemv_batched_ws_bytes(K, N, T, &need)) return rc;
    if (need) {
        MX_REQUIRE_PTR(ws);
        MX_REQUIRE_ALIGN(ws, 16);
        if (ws_bytes < need) return MX_ERR_WORKSPACE;
    }
    *out = SplitWs{static_cast<float*>(const_cast<void*>(ws)), ws_bytes / 4, true};
    return MX_OK;
}
int mx_gemv_batched_ws_bytes(uint32_t K, uint32_t N, uint32_t T, uint64_t* bytes) {
    MX_REQUIRE_PTR(bytes);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && T >= 1 && T <= 16);
    // The query carries no weight format, and which kernel a batch runs on depends on the format (launch_q8: the
    // matrix-core kernel from T = 4 or 5 for most formats, from T = 9 for GGUF Q8_0 blocks), so the answer covers both
    // routes: the vector kernels (batches up to 8) split K >= 8192 over up to kSplitMaxSlices slices, the matrix-core
    // kernel takes the K ranges its row blocks leave room for; T x N partial sums per slice either way.
    uint32_t Z = 1;
    if (T >= 2 && T <= 8 && K >= 8192) Z = kSplitMaxSlices;
    if (T >= 4) {
        const uint32_t zm = T <= 8 ? mmq_dense_ranges(K, N, 1, 4) : mmq_dense_ranges(K, N, 2, 2);
        if (zm > Z) Z = zm;
    }
    *bytes = Z > 1 ? (uint64_t)Z * T * N * sizeof(float) : 0;
    return MX_OK;
}
int mx_gemv_q8_0_soa_q8_batched_ws(mx_stream_t s, const void* x, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t K, uint32_t N,
                                   uint32_t T, void* ws, uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = check_ws(ws, ws_bytes, K, N, T, &w)) return rc;
    return gemv_q8_0_soa_batched(s, x, qs_W, d_W, y, K, N, T, &w);
}
static int gemv_aos_batched_ws(int fmt, mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T, void* ws,
                               uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = check_ws(ws, ws_bytes, K, N, T, &w)) return rc;
    return gemv_aos_q8<half_t>(fmt, s, x, W, reinterpret_cast<half_t*>(y), K, N, T, false, &w);
}
int mx_gemv_q4_K_q8_batched_ws(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T, void* ws, uint64_t ws_bytes) {
    return gemv_aos_batched_ws(1, s, x, W, y, K, N, T, ws, ws_bytes);
}
int mx_gemv_q6_K_q8_batched_ws(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T, void* ws, uint64_t ws_bytes) {
    return gemv_aos_batched_ws(2, s, x, W, y, K, N, T, ws, ws_bytes);
}
int mx_gemv_q8_0_q8_batched_ws(mx_stream_t s, const void* x, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T, void* ws, uint64_t ws_bytes) {
    return gemv_aos_batched_ws(0, s, x, W, y, K, N, T, ws, ws_bytes);
}
int mx_gemv_q8_0_soa_q8(mx_stream_t s, const void* x, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t K, uint32_t N) {
    return mx_gemv_q8_0_soa_q8_batched(s, x, qs_W, d_W, y, K, N, 1);
}

// Repacked K-quant layouts (same dots and fold as the AoS kernels; only the loads differ).
int mx_gemv_q4_K_reorder_q8(mx_stream_t s, const void* x_q8, const void* W_reorder, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(x_q8, y, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W_reorder);
    MX_REQUIRE_ALIGN(x_q8, 8);
    MX_REQUIRE_ALIGN(W_reorder, 16);
    GemvSeg<FmtQ4KStr, half_t> g{FmtQ4KStr::view(static_cast<const uint8_t*>(W_reorder), (uint64_t)N * (K / 256), K / 256), reinterpret_cast<half_t*>(y),
                                 nullptr};
    return launch_q8<FmtQ4KStr, half_t>(s, g, g, 1, x_q8, K, N, 1);
}
int mx_gemv_q4_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q4_q, const int8_t* q4_sc, const int8_t* q4_mn, const uint16_t* q4_d,
                      const uint16_t* q4_dmin, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(x_q8, y, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(q4_q); MX_REQUIRE_PTR(q4_sc); MX_REQUIRE_PTR(q4_mn); MX_REQUIRE_PTR(q4_d); MX_REQUIRE_PTR(q4_dmin);
    MX_REQUIRE_ALIGN(x_q8, 8);
    MX_REQUIRE_ALIGN(q4_q, 16); MX_REQUIRE_ALIGN(q4_sc, 2); MX_REQUIRE_ALIGN(q4_mn, 2);
    GemvSeg<FmtQ4KNat, half_t> g{{q4_q, q4_sc, q4_mn, q4_d, q4_dmin, K}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ4KNat, half_t>(s, g, g, 1, x_q8, K, N, 1);
}
int mx_gemv_q6_soa_q8_batched(mx_stream_t s, const void* x_q8, const uint8_t* q6_lo, const uint8_t* q6_hi, const int8_t* q6_sc,
                              const uint16_t* q6_d, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    if (int rc = check_common(x_q8, y, K, N, T, 256)) return rc;
    MX_REQUIRE_PTR(q6_lo); MX_REQUIRE_PTR(q6_hi); MX_REQUIRE_PTR(q6_sc); MX_REQUIRE_PTR(q6_d);
    MX_REQUIRE_ALIGN(x_q8, 8);
    MX_REQUIRE_ALIGN(q6_lo, 16); MX_REQUIRE_ALIGN(q6_hi, 16); MX_REQUIRE_ALIGN(q6_sc, 4);
    if (T == 1) {   // one token: the plane kernel of gemv_q6_planes.hip where the shape allows
        const int rc = launch_gemv_q6_planes(as_stream(s), 1, x_q8, &q6_lo, &q6_hi, &q6_sc, &q6_d, &y, K, N);
        if (rc != MX_ERR_UNSUPPORTED) return rc;
    }
    GemvSeg<FmtQ6KNat, half_t> g{{q6_lo, q6_hi, q6_sc, q6_d, K}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ6KNat, half_t>(s, g, g, 1, x_q8, K, N, T);
}
// Two plane sets (gate and up) against one q8 row in one launch, as mx_gemv_q6_K_q8_x2 does for GGUF blocks.
int mx_gemv_q6_soa_q8_x2(mx_stream_t s, const void* x_q8, const uint8_t* a_lo, const uint8_t* a_hi, const int8_t* a_sc, const uint16_t* a_d,
                         const uint8_t* b_lo, const uint8_t* b_hi, const int8_t* b_sc, const uint16_t* b_d, uint16_t* y_a, uint16_t* y_b, uint32_t K,
                         uint32_t N) {
    if (int rc = check_common(x_q8, y_a, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(y_b); MX_REQUIRE_PTR(a_lo); MX_REQUIRE_PTR(a_hi); MX_REQUIRE_PTR(a_sc); MX_REQUIRE_PTR(a_d);
    MX_REQUIRE_PTR(b_lo); MX_REQUIRE_PTR(b_hi); MX_REQUIRE_PTR(b_sc); MX_REQUIRE_PTR(b_d);
    MX_REQUIRE_ALIGN(x_q8, 8);
    MX_REQUIRE_ALIGN(a_lo, 16); MX_REQUIRE_ALIGN(a_hi, 16); MX_REQUIRE_ALIGN(a_sc, 4); MX_REQUIRE_ALIGN(b_lo, 16); MX_REQUIRE_ALIGN(b_hi, 16); MX_REQUIRE_ALIGN(b_sc, 4);
    const uint8_t* lo[2] = {a_lo, b_lo};
    const uint8_t* hi[2] = {a_hi, b_hi};
    const int8_t* sc[2] = {a_sc, b_sc};
    const uint16_t* d[2] = {a_d, b_d};
    uint16_t* y[2] = {y_a, y_b};
    const int rc = launch_gemv_q6_planes(as_stream(s), 2, x_q8, lo, hi, sc, d, y, K, N);
    if (rc != MX_ERR_UNSUPPORTED) return rc;
    GemvSeg<FmtQ6KNat, half_t> ga{{a_lo, a_hi, a_sc, a_d, K}, reinterpret_cast<half_t*>(y_a), nullptr}, gb{{b_lo, b_hi, b_sc, b_d, K}, reinterpret_cast<half_t*>(y_b), nullptr};
    return launch_q8<FmtQ6KNat, half_t>(s, ga, gb, 2, x_q8, K, N, 1);
}
int mx_gemv_q6_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q6_lo, const uint8_t* q6_hi, const int8_t* q6_sc, const uint16_t* q6_d,
                      uint16_t* y, uint32_t K, uint32_t N) {
    return mx_gemv_q6_soa_q8_batched(s, x_q8, q6_lo, q6_hi, q6_sc, q6_d, y, K, N, 1);
}

// ---------------------------------------------------------------- Q4_0 (Gemma-4 QAT) and Q5_K
int mx_gemv_q4_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y, K, N, 1, 32)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(W, 2);
    return launch_fact<FmtQ40Aos>(s, FmtQ40Aos::W{static_cast<const uint8_t*>(W), K / 32 * 18u}, reinterpret_cast<const half_t*>(A),
                                  reinterpret_cast<half_t*>(y), K, N);
}
int mx_gemv_q4_0_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    if (int rc = check_common(x_q8, y, K, N, T, 32)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(x_q8, 8); MX_REQUIRE_ALIGN(W, 2);
    GemvSeg<FmtQ40Aos, half_t> g{{static_cast<const uint8_t*>(W), K / 32 * 18u}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ40Aos, half_t>(s, g, g, 1, x_q8, K, N, T);
}
int mx_gemv_q4_0_soa_q8_batched(mx_stream_t s, const void* x_q8, const uint8_t* q4_qs, const uint16_t* q4_d, uint16_t* y, uint32_t K, uint32_t N,
                                uint32_t T) {
    if (int rc = check_common(x_q8, y, K, N, T, 32)) return rc;
    MX_REQUIRE_PTR(q4_qs); MX_REQUIRE_PTR(q4_d);
    MX_REQUIRE_ALIGN(x_q8, 8); MX_REQUIRE_ALIGN(q4_qs, 16); MX_REQUIRE_ALIGN(q4_d, 2);
    GemvSeg<FmtQ40Soa, half_t> g{{q4_qs, q4_d, K}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ40Soa, half_t>(s, g, g, 1, x_q8, K, N, T);
}
int mx_gemv_q4_0_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q4_qs, const uint16_t* q4_d, uint16_t* y, uint32_t K, uint32_t N) {
    return mx_gemv_q4_0_soa_q8_batched(s, x_q8, q4_qs, q4_d, y, K, N, 1);
}
int mx_gemv_q4_0_soa_q8_multi(mx_stream_t s, const void* x_q8, const uint8_t* const* qs, const uint16_t* const* d, uint16_t* const* y,
                              const uint32_t* N, int n_banks, uint32_t K) {
    MX_REQUIRE_PTR(x_q8); MX_REQUIRE_PTR(qs); MX_REQUIRE_PTR(d); MX_REQUIRE_PTR(y); MX_REQUIRE_PTR(N);
    MX_REQUIRE_SHAPE(n_banks >= 1 && n_banks <= 3 && K > 0 && K % 32 == 0);
    MX_REQUIRE_ALIGN(x_q8, 8);
    const uint32_t G = pick_group((K + 63) / 64);
    const uint32_t rows_per_wg = kGemvWaves * (64 / G);
    GemvBanks<FmtQ40Soa> bk{};
    uint32_t total = 0;
    for (int b = 0; b < 3; ++b) {
        const int src = b < n_banks ? b : n_banks - 1;
        if (b < n_banks) {
            MX_REQUIRE_PTR(qs[b]); MX_REQUIRE_PTR(d[b]); MX_REQUIRE_PTR(y[b]);
            MX_REQUIRE_SHAPE(N[b] > 0);
            MX_REQUIRE_ALIGN(qs[b], 16); MX_REQUIRE_ALIGN(d[b], 2);
            total += (N[b] + rows_per_wg - 1) / rows_per_wg;
        }
        bk.w[b] = {qs[src], d[src], K};
        bk.y[b] = reinterpret_cast<half_t*>(y[src]);
        bk.n[b] = N[src];
        bk.rg_end[b] = total;
    }
    const uint32_t per_elem_x32 = 32 + hdr_bytes_per32(FmtQ40Soa::SUM_GRAN);
    const uint32_t KT_max = (kLdsBudget / per_elem_x32) * 32 / 256 * 256;
    const uint32_t K256 = (K + 255) / 256, n_tiles = (K256 * 256 + KT_max - 1) / KT_max;
    const uint32_t KT = (K256 + n_tiles - 1) / n_tiles * 256;
    const uint32_t cap = (uint32_t)cu_count() * kWgsPerCu;
    const dim3 grid(total < cap ? total : cap);
    const uint32_t lds = act_tile_bytes(1, KT, FmtQ40Soa::SUM_GRAN);
    const uint8_t* x = static_cast<const uint8_t*>(x_q8);
    if (G == 16) hipLaunchKernelGGL((gemv_q8_multi_kernel<FmtQ40Soa, 16>), grid, dim3(kGemvThreads), lds, as_stream(s), bk, x, K, KT, n_banks);
    else if (G == 32) hipLaunchKernelGGL((gemv_q8_multi_kernel<FmtQ40Soa, 32>), grid, dim3(kGemvThreads), lds, as_stream(s), bk, x, K, KT, n_banks);
    else hipLaunchKernelGGL((gemv_q8_multi_kernel<FmtQ40Soa, 64>), grid, dim3(kGemvThreads), lds, as_stream(s), bk, x, K, KT, n_banks);
    return launch_status();
}
int mx_gemv_q5_K_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T) {
    if (int rc = check_common(x_q8, y, K, N, T, 256)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(x_q8, 8); MX_REQUIRE_ALIGN(W, 16);
    GemvSeg<FmtQ5K, half_t> g{{static_cast<const uint8_t*>(W), K / 256 * 176u}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtQ5K, half_t>(s, g, g, 1, x_q8, K, N, T);
}
int mx_gemv_q5_K_q8(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return mx_gemv_q5_K_q8_batched(s, x_q8, W, y, K, N, 1);
}
int mx_gemv_q5_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_ALIGN(W, 16);
    return launch_fact<FmtQ5K>(s, FmtQ5K::W{static_cast<const uint8_t*>(W), K / 256 * 176u}, reinterpret_cast<const half_t*>(A),
                               reinterpret_cast<half_t*>(y), K, N);
}

int mx_gemv_mxfp4_soa_q8_batched(mx_stream_t s, const void* x, const uint8_t* qs, const uint8_t* e, uint16_t* y, uint32_t K, uint32_t N,
                                 uint32_t T) {
    if (int rc = check_common(x, y, K, N, T, 32)) return rc;
    MX_REQUIRE_PTR(qs);
    MX_REQUIRE_PTR(e);
    MX_REQUIRE_ALIGN(x, 8);
    MX_REQUIRE_ALIGN(qs, 16);
    GemvSeg<FmtMxfp4Soa, half_t> g{{qs, e, K}, reinterpret_cast<half_t*>(y), nullptr};
    return launch_q8<FmtMxfp4Soa, half_t>(s, g, g, 1, x, K, N, T);
}
int mx_gemv_mxfp4_soa_q8(mx_stream_t s, const void* x, const uint8_t* qs, const uint8_t* e, uint16_t* y, uint32_t K, uint32_t N) {
    return mx_gemv_mxfp4_soa_q8_batched(s, x, qs, e, y, K, N, 1);
}
int mx_gemv_mxfp4_soa_q8_x2(mx_stream_t s, const void* x, const uint8_t* gate_qs, const uint8_t* gate_e, const uint8_t* up_qs,
                            const uint8_t* up_e, const float* gate_bias, const float* up_bias, uint16_t* gate_y, uint16_t* up_y,
                            uint32_t K, uint32_t N) {
    if (int rc = check_common(x, gate_y, K, N, 1, 32)) return rc;
    MX_REQUIRE_PTR(up_y);
    MX_REQUIRE_PTR(gate_qs);
    MX_REQUIRE_PTR(gate_e);
    MX_REQUIRE_PTR(up_qs);
    MX_REQUIRE_PTR(up_e);
    MX_REQUIRE_ALIGN(x, 8);
    MX_REQUIRE_ALIGN(gate_qs, 16);
    MX_REQUIRE_ALIGN(up_qs, 16);
    GemvSeg<FmtMxfp4Soa, half_t> g{{gate_qs, gate_e, K}, reinterpret_cast<half_t*>(gate_y), gate_bias};
    GemvSeg<FmtMxfp4Soa, half_t> u{{up_qs, up_e, K}, reinterpret_cast<half_t*>(up_y), up_bias};
    return launch_q8<FmtMxfp4Soa, half_t>(s, g, u, 2, x, K, N, 1);
}

int mx_gemv_q8_0_soa_q8_x2(mx_stream_t s, const void* x_q8, const int8_t* a_qs, const uint16_t* a_d, const int8_t* b_qs, const uint16_t* b_d,
                           uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    if (int rc = check_common(x_q8, y_a, K, N, 1, 32)) return rc;
    MX_REQUIRE_PTR(y_b); MX_REQUIRE_PTR(a_qs); MX_REQUIRE_PTR(a_d); MX_REQUIRE_PTR(b_qs); MX_REQUIRE_PTR(b_d);
    MX_REQUIRE_ALIGN(x_q8, 8); MX_REQUIRE_ALIGN(a_qs, 16); MX_REQUIRE_ALIGN(b_qs, 16); MX_REQUIRE_ALIGN(a_d, 2); MX_REQUIRE_ALIGN(b_d, 2);
    if (q8_soa_interleaved(K)) return gemv_x2<FmtQ8SoaW>(s, x_q8, {a_qs, a_d, K}, {b_qs, b_d, K}, y_a, y_b, K, N);
    return gemv_x2<FmtQ8Soa>(s, x_q8, {a_qs, a_d, K}, {b_qs, b_d, K}, y_a, y_b, K, N);
}
static int gemv_aos_x2(int fmt, mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    if (int rc = check_common(x_q8, y_a, K, N, 1, fmt == 0 ? 32 : 256)) return rc;
    MX_REQUIRE_PTR(y_b); MX_REQUIRE_PTR(W_a); MX_REQUIRE_PTR(W_b);
    MX_REQUIRE_ALIGN(x_q8, 8); MX_REQUIRE_ALIGN(W_a, fmt == 1 ? 16 : 2); MX_REQUIRE_ALIGN(W_b, fmt == 1 ? 16 : 2);
    const uint8_t *a = static_cast<const uint8_t*>(W_a), *b = static_cast<const uint8_t*>(W_b);
    if (fmt == 1) return gemv_x2<FmtQ4K>(s, x_q8, {a, K / 256 * (uint32_t)kQ4KBytes}, {b, K / 256 * (uint32_t)kQ4KBytes}, y_a, y_b, K, N);
    if (fmt == 2) return gemv_x2<FmtQ6K>(s, x_q8, {a, K / 256 * (uint32_t)kQ6KBytes}, {b, K / 256 * (uint32_t)kQ6KBytes}, y_a, y_b, K, N);
    return gemv_x2<FmtQ8Aos>(s, x_q8, {a, K / 32 * (uint32_t)kQ8_0Bytes}, {b, K / 32 * (uint32_t)kQ8_0Bytes}, y_a, y_b, K, N);
}
int mx_gemv_q4_K_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    return gemv_aos_x2(1, s, x_q8, W_a, W_b, y_a, y_b, K, N);
}
int mx_gemv_q6_K_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    return gemv_aos_x2(2, s, x_q8, W_a, W_b, y_a, y_b, K, N);
}
int mx_gemv_q8_0_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    return gemv_aos_x2(0, s, x_q8, W_a, W_b, y_a, y_b, K, N);
}

int mx_gemv_q4_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(1, s, reinterpret_cast<const half_t*>(A), W, reinterpret_cast<half_t*>(y), K, N);
}
int mx_gemv_q4_K_dual(mx_stream_t s, const uint16_t* A, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y_a, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W_a); MX_REQUIRE_PTR(W_b); MX_REQUIRE_PTR(y_b);
    MX_REQUIRE_ALIGN(W_a, 16); MX_REQUIRE_ALIGN(W_b, 16);
    const uint32_t rb = K / 256 * (uint32_t)kQ4KBytes;
    const FmtQ4K::W wa{static_cast<const uint8_t*>(W_a), rb}, wb{static_cast<const uint8_t*>(W_b), rb};
    return launch_fact<FmtQ4K>(s, wa, reinterpret_cast<const half_t*>(A), reinterpret_cast<half_t*>(y_a), K, N, &wb, reinterpret_cast<half_t*>(y_b));
}
int mx_gemv_q4_K_down_accum(mx_stream_t s, const uint16_t* A, const void* W, const uint16_t* sh_g, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W); MX_REQUIRE_PTR(sh_g);
    MX_REQUIRE_ALIGN(W, 16);
    const FmtQ4K::W w{static_cast<const uint8_t*>(W), K / 256 * (uint32_t)kQ4KBytes};
    return launch_fact<FmtQ4K, half_t, half_t>(s, w, reinterpret_cast<const half_t*>(A), reinterpret_cast<half_t*>(y), K, N, nullptr, nullptr,
                                               reinterpret_cast<const half_t*>(sh_g));
}
int mx_gemv_q4_K_shexp_gate_up(mx_stream_t s, const uint16_t* A, const void* W_gate, const void* W_up, const float* W_shg, uint16_t* y_h,
                               uint16_t* sh_g_out, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y_h, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W_gate); MX_REQUIRE_PTR(W_up); MX_REQUIRE_PTR(W_shg); MX_REQUIRE_PTR(sh_g_out);
    MX_REQUIRE_ALIGN(W_gate, 16); MX_REQUIRE_ALIGN(W_up, 16);
    const uint32_t rb = K / 256 * (uint32_t)kQ4KBytes;
    const FmtQ4K::W wg{static_cast<const uint8_t*>(W_gate), rb}, wu{static_cast<const uint8_t*>(W_up), rb};
    return launch_fact<FmtQ4K, half_t, half_t, FACT_SILU_PAIR>(s, wg, reinterpret_cast<const half_t*>(A), reinterpret_cast<half_t*>(y_h), K, N, &wu,
                                                               nullptr, nullptr, FactTail{W_shg, nullptr, sh_g_out, nullptr});
}
int mx_gemv_q4_K_dual_ssm_gbeta(mx_stream_t s, const uint16_t* A, const void* W_alpha, const void* W_beta, const float* A_log,
                                const float* dt_bias, float* g_out, float* beta_out, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, g_out, K, N, 1, 256)) return rc;
    MX_REQUIRE_PTR(W_alpha); MX_REQUIRE_PTR(W_beta); MX_REQUIRE_PTR(A_log); MX_REQUIRE_PTR(dt_bias); MX_REQUIRE_PTR(beta_out);
    MX_REQUIRE_ALIGN(W_alpha, 16); MX_REQUIRE_ALIGN(W_beta, 16);
    const uint32_t rb = K / 256 * (uint32_t)kQ4KBytes;
    const FmtQ4K::W wa{static_cast<const uint8_t*>(W_alpha), rb}, wb{static_cast<const uint8_t*>(W_beta), rb};
    return launch_fact<FmtQ4K, half_t, half_t, FACT_GBETA>(s, wa, reinterpret_cast<const half_t*>(A), static_cast<half_t*>(nullptr), K, N, &wb,
                                                           nullptr, nullptr, FactTail{A_log, dt_bias, g_out, beta_out});
}
int mx_gemv_q6_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(2, s, reinterpret_cast<const half_t*>(A), W, reinterpret_cast<half_t*>(y), K, N);
}
int mx_gemv_q8_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(0, s, reinterpret_cast<const half_t*>(A), W, reinterpret_cast<half_t*>(y), K, N);
}
int mx_gemv_q4_K_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(1, s, A, W, y, K, N);
}
int mx_gemv_q6_K_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(2, s, A, W, y, K, N);
}
int mx_gemv_q8_0_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N) {
    return gemv_aos_fact(0, s, A, W, y, K, N);
}
int mx_gemv_mxfp4_soa_f16(mx_stream_t s, const uint16_t* A, const uint8_t* qs, const uint8_t* e, uint16_t* y, uint32_t K, uint32_t N) {
    if (int rc = check_common(A, y, K, N, 1, 32)) return rc;
    MX_REQUIRE_PTR(qs);
    MX_REQUIRE_PTR(e);
    MX_REQUIRE_ALIGN(qs, 16);
    return launch_fact<FmtMxfp4Soa>(s, FmtMxfp4Soa::W{qs, e, K}, reinterpret_cast<const half_t*>(A), reinterpret_cast<half_t*>(y), K, N);
}

// ---- decode FFN forms: fused gate + up + SwiGLU, and GEMVs that take the fp16 activation row
int mx_gemv_q8_0_soa_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                             const uint16_t* u_d, uint16_t* h, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(g_qs); MX_REQUIRE_PTR(g_d); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_d);
    MX_REQUIRE_ALIGN(g_qs, 16); MX_REQUIRE_ALIGN(u_qs, 16); MX_REQUIRE_ALIGN(g_d, 2); MX_REQUIRE_ALIGN(u_d, 2);
    if (q8_soa_interleaved(K)) return launch_ffn_x<FmtQ8SoaW, 2>(s, {g_qs, g_d, K}, {u_qs, u_d, K}, x, x_is_f16, h, K, N);
    return launch_ffn_x<FmtQ8Soa, 2>(s, {g_qs, g_d, K}, {u_qs, u_d, K}, x, x_is_f16, h, K, N);
}
static int ffn_aos(int fmt, int nw, mx_stream_t s, const void* x, int x_is_f16, const void* W0, const void* W1, uint16_t* y, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(W0); MX_REQUIRE_PTR(W1);
    MX_REQUIRE_SHAPE(K % (fmt == 0 ? 32u : 256u) == 0);
    MX_REQUIRE_ALIGN(W0, fmt == 1 ? 16 : 2); MX_REQUIRE_ALIGN(W1, fmt == 1 ? 16 : 2);
    const uint8_t *a = static_cast<const uint8_t*>(W0), *b = static_cast<const uint8_t*>(W1);
    if (fmt == 1) {
        const FmtQ4K::W wa{a, K / 256 * (uint32_t)kQ4KBytes}, wb{b, K / 256 * (uint32_t)kQ4KBytes};
        // the single GEMV on a long row of a short matrix: the paired-row walk, as mx_gemv_q4_K_q8 takes it (launch_q8_tg)
        const uint32_t KT4 = (K + 255) / 256 * 256;
        if (nw == 1 && x_is_f16 && K >= 8192 && act_tile_bytes(1, KT4, FmtQ4K::SUM_GRAN) <= kLdsBudget &&
            (N + kGemvWaves * (64 / pick_group(K / 64)) - 1) / (kGemvWaves * (64 / pick_group(K / 64))) <= 2u * (uint32_t)cu_count()) {
            if (int rc = check_common(x, y, K, N, 1, 256)) return rc;
            MX_REQUIRE_ALIGN(x, 16);
            GemvSeg<FmtQ4K, half_t> g{wa, reinterpret_cast<half_t*>(y), nullptr};
            if (launch_wide_pair<FmtQ4K, half_t>(as_stream(s), g, static_cast<const uint8_t*>(x), K, N, KT4, 2u)) return launch_status();
        }
        return nw == 2 ? launch_ffn_x<FmtQ4K, 2>(s, wa, wb, x, x_is_f16, y, K, N) : launch_ffn_x<FmtQ4K, 1>(s, wa, wb, x, x_is_f16, y, K, N);
    }
    if (fmt == 2) {
        const FmtQ6K::W wa{a, K / 256 * (uint32_t)kQ6KBytes}, wb{b, K / 256 * (uint32_t)kQ6KBytes};
        // the single GEMV on a long row of a short matrix: the workgroup-wide walk, as mx_gemv_q6_K_q8 takes it
        // (launch_q8_tg: one K tile, K >= 8192, at most two row groups of eight rows per CU)
        const uint32_t KT = (K + 255) / 256 * 256;
        if (nw == 1 && x_is_f16 && K >= 8192 && act_tile_bytes(1, KT, FmtQ6K::SUM_GRAN) <= kLdsBudget &&
            (N + kGemvWaves * (64 / pick_group(K / 64)) - 1) / (kGemvWaves * (64 / pick_group(K / 64))) <= 2u * (uint32_t)cu_count()) {
            if (int rc = check_common(x, y, K, N, 1, 256)) return rc;
            MX_REQUIRE_ALIGN(x, 16);
            GemvSeg<FmtQ6K, half_t> g{wa, reinterpret_cast<half_t*>(y), nullptr};
            if (launch_wide_pair<FmtQ6K, half_t>(as_stream(s), g, static_cast<const uint8_t*>(x), K, N, KT, 2u)) return launch_status();
            const uint32_t capw = (uint32_t)cu_count() * kWideF16WgsPerCu;
            hipLaunchKernelGGL((gemv_q8_wide_kernel<FmtQ6K, 1, 1, half_t>), dim3(N < capw ? N : capw, 1), dim3(kGemvThreads),
                               act_tile_bytes(1, KT, FmtQ6K::SUM_GRAN), as_stream(s), g, g, static_cast<const uint8_t*>(x), K, N, KT, 1u, 2u);
            return launch_status();
        }
        return nw == 2 ? launch_ffn_x<FmtQ6K, 2>(s, wa, wb, x, x_is_f16, y, K, N) : launch_ffn_x<FmtQ6K, 1>(s, wa, wb, x, x_is_f16, y, K, N);
    }
    const FmtQ8Aos::W wa{a, K / 32 * (uint32_t)kQ8_0Bytes}, wb{b, K / 32 * (uint32_t)kQ8_0Bytes};
    {   // the single GEMV on a long row of a short matrix: the paired-row walk, as mx_gemv_q8_0_q8 takes it (launch_q8_tg)
        const uint32_t KT8 = (K + 255) / 256 * 256;
        if (nw == 1 && x_is_f16 && K >= 8192 && act_tile_bytes(1, KT8, FmtQ8Aos::SUM_GRAN) <= kLdsBudget &&
            (N + kGemvWaves * (64 / pick_group((K + 63) / 64)) - 1) / (kGemvWaves * (64 / pick_group((K + 63) / 64))) <= 2u * (uint32_t)cu_count()) {
            if (int rc = check_common(x, y, K, N, 1, 32)) return rc;
            MX_REQUIRE_ALIGN(x, 16);
            GemvSeg<FmtQ8Aos, half_t> g{wa, reinterpret_cast<half_t*>(y), nullptr};
            if (launch_wide_pair<FmtQ8Aos, half_t>(as_stream(s), g, static_cast<const uint8_t*>(x), K, N, KT8, 2u)) return launch_status();
        }
    }
    return nw == 2 ? launch_ffn_x<FmtQ8Aos, 2>(s, wa, wb, x, x_is_f16, y, K, N) : launch_ffn_x<FmtQ8Aos, 1>(s, wa, wb, x, x_is_f16, y, K, N);
}
int mx_gemv_q4_K_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h, uint32_t K, uint32_t N) {
    return ffn_aos(1, 2, s, x, x_is_f16, gate_W, up_W, h, K, N);
}
int mx_gemv_q6_K_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h, uint32_t K, uint32_t N) {
    return ffn_aos(2, 2, s, x, x_is_f16, gate_W, up_W, h, K, N);
}
int mx_gemv_q8_0_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h, uint32_t K, uint32_t N) {
    return ffn_aos(0, 2, s, x, x_is_f16, gate_W, up_W, h, K, N);
}
int mx_gemv_q8_0_soa_f16q8(mx_stream_t s, const uint16_t* x_f16, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(qs_W); MX_REQUIRE_PTR(d_W);
    MX_REQUIRE_ALIGN(qs_W, 16); MX_REQUIRE_ALIGN(d_W, 2);
    const FmtQ8Soa::W w{qs_W, d_W, K};
    if (q8_soa_wide(K, N)) {   // the same launch as mx_gemv_q8_0_soa_q8 takes for this shape, the row quantized while it is staged
        if (int rc = check_common(x_f16, y, K, N, 1, 32)) return rc;
        MX_REQUIRE_ALIGN(x_f16, 16);
        GemvSeg<FmtQ8SoaW, half_t> g{{qs_W, d_W, K}, reinterpret_cast<half_t*>(y), nullptr};
        const uint32_t KT = (K + 255) / 256 * 256, capw = (uint32_t)cu_count() * kWideF16WgsPerCu;
        if (launch_wide_pair<FmtQ8SoaW, half_t>(as_stream(s), g, reinterpret_cast<const uint8_t*>(x_f16), K, N, KT, 2u)) return launch_status();
        hipLaunchKernelGGL((gemv_q8_wide_kernel<FmtQ8SoaW, 1, 1, half_t>), dim3(N < capw ? N : capw, 1), dim3(kGemvThreads),
                           act_tile_bytes(1, KT, FmtQ8SoaW::SUM_GRAN), as_stream(s), g, g, reinterpret_cast<const uint8_t*>(x_f16), K, N, KT, 1u, 2u);
        return launch_status();
    }
    if (q8_soa_interleaved(K)) return launch_ffn_x<FmtQ8SoaW, 1>(s, w, w, x_f16, 1, y, K, N);
    return launch_ffn_x<FmtQ8Soa, 1>(s, w, w, x_f16, 1, y, K, N);
}
int mx_gemv_q4_K_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return ffn_aos(1, 1, s, x_f16, 1, W, W, y, K, N);
}
int mx_gemv_q6_K_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return ffn_aos(2, 1, s, x_f16, 1, W, W, y, K, N);
}
int mx_gemv_q8_0_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N) {
    return ffn_aos(0, 1, s, x_f16, 1, W, W, y, K, N);
}

int mx_probe_stream_read(mx_stream_t s, const void* src, uint64_t n_bytes, uint32_t* sink) {
    MX_REQUIRE_PTR(src);
    MX_REQUIRE_SHAPE(n_bytes >= 16 && n_bytes % 16 == 0);
    MX_REQUIRE_ALIGN(src, 16);
    const uint64_t n16 = n_bytes / 16, chunks = (n16 + kGemvThreads * 4u - 1) / (kGemvThreads * 4u);
    const uint32_t cap = (uint32_t)cu_count() * kWgsPerCu;
    hipLaunchKernelGGL(stream_read_kernel, dim3((uint32_t)(chunks < cap ? chunks : cap)), dim3(kGemvThreads), 0, as_stream(s),
                       static_cast<const uint4*>(src), n16, sink);
    return launch_status();
}

}  // extern "C"
