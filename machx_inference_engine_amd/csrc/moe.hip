// moe.hip — expert-indexed GEMV kernels (MoE decode and small-batch grouped
// decode) and the row utilities around them.
//
// One kernel serves both addressing modes of the reference:
//   * decode   — blockIdx.y = token slot tk = t*K_top + k; the expert id is read
//                from the device array topk_idx[tk] (include/ie/moe_q8.hpp:17-33,
//                src/ops/moe_q8.cpp:45-147): no host round trip, no per-expert
//                host loop;
//   * grouped  — blockIdx.y = expert e; its activation rows are the expert-sorted
//                rows [expert_offsets[e], expert_offsets[e+1]) (moe_q8.hpp:51-72);
//                the expert's weights are streamed once per tile of up to TT rows,
//                empty experts return at once (src/ops/moe_q8.cpp:211).
// The inner loop is the dense GEMV core (mxq_gemv_core.h).  gate and up rows are
// walked together against one staged activation and fused with the activation
// function in the epilogue.
#include "mxq_gemv_core.h"
#include "mxq_host.h"
#include "mxq_mmq.h"

#include <type_traits>

namespace mxq {

enum { EPI_SILU = 0, EPI_OAI = 1, EPI_DOWN_WEIGHTED = 2, EPI_DOWN_BIAS = 3 };

struct MoeArgs {
    const uint8_t* xq8;              // block_q8_1x rows
    const int32_t* topk_idx;         // decode mode: [n_seg] expert per slot; NULL in grouped mode
    const uint32_t* expert_offsets;  // grouped mode: [E+1]
    const float* bias0;              // [E][N] fp32 or NULL (gate bias / down bias)
    const float* bias1;              // [E][N] fp32 or NULL (up bias)
    const half_t* route_w;           // [rows] fp16 routing weight per output row (EPI_DOWN_WEIGHTED)
    half_t* out;                     // [rows][N]
    float alpha, limit;              // swiglu_oai parameters
    uint32_t act_div;                // activation row of output row r is r / act_div
    uint32_t K, N, KT, n_experts;
    uint32_t q8_split;               // activation rows are block_q8_1s (48 B) instead of block_q8_1x
    uint32_t n_rows;                 // dense mode (no topk_idx, no expert_offsets): one weight matrix, rows [0, n_rows)
    const half_t* act_f16;           // when set: activation rows are fp16 [rows][K] and are quantized while they are staged
};

__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.f + __expf(-g))) * u; }
// src/ops/elementwise.cpp:468-492: x = min(gate, limit), z = clamp(up, -limit, limit), (x * sigmoid(alpha x)) * (z + 1)
__device__ __forceinline__ float swiglu_oai(float g, float u, float alpha, float limit) {
    const float x = fminf(g, limit), z = fmaxf(fminf(u, limit), -limit);
    return (x / (1.f + __expf(alpha * -x))) * (z + 1.f);
}

// NW = weight rows per output element (2: gate and up, 1: down); R outputs per lane group.
// One-token down launches of MXFP4 (36-byte units, decoded by the convert instruction) request whole rows ahead (see below) and are
// held to three resident waves per SIMD, which a decode launch of a few hundred workgroups needs to be resident at once.  (gate + up
// the same way spills: 21 against 12 us.)
template <class F, int TT, int NW>
constexpr bool kMoeWholeRow = TT == 1 && NW == 1 && F::SUM_GRAN == 2;
template <class F, int TT, int NW, int R, int G, int U, int EPI>
__global__ __launch_bounds__(kGemvThreads, (TT == 1 && NW == 1 && F::SUM_GRAN == 2) ? 3 : 1) void moe_gemv_kernel(typename F::Bank bank0, typename F::Bank bank1, MoeArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS * R;
    const uint32_t seg = blockIdx.y;
    uint32_t e, r_begin, r_end;
    if (a.topk_idx) {
        e = (uint32_t)a.topk_idx[seg];
        r_begin = seg;
        r_end = seg + 1;
    } else if (a.expert_offsets) {
        e = seg;
        r_begin = a.expert_offsets[seg];
        r_end = a.expert_offsets[seg + 1];
    } else {
        e = 0;
        r_begin = 0;
        r_end = a.n_rows;
    }
    if (r_begin >= r_end || e >= a.n_experts) return;   // empty expert / invalid id: uniform for the block
    const typename F::W w0 = F::expert(bank0, e), w1 = F::expert(NW == 2 ? bank1 : bank0, e);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    const uint32_t K = a.K, N = a.N, KT = a.KT;
    const size_t q8_row_bytes = (size_t)(K / 32) * (a.q8_split ? kQ81sBytes : kQ81xBytes);
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_tiles = (K + KT - 1) / KT;
    for (uint32_t t0 = r_begin; t0 < r_end; t0 += TT) {
        const uint32_t nt = (r_end - t0 < (uint32_t)TT) ? r_end - t0 : (uint32_t)TT;
        auto xrow = [&](uint32_t t) { return a.xq8 + (size_t)((t0 + (t < nt ? t : nt - 1)) / a.act_div) * q8_row_bytes; };
        ActTile act;
        bool staged = false;
        for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x) {
            const uint32_t n0 = rg * ROWS_PER_WG + (wave * GROUPS + grp) * R;
            float acc[NW * R][TT];
#pragma unroll
            for (int r = 0; r < NW * R; ++r)
#pragma unroll
                for (int t = 0; t < TT; ++t) acc[r][t] = 0.f;
            for (uint32_t tile = 0; tile < n_tiles; ++tile) {
                const uint32_t k0 = tile * KT, kt = (K - k0 < KT) ? K - k0 : KT;
                typename F::Cursor cu[NW * R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t n = (n0 + r < N) ? n0 + r : N - 1;
                    cu[NW * r] = F::cursor(w0, n, k0 / 64 + gl);
                    if (NW == 2) cu[NW * r + 1] = F::cursor(w1, n, k0 / 64 + gl);
                }
                const uint32_t n_units = (kt + 63) / 64;
                const bool half_tail = (kt & 63u) != 0;
                if (kMoeWholeRow<F, TT, NW> && n_tiles == 1 && !staged && !half_tail && n_units <= 3u * G) {
                    // A workgroup of a decode launch lives for one row group.  The whole of its rows (up to three rounds
                    // of units) is requested right behind the activation loads and in front of the barrier, so the launch
                    // is one round trip to memory and the first round is summed while the later ones arrive.  Lanes
                    // past the end of the row read their first unit again and drop the product.
                    constexpr int AHEAD = 3;
                    typename F::Raw pre[3][NW * R];
                    auto request = [&]() {
#pragma unroll
                        for (int u = 0; u < AHEAD; ++u) {
                            const bool lv = u * G + gl < n_units;
#pragma unroll
                            for (int r = 0; r < NW * R; ++r) pre[u][r] = load_unit<F, G>(cu[r], lv ? u : 0, false);
                        }
                    };
                    if (a.act_f16) {
                        auto hrow = [&](uint32_t t) { return a.act_f16 + (size_t)((t0 + (t < nt ? t : nt - 1)) / a.act_div) * K; };
                        act = stage_act_f16<F::SUM_GRAN, TT>(lds, hrow, k0, kt, KT, request);
                    } else {
                        act = stage_act<F::SUM_GRAN, TT>(lds, xrow, k0, kt, KT, a.q8_split != 0, request);
                    }
                    __syncthreads();
                    staged = true;
#pragma unroll
                    for (int u = 0; u < 3; ++u) {
                        if (u > 0 && u - 1 + AHEAD < 3) {   // a round that was not requested ahead takes the registers of a summed one
                            const bool lq = (u - 1 + AHEAD) * G + gl < n_units;
#pragma unroll
                            for (int r = 0; r < NW * R; ++r) pre[u - 1 + AHEAD][r] = load_unit<F, G>(cu[r], lq ? u - 1 + AHEAD : 0, false);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        const bool lv = u * G + gl < n_units;
                        float part[NW * R][TT];
#pragma unroll
                        for (int r = 0; r < NW * R; ++r)
#pragma unroll
                            for (int t = 0; t < TT; ++t) part[r][t] = 0.f;
                        gemv_step<F, TT, NW * R>(pre[u], cu, lv ? gl + u * G : gl, act, part);
#pragma unroll
                        for (int r = 0; r < NW * R; ++r)
#pragma unroll
                            for (int t = 0; t < TT; ++t) acc[r][t] += lv ? part[r][t] : 0.f;
                    }
                    continue;
                }
                if (n_tiles > 1 || !staged) {
                    __syncthreads();
                    if (a.act_f16) {
                        auto hrow = [&](uint32_t t) { return a.act_f16 + (size_t)((t0 + (t < nt ? t : nt - 1)) / a.act_div) * K; };
                        act = stage_act_f16<F::SUM_GRAN, TT>(lds, hrow, k0, kt, KT);
                    } else {
                        act = stage_act<F::SUM_GRAN, TT>(lds, xrow, k0, kt, KT, a.q8_split != 0);
                    }
                    __syncthreads();
                    staged = true;
                }
                gemv_rows<F, TT, NW * R, G, U>(cu, n_units, half_tail, gl, act, acc);
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const float v0 = group_sum<G>(acc[NW * r][t]);
                    const float v1 = (NW == 2) ? group_sum<G>(acc[NW * r + 1][t]) : 0.f;
                    const uint32_t n = n0 + r;
                    if (lane == (uint32_t)group_sum_lane<G>(lane) && n < N && (uint32_t)t < nt) {
                        const uint32_t row = t0 + t;
                        float o;
                        if (EPI == EPI_SILU) {
                            o = silu_mul(v0, v1);                                   // src/ops/moe_q8.cpp:94-97
                        } else if (EPI == EPI_OAI) {
                            // rounding points of the reference chain: half(acc + bias) per projection, then the fp16 activation
                            const float g = (float)(half_t)(v0 + (a.bias0 ? a.bias0[(size_t)e * N + n] : 0.f));
                            const float u = (float)(half_t)(v1 + (a.bias1 ? a.bias1[(size_t)e * N + n] : 0.f));
                            o = swiglu_oai(g, u, a.alpha, a.limit);
                        } else if (EPI == EPI_DOWN_WEIGHTED) {
                            o = (float)a.route_w[row] * v0;                        // src/ops/moe_q8.cpp:143-144
                        } else {
                            o = (float)(half_t)v0;                                 // gemv out, then add_bias (elementwise.cpp:782-793)
                            if (a.bias0) o += a.bias0[(size_t)e * N + n];
                        }
                        a.out[(size_t)row * N + n] = (half_t)o;
                    }
                }
        }
    }
}

// ---------------------------------------------------------------- fp16-activation decode (K-quant expert banks)
// The reference's decode kernels for Q4_K / Q6_K experts take fp16 activations and fold in fp32
// (src/ops/moe_fused.cpp:82-211, 224-330, 352-522).  Same unit walk as the float-activation GEMV.
//   FACT_GATE_UP: grid (x, slot tk): h_out[tk, n] = half(silu(gate_e . x_t) * (up_e . x_t)), t = tk / K_top
//   FACT_DOWN   : grid (x, token t): y[t, n] = half(sum_k w[t,k] * (down_e(t,k) . h[t*K_top + k])),
//                 the K_top products summed in fp32 before the single rounding (moe_fused.cpp:268-318);
//                 all K_top activation rows of the token are staged side by side.
enum { FACT_GATE_UP = 0, FACT_DOWN = 1 };

struct MoeFactArgs {
    const half_t* act;          // gate/up: x [T, K]; down: h [T*K_top, K]
    const int32_t* topk_idx;    // [T*K_top]
    const half_t* topk_w;       // down: [T*K_top]
    half_t* out;                // gate/up: [T*K_top, N]; down: [T, N]
    uint32_t K, N, KT, K_top;
};

template <class F, int G, int MODE>
__global__ __launch_bounds__(kGemvThreads) void moe_fact_kernel(typename F::Bank bank0, typename F::Bank bank1, MoeFactArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int GROUPS = 64 / G;
    constexpr int ROWS_PER_WG = kGemvWaves * GROUPS;
    constexpr int NW = (MODE == FACT_GATE_UP) ? 2 : 1;
    const uint32_t K = a.K, N = a.N, KT = a.KT;
    const uint32_t n_act = (MODE == FACT_DOWN) ? a.K_top : 1u;   // activation rows staged together
    float* xa = reinterpret_cast<float*>(lds);                    // [n_act][KT]
    float* s16 = xa + (size_t)n_act * KT;                         // [n_act][KT/16]
    const uint32_t seg = blockIdx.y;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t grp = lane / G, gl = lane % G;
    const uint32_t n_rg = (N + ROWS_PER_WG - 1) / ROWS_PER_WG;
    const uint32_t n_tiles = (K + KT - 1) / KT;
    const half_t* act0 = (MODE == FACT_DOWN) ? a.act + (size_t)seg * a.K_top * K : a.act + (size_t)(seg / a.K_top) * K;
    bool staged = false;
    for (uint32_t rg = blockIdx.x; rg < n_rg; rg += gridDim.x) {
        const uint32_t n0 = rg * ROWS_PER_WG + wave * GROUPS + grp;
        const uint32_t n = n0 < N ? n0 : N - 1;
        float tot0 = 0.f, tot1 = 0.f;
        for (uint32_t tile = 0; tile < n_tiles; ++tile) {
            const uint32_t k0 = tile * KT, kt = (K - k0 < KT) ? K - k0 : KT;
            if (n_tiles > 1 || !staged) {
                __syncthreads();
                for (uint32_t j = 0; j < n_act; ++j) stage_fact(xa + (size_t)j * KT, s16 + (size_t)j * (KT / 16), act0 + (size_t)j * K + k0, kt);
                __syncthreads();
                staged = true;
            }
            const uint32_t n_units = (kt + 63) / 64;
            const bool half_tail = (kt & 63u) != 0;
            for (uint32_t j = 0; j < n_act; ++j) {
                const uint32_t slot = (MODE == FACT_DOWN) ? seg * a.K_top + j : seg;
                const uint32_t e = (uint32_t)a.topk_idx[slot];
                if (e >= 0x80000000u) continue;   // negative id: the slot contributes nothing (uniform for the block); the signature carries no expert count
                const typename F::W w0 = F::expert(bank0, e), w1 = F::expert(NW == 2 ? bank1 : bank0, e);
                typename F::Cursor c0 = F::cursor(w0, n, k0 / 64 + gl), c1 = F::cursor(w1, n, k0 / 64 + gl);
                const float* xj = xa + (size_t)j * KT;
                const float* sj = s16 + (size_t)j * (KT / 16);
                float acc0 = 0.f, acc1 = 0.f;
                for (uint32_t it = 0; it * G + gl < n_units; ++it) {
                    const uint32_t ul = it * G + gl, e0 = F::elem_off(ul);
                    const bool tail = half_tail && ul == n_units - 1;
                    const typename F::Raw r0 = load_unit<F, G>(c0, it, tail);
                    if (NW == 2) {
                        const typename F::Raw r1 = load_unit<F, G>(c1, it, tail);
                        acc1 += fact_unit<F>(r1, c1, xj, sj, e0);
                    }
                    acc0 += fact_unit<F>(r0, c0, xj, sj, e0);
                }
                if (MODE == FACT_DOWN) tot0 += (float)a.topk_w[slot] * acc0;
                else { tot0 += acc0; tot1 += acc1; }
            }
        }
        const float v0 = group_sum<G>(tot0);
        const float v1 = (NW == 2) ? group_sum<G>(tot1) : 0.f;
        if (lane == (uint32_t)group_sum_lane<G>(lane) && n0 < N)
            a.out[(size_t)seg * N + n0] = (half_t)((MODE == FACT_GATE_UP) ? silu_mul(v0, v1) : v0);
    }
}

// ---------------------------------------------------------------- row utilities
// moe_gather_rows (src/ops/moe.cpp:262-282): y_packed[i] = x[indices[i]]
__global__ __launch_bounds__(256) void gather_rows_kernel(const half_t* x, const int32_t* idx, half_t* y, uint32_t n_rows, uint32_t hidden) {
    const uint32_t row = blockIdx.y;
    const uint32_t c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (row >= n_rows || c >= hidden) return;
    const half_t* src = x + (size_t)idx[row] * hidden + c;
    half_t* dst = y + (size_t)row * hidden + c;
    if (c + 8 <= hidden && (hidden & 7u) == 0) {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
    } else {
        for (uint32_t i = 0; i < 8 && c + i < hidden; ++i) dst[i] = src[i];
    }
}

// moe_scatter_add (src/ops/moe.cpp:284-313): y[indices[i]] = half(float(y[indices[i]]) + float(x_packed[i]) * w[i]).
// Plain read-modify-write as in the reference: the rows named by one call must be distinct.
__global__ __launch_bounds__(256) void scatter_add_kernel(const half_t* x, const int32_t* idx, const half_t* w, half_t* y, uint32_t n_rows,
                                                          uint32_t hidden) {
    const uint32_t row = blockIdx.y;
    const uint32_t c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (row >= n_rows || c >= hidden) return;
    const float wr = (float)w[row];
    const half_t* src = x + (size_t)row * hidden + c;
    half_t* dst = y + (size_t)idx[row] * hidden + c;
    if (c + 8 <= hidden && (hidden & 7u) == 0) {
        union { uint4 v; half_t h[8]; } a, b;
        a.v = *reinterpret_cast<const uint4*>(src);
        b.v = *reinterpret_cast<const uint4*>(dst);
#pragma unroll
        for (int i = 0; i < 8; ++i) b.h[i] = (half_t)((float)b.h[i] + (float)a.h[i] * wr);
        *reinterpret_cast<uint4*>(dst) = b.v;
    } else {
        for (uint32_t i = 0; i < 8 && c + i < hidden; ++i) dst[i] = (half_t)((float)dst[i] + (float)src[i] * wr);
    }
}

// moe_prefill_merge_fp32_to_fp16 (src/ops/moe_fused.cpp:1956-1972): y16[i] = half(float(y16[i]) + y32[i])
__global__ __launch_bounds__(256) void merge_f32_kernel(const float* y32, half_t* y16, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y16[i] = (half_t)((float)y16[i] + y32[i]);
}

// moe_reduce_q8 (src/ops/moe_q8.cpp:149-158): y[t] = sum_k y_packed[t*K+k]
// moe_prefill_reduce_sum (:368-384): y[t] = sum_k out_packed[tk_to_packed[t*K+k]]
// moe_prefill_reduce (src/ops/moe_fused.cpp:1927-1954): y[t] += sum_k w[row] * out_packed[row]
template <bool WEIGHTED, bool ACCUMULATE>
__global__ __launch_bounds__(256) void moe_reduce_kernel(const half_t* packed, const uint32_t* tk_to_packed, const half_t* w, half_t* y,
                                                         uint32_t T, uint32_t Ktop, uint32_t H) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (uint64_t)T * H) return;
    const uint32_t t = (uint32_t)(i / H), n = (uint32_t)(i % H);
    float s = ACCUMULATE ? (float)y[i] : 0.f;
    for (uint32_t k = 0; k < Ktop; ++k) {
        const uint32_t row = tk_to_packed ? tk_to_packed[(size_t)t * Ktop + k] : t * Ktop + k;
        const float v = (float)packed[(size_t)row * H + n];
        s += WEIGHTED ? (float)w[row] * v : v;
    }
    y[i] = (half_t)s;
}

// ---------------------------------------------------------------- host side
static int cu_count_moe() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    }
    return n;
}
constexpr uint32_t kMoeLdsBudget = 48 * 1024;
constexpr uint32_t kMoeFactLds = 60 * 1024;   // staged fp32 activations of the fp16-activation decode kernels

static uint32_t pick_group_moe(uint32_t units) {
    uint32_t best = 64, waste = (units + 63) / 64 * 64 - units;
    for (uint32_t g : {32u, 16u}) {
        const uint32_t w = (units + g - 1) / g * g - units;
        if (w < waste) { best = g; waste = w; }
    }
    return best;
}

template <class F, int TT, int NW, int G, int EPI>
static int launch_moe_tg(hipStream_t st, const typename F::Bank& b0, const typename F::Bank& b1, MoeArgs a, uint32_t n_seg) {
    constexpr int R = (NW == 2 || TT == 1) ? 1 : 2;
    constexpr int U = (TT == 1) ? 2 : 1;
    constexpr uint32_t rows_per_wg = kGemvWaves * (64 / G) * R;
    const uint32_t per32 = qs_bytes_per32(F::SUM_GRAN) + hdr_bytes_per32(F::SUM_GRAN);
    const uint32_t KT_max = (kMoeLdsBudget / (per32 * TT)) * 32 / 256 * 256;
    if (KT_max == 0) return MX_ERR_SHAPE;
    const uint32_t K256 = (a.K + 255) / 256, n_tiles = (K256 * 256 + KT_max - 1) / KT_max;
    a.KT = (K256 + n_tiles - 1) / n_tiles * 256;
    const uint32_t n_rg = (a.N + rows_per_wg - 1) / rows_per_wg;
    uint32_t gx = (uint32_t)cu_count_moe() * 8 / (n_seg ? n_seg : 1);
    if (gx < 1) gx = 1;
    if (gx > n_rg) gx = n_rg;
    if (n_seg > 65535) return MX_ERR_SHAPE;
    hipLaunchKernelGGL((moe_gemv_kernel<F, TT, NW, R, G, U, EPI>), dim3(gx, n_seg), dim3(kGemvThreads), act_tile_bytes(TT, a.KT, F::SUM_GRAN), st,
                       b0, b1, a);
    return launch_status();
}

template <class F, int NW, int EPI>
static int launch_moe(mx_stream_t s, const typename F::Bank& b0, const typename F::Bank& b1, const MoeArgs& a, uint32_t n_seg, uint32_t tt) {
    const uint32_t G = pick_group_moe((a.K + 63) / 64);
    hipStream_t st = as_stream(s);
#define MX_MOE_G(TT)                                                                     \
    (G == 16 ? launch_moe_tg<F, TT, NW, 16, EPI>(st, b0, b1, a, n_seg)                   \
             : G == 32 ? launch_moe_tg<F, TT, NW, 32, EPI>(st, b0, b1, a, n_seg)         \
                       : launch_moe_tg<F, TT, NW, 64, EPI>(st, b0, b1, a, n_seg))
    if (tt == 1) return MX_MOE_G(1);
    if (tt <= 4) return MX_MOE_G(4);
    return MX_MOE_G(8);
#undef MX_MOE_G
}

// ---------------------------------------------------------------- expert-grouped rows on the matrix cores (mxq_mmq.h)
// grid (blocks of 32 WR weight rows, experts): a workgroup walks its expert's rows in passes of 2 TV tokens; its slice of
// the expert's weights (32 WR rows) is re-read from L2 by every pass after the first.
constexpr uint32_t kMmqMoeLdsBudget = 48 * 1024, kMmqMoeLdsBudgetBig = 78 * 1024;   // the larger one for 32-token passes (opt-in above 64 KB)

template <class P, int TV, int NW, int WR, int WK, int EPI>
static int launch_mmq_grouped_cfg(hipStream_t st, const typename P::Bank& b0, const typename P::Bank& b1, const MoeArgs& m, uint32_t E, uint32_t avg) {
    constexpr bool NATIVE = mmq_native<P>::value;
    MmqArgs<P> a{};
    a.bank0 = b0; a.bank1 = b1; a.xq8 = m.xq8; a.expert_offsets = m.expert_offsets; a.out = m.out; a.bias0 = m.bias0; a.bias1 = m.bias1;
    a.route_w = m.route_w; a.alpha = m.alpha; a.limit = m.limit; a.M = 0; a.K = m.K; a.N = m.N; a.E = E; a.q8_split = m.q8_split;
    a.act_f16 = m.act_f16;
    if (!m.expert_offsets) {   // one matrix, rows [0, n_rows): the token tiles are dealt over gridDim.z
        a.M = m.n_rows;
        a.deal_rows = 1;
    }
    constexpr uint32_t TT = 2 * TV, gran = 256u * WK;
    constexpr uint32_t red = (uint32_t)(NW * WR * WK) * TV * 64u * 4u;
    const uint32_t per256 = TT * (NATIVE ? 512u : 256u) + 8u * TT * 4u * (P::HAS_MIN ? 2u : 1u);
    const uint32_t budget = (TV == 16 || (NATIVE && TV == 8)) ? kMmqMoeLdsBudgetBig : (NATIVE ? 64u * 1024u : kMmqMoeLdsBudget);
    const uint32_t need = ((m.K + 255u) / 256u + WK - 1u) / WK * WK * 256u;
    auto range = [&](uint32_t bytes) {
        uint32_t k = (bytes - 32u * TT) / per256 * 256u / gran * gran;
        if (!k) k = gran;
        return k > need ? need : k;
    };
    // the exchange area sits behind the image when both fit the budget with the whole K range staged (the image then
    // survives from row block to row block); otherwise it overlays the image, which is rebuilt for every row block
    uint32_t kr = range(budget - red);
    const bool overlay = kr < need;
    if (overlay) kr = range(budget);
    a.kr = kr;
    const uint32_t image = (mmq_lds_bytes(TT, kr, TV, P::HAS_MIN, NATIVE) + 15u) & ~15u;
    a.red_off = overlay ? 0u : image;
    const uint32_t lds = overlay ? (image > red ? image : red) : image + red;
    const uint32_t rgs = (m.N + 32u * WR - 1u) / (32u * WR);
    if (E > 65535u) return MX_ERR_SHAPE;
    if (lds > 64u * 1024u) {
        static bool attr_set = false;   // LDS above the 64 KB default limit: opt in once per kernel
        if (!attr_set) {
            const hipError_t er = hipFuncSetAttribute(reinterpret_cast<const void*>(&mmq_kernel<P, TV, NW, WR, WK, EPI>),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMmqMoeLdsBudgetBig);
            if (er != hipSuccess) {
                g_last_hip_error = (int)er;
                return MX_ERR_LAUNCH;
            }
            attr_set = true;
        }
    }
    // token tiles of an expert are dealt over gridDim.z workgroups: the expert sizes live on the device and are skewed (a few
    // experts hold most rows), so the split is sized for experts several times the average; workgroups without a tile leave at once
    uint32_t zt = 2;   // even with small experts a few hold more rows than one tile: their second tile gets a workgroup of its own
    if (!m.expert_offsets) {
        zt = (m.n_rows + TT - 1u) / TT;   // every tile its own workgroup, up to the 32 that share a row block's weights through L2
        if (zt > 32u) zt = 32u;
    } else if (avg == 0 || avg > TT) {
        zt = avg ? (4u * avg + TT - 1u) / TT : 8u;
        if (zt > 32u) zt = 32u;
    }
    // workgroups per expert along the weight rows: when the staged image covers K, about two resident workgroups per CU in
    // all, each streaming several row blocks against its one image; otherwise one workgroup per row block
    uint32_t gx = rgs;
    if (!overlay && avg && avg <= TT) {   // known, small experts only: with skewed or unknown sizes the row blocks stay spread
        const uint64_t slots = 2ull * (uint64_t)cu_count_moe();
        const uint32_t per = (uint32_t)(((uint64_t)rgs * E + slots - 1u) / slots);   // nearly every expert has one tile
        if (per > 1u) gx = (rgs + per - 1u) / per;
    }
    hipLaunchKernelGGL((mmq_kernel<P, TV, NW, WR, WK, EPI>), dim3(gx, E, zt), dim3(64 * NW * WR * WK), lds, st, a);
    return launch_status();
}

// avg_rows = expected rows per expert (0: unknown)
template <class P, int NW, int EPI>
static int launch_mmq_grouped(mx_stream_t s, const typename P::Bank& b0, const typename P::Bank& b1, const MoeArgs& m, uint32_t E, uint32_t avg_rows) {
    hipStream_t st = as_stream(s);
    if (avg_rows && avg_rows <= 8) return launch_mmq_grouped_cfg<P, 4, NW, 1, 4 / NW, EPI>(st, b0, b1, m, E, avg_rows);
    if (avg_rows && avg_rows <= 16) return launch_mmq_grouped_cfg<P, 8, NW, 1, 4 / NW, EPI>(st, b0, b1, m, E, avg_rows);
    if constexpr (mmq_native<P>::value) return launch_mmq_grouped_cfg<P, 8, NW, 1, 4 / NW, EPI>(st, b0, b1, m, E, avg_rows);   // passes of at most 16 tokens
    else return launch_mmq_grouped_cfg<P, 16, NW, (NW == 1 ? 4 : 2), 1, EPI>(st, b0, b1, m, E, avg_rows);
}

// rows per token tile in grouped mode: expected rows per expert, rounded up to 4 or 8
static uint32_t grouped_tt(uint64_t total_rows, uint32_t E) { return (total_rows <= 4ull * E) ? 4 : 8; }
// expected rows per expert for the matrix-core launch (0: the signature carries no row count)
static uint32_t avg_rows(uint32_t total_rows, uint32_t E) { return total_rows == 0xFFFFFFFFu ? 0u : (total_rows + E - 1u) / E; }

template <class F, int MODE>
static int launch_moe_fact(mx_stream_t s, const typename F::Bank& b0, const typename F::Bank& b1, MoeFactArgs a, uint32_t n_seg) {
    const uint32_t n_act = (MODE == FACT_DOWN) ? a.K_top : 1u;
    const uint32_t K256 = (a.K + 255) / 256 * 256;
    uint32_t KT = K256;                                           // whole rows if they fit, else balanced K tiles
    const uint32_t kt_max = (kMoeFactLds / (n_act * 17u)) * 4u / 256u * 256u;   // 4.25 bytes per staged element
    if (kt_max == 0) return MX_ERR_SHAPE;
    if (KT > kt_max) {
        const uint32_t n_tiles = (K256 + kt_max - 1) / kt_max;
        KT = (K256 / 256 + n_tiles - 1) / n_tiles * 256;
    }
    a.KT = KT;
    const uint32_t lds = n_act * (KT * 4 + KT / 16 * 4);
    const uint32_t G = pick_group_moe((a.K + 63) / 64);
    const uint32_t rows_per_wg = kGemvWaves * (64 / G);
    const uint32_t n_rg = (a.N + rows_per_wg - 1) / rows_per_wg;
    uint32_t gx = (uint32_t)cu_count_moe() * 8 / n_seg;
    if (gx < 1) gx = 1;
    if (gx > n_rg) gx = n_rg;
    if (n_seg > 65535) return MX_ERR_SHAPE;
    hipStream_t st = as_stream(s);
    if (G == 16) hipLaunchKernelGGL((moe_fact_kernel<F, 16, MODE>), dim3(gx, n_seg), dim3(kGemvThreads), lds, st, b0, b1, a);
    else if (G == 32) hipLaunchKernelGGL((moe_fact_kernel<F, 32, MODE>), dim3(gx, n_seg), dim3(kGemvThreads), lds, st, b0, b1, a);
    else hipLaunchKernelGGL((moe_fact_kernel<F, 64, MODE>), dim3(gx, n_seg), dim3(kGemvThreads), lds, st, b0, b1, a);
    return launch_status();
}

template <class F, int MODE>
static int moe_decode_fact(mx_stream_t s, const uint16_t* act, const void* W0, const void* W1, const int32_t* topk_idx, const uint16_t* topk_w,
                           uint16_t* out, uint32_t K, uint32_t N, uint32_t K_top, uint32_t T, uint64_t expert_stride_bytes) {
    constexpr uint32_t w_align = F::W_ALIGN;
    MX_REQUIRE_PTR(act); MX_REQUIRE_PTR(W0); MX_REQUIRE_PTR(W1); MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(out);
    if (MODE == FACT_DOWN) MX_REQUIRE_PTR(topk_w);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && K % 256 == 0 && K_top > 0 && T > 0 && expert_stride_bytes % w_align == 0);
    MX_REQUIRE_ALIGN(W0, w_align); MX_REQUIRE_ALIGN(W1, w_align);
    MoeFactArgs a{};
    a.act = reinterpret_cast<const half_t*>(act); a.topk_idx = topk_idx; a.topk_w = reinterpret_cast<const half_t*>(topk_w);
    a.out = reinterpret_cast<half_t*>(out); a.K = K; a.N = N; a.K_top = K_top;
    const typename F::Bank b0 = F::bank(W0, expert_stride_bytes, K, N), b1 = F::bank(W1, expert_stride_bytes, K, N);
    return launch_moe_fact<F, MODE>(s, b0, b1, a, MODE == FACT_DOWN ? T : T * K_top);
}

static int check_moe(const void* x, const void* out, uint32_t K, uint32_t N, uint32_t n_seg) {
    MX_REQUIRE_PTR(x);
    MX_REQUIRE_PTR(out);
    MX_REQUIRE_SHAPE(K > 0 && N > 0 && K % 32 == 0 && n_seg > 0);
    MX_REQUIRE_ALIGN(x, 8);
    return MX_OK;
}

// K-quant AoS expert banks, expert-grouped rows, int-dot: shared argument checks and launch
template <class F, int NW, int EPI>
static int moe_grouped_kquant(mx_stream_t s, const void* act_q8, bool split, const void* W0, const void* W1, uint64_t expert_stride_bytes,
                              const uint32_t* expert_offsets, uint16_t* out, uint32_t E, uint32_t K, uint32_t N, uint32_t total_rows) {
    constexpr uint32_t w_align = F::W_ALIGN;
    if (int rc = check_moe(act_q8, out, K, N, E)) return rc;
    MX_REQUIRE_PTR(W0); MX_REQUIRE_PTR(W1); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(K % 256 == 0 && expert_stride_bytes % w_align == 0);
    MX_REQUIRE_ALIGN(W0, w_align); MX_REQUIRE_ALIGN(W1, w_align);
    if (split) MX_REQUIRE_ALIGN(act_q8, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(act_q8); a.expert_offsets = expert_offsets; a.out = reinterpret_cast<half_t*>(out);
    a.act_div = 1; a.K = K; a.N = N; a.n_experts = E; a.q8_split = split ? 1u : 0u;
    const typename F::Bank b0 = F::bank(W0, expert_stride_bytes, K, N), b1 = F::bank(W1, expert_stride_bytes, K, N);
    constexpr int MEPI = EPI == EPI_SILU ? MMQ_SILU : MMQ_DOWN_BIAS;
    if constexpr (std::is_same<F, FmtQ4K>::value) return launch_mmq_grouped<MmqQ4K, NW, MEPI>(s, b0, b1, a, E, avg_rows(total_rows, E));
    if constexpr (std::is_same<F, FmtQ6K>::value) return launch_mmq_grouped<MmqQ6K, NW, MEPI>(s, b0, b1, a, E, avg_rows(total_rows, E));
    if constexpr (std::is_same<F, FmtQ4KStr>::value) return launch_mmq_grouped<MmqQ4KStr, NW, MEPI>(s, b0, b1, a, E, avg_rows(total_rows, E));
    if constexpr (std::is_same<F, FmtQ6KStr>::value) return launch_mmq_grouped<MmqQ6KStr, NW, MEPI>(s, b0, b1, a, E, avg_rows(total_rows, E));
    return launch_moe<F, NW, EPI>(s, b0, b1, a, E, grouped_tt(total_rows, E));
}

}  // namespace mxq

using namespace mxq;

// The same for K-quant and Q8_0 matrices (no counterpart in the reference, whose dense int-dot GEMM exists for Q4_0 only):
// y[M, N] = q8(x)[M, K] . W[N, K]^T over block_q8_1s rows, int8 matrix cores with the fp32 fold per block.
template <class P, class F>
static int gemm_q8_rows(mx_stream_t s, const void* xq8s_packed, const typename F::Bank& b, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, uint32_t k_align) {
    if (int rc = check_moe(xq8s_packed, y, K, N, 1)) return rc;
    MX_REQUIRE_SHAPE(M > 0 && K % k_align == 0);
    MX_REQUIRE_ALIGN(xq8s_packed, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(xq8s_packed); a.out = reinterpret_cast<half_t*>(y);
    a.act_div = 1; a.K = K; a.N = N; a.n_experts = 1; a.q8_split = 1; a.n_rows = M;
    return launch_mmq_grouped<P, 1, MMQ_STORE>(s, b, b, a, 1, M);
}
extern "C" {

// ------------------------------------------------------------ Q8_0 SoA experts, decode
// The reference signatures carry no expert count, so through them only negative ids can be told apart (their slots are
// skipped); the *_n forms take the count and skip every id outside [0, n_experts).
constexpr uint32_t kAnyExpert = 0x80000000u;
int mx_moe_gate_up_silu_q8_n(mx_stream_t s, const void* x_q8, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs, const uint16_t* u_d,
                             uint64_t qs_stride, uint64_t d_stride, const int32_t* topk_idx, uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H,
                             uint32_t E_ffn, uint32_t n_experts) {
    if (int rc = check_moe(x_q8, h_out, H, E_ffn, T * K)) return rc;
    MX_REQUIRE_PTR(g_qs); MX_REQUIRE_PTR(g_d); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_d); MX_REQUIRE_PTR(topk_idx);
    MX_REQUIRE_SHAPE(K > 0 && n_experts > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(g_qs, 16); MX_REQUIRE_ALIGN(u_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(x_q8); a.topk_idx = topk_idx; a.out = reinterpret_cast<half_t*>(h_out);
    a.act_div = K; a.K = H; a.N = E_ffn; a.n_experts = n_experts;
    FmtQ8Soa::Bank bg{g_qs, g_d, qs_stride, d_stride, H}, bu{u_qs, u_d, qs_stride, d_stride, H};
    return launch_moe<FmtQ8Soa, 2, EPI_SILU>(s, bg, bu, a, T * K, 1);
}
int mx_moe_gate_up_silu_q8(mx_stream_t s, const void* x_q8, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs, const uint16_t* u_d,
                           uint64_t qs_stride, uint64_t d_stride, const int32_t* topk_idx, uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H,
                           uint32_t E_ffn) {
    return mx_moe_gate_up_silu_q8_n(s, x_q8, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, topk_idx, h_out, T, K, H, E_ffn, kAnyExpert);
}
int mx_moe_down_q8_n(mx_stream_t s, const void* h_q8, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                     const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H,
                     uint32_t n_experts) {
    if (int rc = check_moe(h_q8, y_packed, E_ffn, H, T * K)) return rc;
    MX_REQUIRE_PTR(d_qs); MX_REQUIRE_PTR(d_d); MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w);
    MX_REQUIRE_SHAPE(n_experts > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(d_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(h_q8); a.topk_idx = topk_idx; a.route_w = reinterpret_cast<const half_t*>(topk_w);
    a.out = reinterpret_cast<half_t*>(y_packed); a.act_div = 1; a.K = E_ffn; a.N = H; a.n_experts = n_experts;
    FmtQ8Soa::Bank b{d_qs, d_d, qs_stride, d_stride, E_ffn};
    return launch_moe<FmtQ8Soa, 1, EPI_DOWN_WEIGHTED>(s, b, b, a, T * K, 1);
}
int mx_moe_down_q8(mx_stream_t s, const void* h_q8, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                   const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H) {
    return mx_moe_down_q8_n(s, h_q8, d_qs, d_d, qs_stride, d_stride, topk_idx, topk_w, y_packed, T, K, E_ffn, H, kAnyExpert);
}
// ------------------------------------------------------------ K-quant experts, fp16 activations, decode
// soa != 0: every expert region holds its blocks as per-field streams (include/ie/quant_soa.hpp:33-51)
int mx_moe_decode_gate_up_silu_q4k(mx_stream_t s, const uint16_t* x, const void* gate_W, const void* up_W, const int32_t* topk_idx, uint16_t* h_out,
                                   uint32_t H, uint32_t E_ffn, uint32_t K_top, uint64_t expert_stride_bytes, int soa, uint32_t T) {
    if (soa) return moe_decode_fact<FmtQ4KStr, FACT_GATE_UP>(s, x, gate_W, up_W, topk_idx, nullptr, h_out, H, E_ffn, K_top, T, expert_stride_bytes);
    return moe_decode_fact<FmtQ4K, FACT_GATE_UP>(s, x, gate_W, up_W, topk_idx, nullptr, h_out, H, E_ffn, K_top, T, expert_stride_bytes);
}
int mx_moe_decode_down_q4k(mx_stream_t s, const uint16_t* h, const void* down_W, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_out,
                           uint32_t H, uint32_t E_ffn, uint32_t K_top, uint64_t expert_stride_bytes, int soa, uint32_t T) {
    if (soa) return moe_decode_fact<FmtQ4KStr, FACT_DOWN>(s, h, down_W, down_W, topk_idx, topk_w, y_out, E_ffn, H, K_top, T, expert_stride_bytes);
    return moe_decode_fact<FmtQ4K, FACT_DOWN>(s, h, down_W, down_W, topk_idx, topk_w, y_out, E_ffn, H, K_top, T, expert_stride_bytes);
}
int mx_moe_decode_down_q6k(mx_stream_t s, const uint16_t* h, const void* down_W, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_out,
                           uint32_t H, uint32_t E_ffn, uint32_t K_top, uint64_t expert_stride_bytes, int soa, uint32_t T) {
    if (soa) return moe_decode_fact<FmtQ6KStr, FACT_DOWN>(s, h, down_W, down_W, topk_idx, topk_w, y_out, E_ffn, H, K_top, T, expert_stride_bytes);
    return moe_decode_fact<FmtQ6K, FACT_DOWN>(s, h, down_W, down_W, topk_idx, topk_w, y_out, E_ffn, H, K_top, T, expert_stride_bytes);
}
// ------------------------------------------------------------ K-quant experts, grouped rows, int-dot
// Every entry of this family reads block_q8_1s rows (48 B: {d, s0, s1, pad, qs[32]}), as the reference kernels do
// (src/ops/moe_fused.cpp:559-566,672-687: header as one float4, quants at +16 B, min term on s0 + s1;
// src/ops/moe_qwen3.cpp:346); their callers quantize with quantize_q8_1s (src/model/qwen3moe.cpp:563,588).
int mx_moe_prefill_gate_up_silu_q4k_q8(mx_stream_t s, const void* xq8s_packed, const void* gate_W, const void* up_W, const uint32_t* expert_offsets,
                                       uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa,
                                       uint32_t total_rows) {
    if (soa)
        return moe_grouped_kquant<FmtQ4KStr, 2, EPI_SILU>(s, xq8s_packed, true, gate_W, up_W, expert_stride_bytes, expert_offsets, h_packed, E, H, E_ffn, total_rows);
    return moe_grouped_kquant<FmtQ4K, 2, EPI_SILU>(s, xq8s_packed, true, gate_W, up_W, expert_stride_bytes, expert_offsets, h_packed, E, H, E_ffn, total_rows);
}
int mx_moe_prefill_gate_up_silu_q6k_q8(mx_stream_t s, const void* xq8s_packed, const void* gate_W, const void* up_W, const uint32_t* expert_offsets,
                                       uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa,
                                       uint32_t total_rows) {
    if (soa)
        return moe_grouped_kquant<FmtQ6KStr, 2, EPI_SILU>(s, xq8s_packed, true, gate_W, up_W, expert_stride_bytes, expert_offsets, h_packed, E, H, E_ffn, total_rows);
    return moe_grouped_kquant<FmtQ6K, 2, EPI_SILU>(s, xq8s_packed, true, gate_W, up_W, expert_stride_bytes, expert_offsets, h_packed, E, H, E_ffn, total_rows);
}
int mx_moe_prefill_down_packed_q4k_q8(mx_stream_t s, const void* hq8s_packed, const void* down_W, const uint32_t* expert_offsets, uint16_t* out_packed,
                                      uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    if (soa)
        return moe_grouped_kquant<FmtQ4KStr, 1, EPI_DOWN_BIAS>(s, hq8s_packed, true, down_W, down_W, expert_stride_bytes, expert_offsets, out_packed, E, E_ffn, H, total_rows);
    return moe_grouped_kquant<FmtQ4K, 1, EPI_DOWN_BIAS>(s, hq8s_packed, true, down_W, down_W, expert_stride_bytes, expert_offsets, out_packed, E, E_ffn, H, total_rows);
}
int mx_moe_prefill_down_packed_q6k_q8(mx_stream_t s, const void* hq8s_packed, const void* down_W, const uint32_t* expert_offsets, uint16_t* out_packed,
                                      uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    if (soa)
        return moe_grouped_kquant<FmtQ6KStr, 1, EPI_DOWN_BIAS>(s, hq8s_packed, true, down_W, down_W, expert_stride_bytes, expert_offsets, out_packed, E, E_ffn, H, total_rows);
    return moe_grouped_kquant<FmtQ6K, 1, EPI_DOWN_BIAS>(s, hq8s_packed, true, down_W, down_W, expert_stride_bytes, expert_offsets, out_packed, E, E_ffn, H, total_rows);
}
// ------------------------------------------------------------ Q8_0 SoA experts, grouped rows, int-dot GEMV form
static int moe_grouped_gate_up_silu_q8_gemv(mx_stream_t s, const void* xq8_packed, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                                   const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets,
                                   uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    if (int rc = check_moe(xq8_packed, h_packed, H, E_ffn, E)) return rc;
    MX_REQUIRE_PTR(g_qs); MX_REQUIRE_PTR(g_d); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_d); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(g_qs, 16); MX_REQUIRE_ALIGN(u_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(xq8_packed); a.expert_offsets = expert_offsets; a.out = reinterpret_cast<half_t*>(h_packed);
    a.act_div = 1; a.K = H; a.N = E_ffn; a.n_experts = E;
    FmtQ8Soa::Bank bg{g_qs, g_d, qs_stride, d_stride, H}, bu{u_qs, u_d, qs_stride, d_stride, H};
    return launch_mmq_grouped<MmqQ8Soa, 2, MMQ_SILU>(s, bg, bu, a, E, avg_rows(total_rows, E));
}
static int moe_grouped_down_q8_gemv(mx_stream_t s, const void* hq8_packed, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                           uint64_t d_stride, const uint32_t* expert_offsets, const uint16_t* sorted_w, uint16_t* out_packed, uint32_t E,
                           uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    if (int rc = check_moe(hq8_packed, out_packed, E_ffn, H, E)) return rc;
    MX_REQUIRE_PTR(d_qs); MX_REQUIRE_PTR(d_d); MX_REQUIRE_PTR(expert_offsets); MX_REQUIRE_PTR(sorted_w);
    MX_REQUIRE_SHAPE(qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(d_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(hq8_packed); a.expert_offsets = expert_offsets; a.route_w = reinterpret_cast<const half_t*>(sorted_w);
    a.out = reinterpret_cast<half_t*>(out_packed); a.act_div = 1; a.K = E_ffn; a.N = H; a.n_experts = E;
    FmtQ8Soa::Bank b{d_qs, d_d, qs_stride, d_stride, E_ffn};
    return launch_mmq_grouped<MmqQ8Soa, 1, MMQ_DOWN_WEIGHTED>(s, b, b, a, E, avg_rows(total_rows, E));
}

int mx_moe_prefill_gate_up_silu_q8(mx_stream_t s, const void* xq8_packed, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                                   const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets,
                                   uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn) {
    return moe_grouped_gate_up_silu_q8_gemv(s, xq8_packed, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, expert_offsets, h_packed, E, H, E_ffn,
                                            0xFFFFFFFFu);
}
int mx_moe_prefill_down_q8(mx_stream_t s, const void* hq8_packed, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                           const uint32_t* expert_offsets, const uint16_t* sorted_w, uint16_t* out_packed, uint32_t E, uint32_t H,
                           uint32_t E_ffn) {
    return moe_grouped_down_q8_gemv(s, hq8_packed, d_qs, d_d, qs_stride, d_stride, expert_offsets, sorted_w, out_packed, E, H, E_ffn, 0xFFFFFFFFu);
}

// ------------------------------------------------------------ MXFP4 SoA experts (gpt-oss)
static int moe_mxfp4_gate_up(mx_stream_t s, const void* x_q8, const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e,
                             uint64_t qs_stride, uint64_t e_stride, const float* gate_bias, const float* up_bias, const int32_t* topk_idx,
                             const uint32_t* expert_offsets, uint16_t* h_out, uint32_t n_seg, uint32_t act_div, uint32_t H, uint32_t E_ffn,
                             uint32_t n_experts, float alpha, float limit, uint32_t tt) {
    if (int rc = check_moe(x_q8, h_out, H, E_ffn, n_seg)) return rc;
    MX_REQUIRE_PTR(g_qs); MX_REQUIRE_PTR(g_e); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_e);
    MX_REQUIRE_SHAPE(n_experts > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(g_qs, 16); MX_REQUIRE_ALIGN(u_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(x_q8); a.topk_idx = topk_idx; a.expert_offsets = expert_offsets; a.bias0 = gate_bias; a.bias1 = up_bias;
    a.out = reinterpret_cast<half_t*>(h_out); a.alpha = alpha; a.limit = limit; a.act_div = act_div; a.K = H; a.N = E_ffn; a.n_experts = n_experts;
    FmtMxfp4Soa::Bank bg{g_qs, g_e, qs_stride, e_stride, H}, bu{u_qs, u_e, qs_stride, e_stride, H};
    if (expert_offsets && H >= 256) return launch_mmq_grouped<MmqMxfp4Native, 2, MMQ_OAI>(s, bg, bu, a, n_seg, tt);   // grouped: tt = expected rows per expert
    if (expert_offsets) return launch_mmq_grouped<MmqMxfp4Soa, 2, MMQ_OAI>(s, bg, bu, a, n_seg, tt);
    return launch_moe<FmtMxfp4Soa, 2, EPI_OAI>(s, bg, bu, a, n_seg, tt);
}
int mx_moe_gate_up_oai_mxfp4(mx_stream_t s, const void* x_q8, const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e,
                             uint64_t qs_stride, uint64_t e_stride, const float* gate_bias, const float* up_bias, const int32_t* topk_idx,
                             uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H, uint32_t E_ffn, uint32_t n_experts, float alpha, float limit) {
    MX_REQUIRE_PTR(topk_idx);
    MX_REQUIRE_SHAPE(K > 0);
    return moe_mxfp4_gate_up(s, x_q8, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, topk_idx, nullptr, h_out, T * K, K, H, E_ffn,
                             n_experts, alpha, limit, 1);
}
int mx_moe_grouped_gate_up_oai_mxfp4(mx_stream_t s, const void* xq8_packed, const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs,
                                     const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride, const float* gate_bias, const float* up_bias,
                                     const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                                     uint32_t total_rows, float alpha, float limit) {
    MX_REQUIRE_PTR(expert_offsets);
    return moe_mxfp4_gate_up(s, xq8_packed, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, nullptr, expert_offsets, h_packed, E, 1,
                             H, E_ffn, E, alpha, limit, avg_rows(total_rows, E));
}
static int moe_mxfp4_down(mx_stream_t s, const void* h_q8, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride, uint64_t e_stride,
                          const float* down_bias, const int32_t* topk_idx, const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t n_seg,
                          uint32_t E_ffn, uint32_t H, uint32_t n_experts, uint32_t tt, bool act_is_f16 = false) {
    if (int rc = check_moe(h_q8, out_packed, E_ffn, H, n_seg)) return rc;
    if (act_is_f16) MX_REQUIRE_ALIGN(h_q8, 16);
    MX_REQUIRE_PTR(d_qs); MX_REQUIRE_PTR(d_e);
    MX_REQUIRE_SHAPE(n_experts > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(d_qs, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(h_q8); a.topk_idx = topk_idx; a.expert_offsets = expert_offsets; a.bias0 = down_bias;
    a.out = reinterpret_cast<half_t*>(out_packed); a.act_div = 1; a.K = E_ffn; a.N = H; a.n_experts = n_experts;
    if (act_is_f16) a.act_f16 = static_cast<const half_t*>(h_q8);
    FmtMxfp4Soa::Bank b{d_qs, d_e, qs_stride, e_stride, E_ffn};
    if (expert_offsets && E_ffn >= 256) return launch_mmq_grouped<MmqMxfp4Native, 1, MMQ_DOWN_BIAS>(s, b, b, a, n_seg, tt);   // grouped: tt = expected rows per expert
    if (expert_offsets) return launch_mmq_grouped<MmqMxfp4Soa, 1, MMQ_DOWN_BIAS>(s, b, b, a, n_seg, tt);
    return launch_moe<FmtMxfp4Soa, 1, EPI_DOWN_BIAS>(s, b, b, a, n_seg, tt);
}
int mx_moe_down_mxfp4(mx_stream_t s, const void* h_q8, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride, uint64_t e_stride,
                      const float* down_bias, const int32_t* topk_idx, uint16_t* out_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H,
                      uint32_t n_experts) {
    MX_REQUIRE_PTR(topk_idx);
    return moe_mxfp4_down(s, h_q8, d_qs, d_e, qs_stride, e_stride, down_bias, topk_idx, nullptr, out_packed, T * K, E_ffn, H, n_experts, 1);
}
int mx_moe_grouped_down_mxfp4(mx_stream_t s, const void* hq8_packed, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                              uint64_t e_stride, const float* down_bias, const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E,
                              uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    MX_REQUIRE_PTR(expert_offsets);
    return moe_mxfp4_down(s, hq8_packed, d_qs, d_e, qs_stride, e_stride, down_bias, nullptr, expert_offsets, out_packed, E, E_ffn, H, E,
                          avg_rows(total_rows, E));
}

// The down projections taking h as fp16 and quantizing it while staging (same q8 values as mx_quantize_q8_1(h)): no quantize launch.
int mx_moe_down_mxfp4_f16(mx_stream_t s, const uint16_t* h_f16, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride, uint64_t e_stride,
                          const float* down_bias, const int32_t* topk_idx, uint16_t* out_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H,
                          uint32_t n_experts) {
    MX_REQUIRE_PTR(topk_idx);
    return moe_mxfp4_down(s, h_f16, d_qs, d_e, qs_stride, e_stride, down_bias, topk_idx, nullptr, out_packed, T * K, E_ffn, H, n_experts, 1, true);
}
int mx_moe_grouped_down_mxfp4_f16(mx_stream_t s, const uint16_t* h_packed_f16, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                                  uint64_t e_stride, const float* down_bias, const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E,
                                  uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    MX_REQUIRE_PTR(expert_offsets);
    return moe_mxfp4_down(s, h_packed_f16, d_qs, d_e, qs_stride, e_stride, down_bias, nullptr, expert_offsets, out_packed, E, E_ffn, H, E,
                          avg_rows(total_rows, E), true);
}
int mx_moe_down_q8_f16_n(mx_stream_t s, const uint16_t* h_f16, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                         const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H,
                         uint32_t n_experts) {
    if (int rc = check_moe(h_f16, y_packed, E_ffn, H, T * K)) return rc;
    MX_REQUIRE_PTR(d_qs); MX_REQUIRE_PTR(d_d); MX_REQUIRE_PTR(topk_idx); MX_REQUIRE_PTR(topk_w);
    MX_REQUIRE_SHAPE(n_experts > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(d_qs, 16); MX_REQUIRE_ALIGN(h_f16, 16);
    MoeArgs a{};
    a.act_f16 = reinterpret_cast<const half_t*>(h_f16); a.xq8 = reinterpret_cast<const uint8_t*>(h_f16); a.topk_idx = topk_idx;
    a.route_w = reinterpret_cast<const half_t*>(topk_w); a.out = reinterpret_cast<half_t*>(y_packed); a.act_div = 1; a.K = E_ffn; a.N = H;
    a.n_experts = n_experts;
    FmtQ8Soa::Bank b{d_qs, d_d, qs_stride, d_stride, E_ffn};
    return launch_moe<FmtQ8Soa, 1, EPI_DOWN_WEIGHTED>(s, b, b, a, T * K, 1);
}
int mx_moe_down_q8_f16(mx_stream_t s, const uint16_t* h_f16, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                       const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T, uint32_t K, uint32_t E_ffn, uint32_t H) {
    return mx_moe_down_q8_f16_n(s, h_f16, d_qs, d_d, qs_stride, d_stride, topk_idx, topk_w, y_packed, T, K, E_ffn, H, kAnyExpert);
}

// ------------------------------------------------------------ Q4_0 experts (Gemma-4 MoE) and the dense W4A8 GEMM
// Plain projections out_packed[row, n] = half(W_e[n, :] . q8(x_row)), rows partitioned by expert_offsets.
int mx_moe_prefill_proj_q4_0_q8(mx_stream_t s, const void* xq8s_packed, const void* W_q4_0, const uint32_t* expert_offsets, uint16_t* out_packed,
                                uint32_t E, uint32_t K, uint32_t N, uint64_t expert_stride_bytes, uint32_t total_rows) {
    if (int rc = check_moe(xq8s_packed, out_packed, K, N, E)) return rc;
    MX_REQUIRE_PTR(W_q4_0); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(expert_stride_bytes % 2 == 0);
    MX_REQUIRE_ALIGN(W_q4_0, 2); MX_REQUIRE_ALIGN(xq8s_packed, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(xq8s_packed); a.expert_offsets = expert_offsets; a.out = reinterpret_cast<half_t*>(out_packed);
    a.act_div = 1; a.K = K; a.N = N; a.n_experts = E; a.q8_split = 1;
    FmtQ40Aos::Bank b{static_cast<const uint8_t*>(W_q4_0), expert_stride_bytes, K / 32 * 18u};
    return launch_mmq_grouped<MmqQ40Aos, 1, MMQ_DOWN_BIAS>(s, b, b, a, E, avg_rows(total_rows, E));
}
int mx_moe_prefill_proj_q4_0_soa_q8(mx_stream_t s, const void* xq8s_packed, const uint8_t* qs_bank, const uint16_t* d_bank,
                                    const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E, uint32_t K, uint32_t N, uint64_t qs_stride,
                                    uint64_t d_stride, uint32_t total_rows) {
    if (int rc = check_moe(xq8s_packed, out_packed, K, N, E)) return rc;
    MX_REQUIRE_PTR(qs_bank); MX_REQUIRE_PTR(d_bank); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(qs_bank, 16); MX_REQUIRE_ALIGN(d_bank, 2); MX_REQUIRE_ALIGN(xq8s_packed, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(xq8s_packed); a.expert_offsets = expert_offsets; a.out = reinterpret_cast<half_t*>(out_packed);
    a.act_div = 1; a.K = K; a.N = N; a.n_experts = E; a.q8_split = 1;
    FmtQ40Soa::Bank b{qs_bank, d_bank, qs_stride, d_stride, K};
    return launch_mmq_grouped<MmqQ40Soa, 1, MMQ_DOWN_BIAS>(s, b, b, a, E, avg_rows(total_rows, E));
}
// gemm_q4_0_q8: y[M, N] = q8(x)[M, K] . W[N, K]^T for any M, int-dot: the rows run as token tiles of 8 over one matrix.
int mx_gemm_q4_0_q8(mx_stream_t s, const void* xq8s_packed, const void* W_q4_0, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    if (int rc = check_moe(xq8s_packed, y, K, N, 1)) return rc;
    MX_REQUIRE_PTR(W_q4_0);
    MX_REQUIRE_SHAPE(M > 0);
    MX_REQUIRE_ALIGN(W_q4_0, 2); MX_REQUIRE_ALIGN(xq8s_packed, 16);
    MoeArgs a{};
    a.xq8 = static_cast<const uint8_t*>(xq8s_packed); a.out = reinterpret_cast<half_t*>(y);
    a.act_div = 1; a.K = K; a.N = N; a.n_experts = 1; a.q8_split = 1; a.n_rows = M;
    FmtQ40Aos::Bank b{static_cast<const uint8_t*>(W_q4_0), 0, K / 32 * 18u};
    if (M >= 5) return launch_mmq_grouped<MmqQ40Aos, 1, MMQ_DOWN_BIAS>(s, b, b, a, 1, M);   // batches on the matrix cores
    return launch_moe<FmtQ40Aos, 1, EPI_DOWN_BIAS>(s, b, b, a, 1, M == 1 ? 1u : 4u);
}
int mx_gemm_q4_K_q8(mx_stream_t s, const void* xq8s_packed, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(W); MX_REQUIRE_ALIGN(W, 16);
    return gemm_q8_rows<MmqQ4K, FmtQ4K>(s, xq8s_packed, FmtQ4K::Bank{static_cast<const uint8_t*>(W), 0, K / 256 * (uint32_t)kQ4KBytes}, y, M, K, N, 256);
}
int mx_gemm_q6_K_q8(mx_stream_t s, const void* xq8s_packed, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(W); MX_REQUIRE_ALIGN(W, 2);
    return gemm_q8_rows<MmqQ6K, FmtQ6K>(s, xq8s_packed, FmtQ6K::Bank{static_cast<const uint8_t*>(W), 0, K / 256 * (uint32_t)kQ6KBytes}, y, M, K, N, 256);
}
int mx_gemm_q8_0_soa_q8(mx_stream_t s, const void* xq8s_packed, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    MX_REQUIRE_PTR(qs_W); MX_REQUIRE_PTR(d_W); MX_REQUIRE_ALIGN(qs_W, 16);
    return gemm_q8_rows<MmqQ8Soa, FmtQ8Soa>(s, xq8s_packed, FmtQ8Soa::Bank{qs_W, d_W, 0, 0, K}, y, M, K, N, 32);
}

// ------------------------------------------------------------ row utilities
int mx_moe_gather_rows(mx_stream_t s, const uint16_t* x, const int32_t* indices, uint16_t* y_packed, uint32_t n_rows, uint32_t hidden) {
    MX_REQUIRE_PTR(x); MX_REQUIRE_PTR(indices); MX_REQUIRE_PTR(y_packed);
    MX_REQUIRE_SHAPE(n_rows > 0 && hidden > 0 && n_rows <= 65535);
    MX_REQUIRE_ALIGN(x, 16); MX_REQUIRE_ALIGN(y_packed, 16);
    hipLaunchKernelGGL(gather_rows_kernel, dim3((hidden + 2047) / 2048, n_rows), dim3(256), 0, as_stream(s), reinterpret_cast<const half_t*>(x),
                       indices, reinterpret_cast<half_t*>(y_packed), n_rows, hidden);
    return launch_status();
}
int mx_moe_scatter_add(mx_stream_t s, const uint16_t* x_packed, const int32_t* indices, const uint16_t* weights, uint16_t* y, uint32_t n_tok,
                       uint32_t hidden) {
    MX_REQUIRE_PTR(x_packed); MX_REQUIRE_PTR(indices); MX_REQUIRE_PTR(weights); MX_REQUIRE_PTR(y);
    MX_REQUIRE_SHAPE(n_tok > 0 && hidden > 0 && n_tok <= 65535);
    MX_REQUIRE_ALIGN(x_packed, 16); MX_REQUIRE_ALIGN(y, 16);
    hipLaunchKernelGGL(scatter_add_kernel, dim3((hidden + 2047) / 2048, n_tok), dim3(256), 0, as_stream(s),
                       reinterpret_cast<const half_t*>(x_packed), indices, reinterpret_cast<const half_t*>(weights), reinterpret_cast<half_t*>(y),
                       n_tok, hidden);
    return launch_status();
}
int mx_moe_prefill_merge_fp32_to_fp16(mx_stream_t s, const float* y_fp32, uint16_t* y_fp16, uint64_t n) {
    MX_REQUIRE_PTR(y_fp32); MX_REQUIRE_PTR(y_fp16);
    MX_REQUIRE_SHAPE(n > 0 && (n + 255) / 256 <= 0x7FFFFFFFull);
    hipLaunchKernelGGL(merge_f32_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, as_stream(s), y_fp32, reinterpret_cast<half_t*>(y_fp16), n);
    return launch_status();
}
static int reduce_common(const void* packed, const void* y, uint32_t T, uint32_t K, uint32_t H) {
    MX_REQUIRE_PTR(packed); MX_REQUIRE_PTR(y);
    MX_REQUIRE_SHAPE(T > 0 && K > 0 && H > 0);
    return MX_OK;
}
int mx_moe_reduce_q8(mx_stream_t s, const uint16_t* y_packed, uint16_t* y, uint32_t T, uint32_t K, uint32_t H) {
    if (int rc = reduce_common(y_packed, y, T, K, H)) return rc;
    hipLaunchKernelGGL((moe_reduce_kernel<false, false>), dim3((uint32_t)(((uint64_t)T * H + 255) / 256)), dim3(256), 0, as_stream(s),
                       reinterpret_cast<const half_t*>(y_packed), nullptr, nullptr, reinterpret_cast<half_t*>(y), T, K, H);
    return launch_status();
}
int mx_moe_prefill_reduce_sum(mx_stream_t s, const uint16_t* out_packed, const uint32_t* tk_to_packed, uint16_t* y, uint32_t T, uint32_t K,
                              uint32_t H) {
    if (int rc = reduce_common(out_packed, y, T, K, H)) return rc;
    MX_REQUIRE_PTR(tk_to_packed);
    hipLaunchKernelGGL((moe_reduce_kernel<false, false>), dim3((uint32_t)(((uint64_t)T * H + 255) / 256)), dim3(256), 0, as_stream(s),
                       reinterpret_cast<const half_t*>(out_packed), tk_to_packed, nullptr, reinterpret_cast<half_t*>(y), T, K, H);
    return launch_status();
}
int mx_moe_prefill_reduce(mx_stream_t s, const uint16_t* out_packed, const uint32_t* tk_to_packed, const uint16_t* weights_packed, uint16_t* y,
                          uint32_t T, uint32_t K_top, uint32_t H) {
    if (int rc = reduce_common(out_packed, y, T, K_top, H)) return rc;
    MX_REQUIRE_PTR(tk_to_packed); MX_REQUIRE_PTR(weights_packed);
    hipLaunchKernelGGL((moe_reduce_kernel<true, true>), dim3((uint32_t)(((uint64_t)T * H + 255) / 256)), dim3(256), 0, as_stream(s),
                       reinterpret_cast<const half_t*>(out_packed), tk_to_packed, reinterpret_cast<const half_t*>(weights_packed),
                       reinterpret_cast<half_t*>(y), T, K_top, H);
    return launch_status();
}

// build_moe_packing (src/model/qwen3moe_pack.cpp:5-31), host pointers: stable counting sort of the
// T*K (token, slot) pairs by expert id.
int mx_build_moe_packing(const int32_t* topk_ids, const float* topk_w, uint32_t T, uint32_t K, uint32_t E, uint32_t* expert_offsets,
                         int32_t* sorted_idx, float* weights_packed, int32_t* tk_to_packed) {
    if (!topk_ids || !topk_w || !expert_offsets || !sorted_idx || !weights_packed || !tk_to_packed) return MX_ERR_NULL;
    if (!T || !K || !E) return MX_ERR_SHAPE;
    for (uint32_t i = 0; i <= E; ++i) expert_offsets[i] = 0;
    for (uint64_t i = 0; i < (uint64_t)T * K; ++i) {
        if (topk_ids[i] < 0 || (uint32_t)topk_ids[i] >= E) return MX_ERR_SHAPE;
        ++expert_offsets[topk_ids[i] + 1];
    }
    for (uint32_t e = 0; e < E; ++e) expert_offsets[e + 1] += expert_offsets[e];
    uint32_t* cur = new uint32_t[E];
    for (uint32_t e = 0; e < E; ++e) cur[e] = expert_offsets[e];
    for (uint32_t t = 0; t < T; ++t)
        for (uint32_t k = 0; k < K; ++k) {
            const uint32_t pos = cur[topk_ids[(size_t)t * K + k]]++;
            sorted_idx[pos] = (int32_t)t;
            weights_packed[pos] = topk_w[(size_t)t * K + k];
            tk_to_packed[(size_t)t * K + k] = (int32_t)pos;
        }
    delete[] cur;
    return MX_OK;
}

}  // extern "C"
