// gemm.hip — prefill quant-GEMM and expert-grouped GEMM on the matrix cores.
//
//   Y[t, n] = sum_k A[t, k] * half(deq(W)[n, k])      fp16 x fp16 -> fp32 accumulate -> fp16
//
// i.e. the arithmetic of the reference's XMX route (weights dequantized to fp16,
// src/ops/gemm_q4k_xmx.cpp:71-111,183-231) and of its dequant + dense-GEMM route
// (src/model/dense_dispatch.hpp:658-693) without ever materialising the fp16
// weight matrix: every weight byte is read once per 128-token tile and
// dequantized in registers straight into MFMA operand fragments.
//
// Tiling (wave64, v_mfma_f32_32x32x16_f16):
//   workgroup = 4 waves, 128 tokens x (4 x 64) weight rows, K walked in chunks of 128;
//   wave      = 128 tokens x 64 rows = 4 x 2 MFMA tiles (128 accumulator VGPRs);
//   tokens    : the fp16 A chunk [128 x 128] is staged in LDS (double buffered, row
//               pitch padded to 272 B so a fragment read is bank-conflict free) and
//               shared by the four waves;
//   weights   : lane (r = lane%32, h = lane/32) of a wave owns weight row r of a tile
//               and the 64 consecutive elements [64h, 64h+64) of the chunk: it loads
//               them from global as 128-bit words (32 B of Q4_K nibbles or 64 B of
//               Q8_0 quants), unpacks scale/min once per chunk and emits, for MFMA
//               step s, the 8 halfs of elements 64h + 8s .. +7 — exactly the MFMA
//               operand layout (lane%32 = row, lane/32 = k group), so no LDS round
//               trip and no redundant dequantisation inside a workgroup.
// The k order inside a chunk is (lanes 0-31: 8s.., lanes 32-63: 64+8s..); the
// A fragments are read from LDS with the same order, so the products pair up.
#include "mxq_device.h"
#include "mxq_host.h"

namespace mxq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float2_t __attribute__((ext_vector_type(2)));

constexpr int kBM = 128;            // tokens per workgroup tile
constexpr int kBK = 128;            // K chunk
constexpr int kWaveN = 64;          // weight rows per wave (2 MFMA tiles)
constexpr int kPitch = kBK + 8;     // LDS row pitch in halfs (272 B)
constexpr int kGemmThreads = 256;
constexpr uint32_t kGemmLds = 2u * kBM * kPitch * 2u;

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const float2_t f = {a, b};
    const half2_t h = __builtin_convertvector(f, half2_t);   // v_cvt_pk_f16_f32, RNE
    return __builtin_bit_cast(uint32_t, h);
}

union Frag {
    half8_t v;
    uint32_t u[4];
    uint4 q;
};

// ---------------------------------------------------------------- weight fragment producers
// Q4_K: chunk kc of a row = half c = kc%2 of block kc/2; lane half h owns the 32 bytes
// qs[32g, 32g+32), g = 2c + h: low nibbles = sub-block 2g, high = sub-block 2g+1.
// value = half(fma(d*sc, q, -(dmin*m))): the products are exact in fp32 so this is
// the single fp32 rounding of the reference expression, then one RNE to fp16.
struct GemmQ4K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint32_t row_bytes;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.base + (size_t)e * b.expert_stride_bytes, b.row_bytes}; }
    struct Raw {
        uint4 hdr, q0, q1;
    };
    struct Dec {
        float d1[2], m1[2];
    };
    static constexpr uint32_t K_ALIGN = 256;
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)(kc >> 1) * kQ4KBytes;
        const uint4* q = reinterpret_cast<const uint4*>(blk + 16 + (2u * (kc & 1u) + h) * 32u);
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t kc, uint32_t h) {
        uint32_t sc, mn;
        q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, (int)(2u * (kc & 1u) + h), sc, mn);
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        Dec o;
        o.d1[0] = d * (float)(sc & 0xFFu);
        o.d1[1] = d * (float)(sc >> 8);
        o.m1[0] = -(dmin * (float)(mn & 0xFFu));
        o.m1[1] = -(dmin * (float)(mn >> 8));
        return o;
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int sub = S / 4, p = S % 4;
        const uint32_t w0 = p == 0 ? r.q0.x : p == 1 ? r.q0.z : p == 2 ? r.q1.x : r.q1.z;
        const uint32_t w1 = p == 0 ? r.q0.y : p == 1 ? r.q0.w : p == 2 ? r.q1.y : r.q1.w;
        const uint32_t n0 = sub ? (w0 >> 4) & 0x0F0F0F0Fu : w0 & 0x0F0F0F0Fu;
        const uint32_t n1 = sub ? (w1 >> 4) & 0x0F0F0F0Fu : w1 & 0x0F0F0F0Fu;
        const float d1 = dc.d1[sub], m1 = dc.m1[sub];
        f.u[0] = pack_h2(__builtin_fmaf(d1, (float)(n0 & 0xFFu), m1), __builtin_fmaf(d1, (float)((n0 >> 8) & 0xFFu), m1));
        f.u[1] = pack_h2(__builtin_fmaf(d1, (float)((n0 >> 16) & 0xFFu), m1), __builtin_fmaf(d1, (float)(n0 >> 24), m1));
        f.u[2] = pack_h2(__builtin_fmaf(d1, (float)(n1 & 0xFFu), m1), __builtin_fmaf(d1, (float)((n1 >> 8) & 0xFFu), m1));
        f.u[3] = pack_h2(__builtin_fmaf(d1, (float)((n1 >> 16) & 0xFFu), m1), __builtin_fmaf(d1, (float)(n1 >> 24), m1));
    }
};

// Q8_0 SoA planes: lane half h owns quants [128 kc + 64h, +64) of the row and the two
// block scales.  value = half(d * q) (exact product, one RNE to fp16), computed as
// fma(d, q + 128, -128 d) on the bias-flipped byte so that the conversion is a
// single v_cvt_f32_ubyte.
struct GemmQ8Soa {
    struct W {
        const int8_t* qs;
        const uint16_t* d;
        uint32_t K;
    };
    struct Bank {
        const int8_t* qs;
        const uint16_t* d;
        uint64_t qs_stride, d_stride;
        uint32_t K;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.qs + (size_t)e * b.qs_stride, b.d + (size_t)e * b.d_stride, b.K}; }
    struct Raw {
        uint4 q[4];
        uint32_t d2;
    };
    struct Dec {
        float d[2], o[2];
    };
    static constexpr uint32_t K_ALIGN = 128;
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint4* p = reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)kc * 128u + 64u * h);
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r.q[i] = p[i];
        r.d2 = *reinterpret_cast<const uint32_t*>(w.d + (size_t)n * (w.K >> 5) + kc * 4u + 2u * h);
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t) {
        Dec o;
        o.d[0] = h2f(r.d2 & 0xFFFFu);
        o.d[1] = h2f(r.d2 >> 16);
        o.o[0] = -128.f * o.d[0];
        o.o[1] = -128.f * o.d[1];
        return o;
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int blk = S / 4, i = (S * 2) / 4, e = (S * 2) % 4;
        const uint32_t a = (e == 0 ? r.q[i].x : r.q[i].z) ^ 0x80808080u, b = (e == 0 ? r.q[i].y : r.q[i].w) ^ 0x80808080u;
        const float d = dc.d[blk], o = dc.o[blk];
        f.u[0] = pack_h2(__builtin_fmaf(d, (float)(a & 0xFFu), o), __builtin_fmaf(d, (float)((a >> 8) & 0xFFu), o));
        f.u[1] = pack_h2(__builtin_fmaf(d, (float)((a >> 16) & 0xFFu), o), __builtin_fmaf(d, (float)(a >> 24), o));
        f.u[2] = pack_h2(__builtin_fmaf(d, (float)(b & 0xFFu), o), __builtin_fmaf(d, (float)((b >> 8) & 0xFFu), o));
        f.u[3] = pack_h2(__builtin_fmaf(d, (float)((b >> 16) & 0xFFu), o), __builtin_fmaf(d, (float)(b >> 24), o));
    }
};

// ---------------------------------------------------------------- kernel
enum { GEMM_DENSE = 0, GEMM_MOE_GATE_UP_SILU = 1, GEMM_MOE_DOWN = 2 };

struct GemmArgs {
    const half_t* A;                  // [M, K] fp16 (dense) or expert-sorted rows [TK, K]
    half_t* Y;                        // [M, N]
    const uint32_t* expert_offsets;   // grouped: [E+1]
    const half_t* route_w;            // GEMM_MOE_DOWN: [TK] fp16
    uint32_t M, K, N, E;
    uint32_t tiles_m, tiles_n;        // dense tile grid; grouped: tiles_m is an upper bound
};

__device__ __forceinline__ float silu_mul_f(float g, float u) { return (g / (1.f + __expf(-g))) * u; }

// `mi` = number of live 32-token tiles of this workgroup tile (4 unless PARTIAL: expert-grouped
// tiles are often mostly empty, and their dead token tiles skip both the LDS reads and the MFMAs).
template <int S, class QF, bool PARTIAL>
__device__ __forceinline__ void mma_step(const typename QF::Raw (&raw)[2], const typename QF::Dec (&dec)[2], const half_t* a_lds, uint32_t r,
                                         uint32_t h, float16_t (&acc)[4][2], uint32_t mi) {
    Frag bf[2];
    QF::template frag<S>(raw[0], dec[0], bf[0]);
    QF::template frag<S>(raw[1], dec[1], bf[1]);
    if (PARTIAL) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if ((uint32_t)i < mi) {
                Frag af;
                af.q = *reinterpret_cast<const uint4*>(a_lds + (size_t)(32 * i + r) * kPitch + 64 * h + 8 * S);
                acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af.v, bf[0].v, acc[i][0], 0, 0, 0);
                acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af.v, bf[1].v, acc[i][1], 0, 0, 0);
            }
        return;
    }
    Frag af[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i].q = *reinterpret_cast<const uint4*>(a_lds + (size_t)(32 * i + r) * kPitch + 64 * h + 8 * S);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i].v, bf[j].v, acc[i][j], 0, 0, 0);
}

template <class QF, int MODE>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_kernel(typename QF::Bank bank0, typename QF::Bank bank1, GemmArgs g) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    half_t* lds = reinterpret_cast<half_t*>(lds_raw);
    constexpr bool GATE_UP = MODE == GEMM_MOE_GATE_UP_SILU;
    constexpr uint32_t BN = GATE_UP ? 4 * 32 : 4 * kWaveN;   // output columns per workgroup

    // ---- which tile: XCD-aware order (workgroup i runs on XCD i % 8; each XCD walks a
    // contiguous range of tiles, 4 token tiles x consecutive column tiles at a time)
    const uint32_t total = g.tiles_m * g.tiles_n;
    const uint32_t per_xcd = (total + 7) / 8;
    const uint32_t linear = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= per_xcd || linear >= total) return;
    uint32_t tm, tn;
    {
        constexpr uint32_t GM = 4;
        const uint32_t grp = linear / (GM * g.tiles_n), in = linear - grp * (GM * g.tiles_n);
        const uint32_t rows_here = (g.tiles_m - grp * GM < GM) ? g.tiles_m - grp * GM : GM;
        tn = in / rows_here;
        tm = grp * GM + in - tn * rows_here;
    }
    uint32_t e = 0, row_lo = 0, row_hi = g.M;
    if (MODE != GEMM_DENSE) {
        // tm-th 128-row tile over all experts: wave 0 scans the per-expert tile counts, 64 experts at a time
        __shared__ uint32_t s_tile[3];
        const uint32_t ln = threadIdx.x & 63u;
        if (threadIdx.x < 64) {
            uint32_t base = 0;
            bool found = false;
            for (uint32_t e0 = 0; e0 < g.E && !found; e0 += 64) {
                const uint32_t ee = e0 + ln;
                const uint32_t lo = ee < g.E ? g.expert_offsets[ee] : 0u, hi = ee < g.E ? g.expert_offsets[ee + 1] : 0u;
                const uint32_t nt = (hi - lo + kBM - 1) / kBM;
                uint32_t incl = nt;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) {
                    const uint32_t v = (uint32_t)__shfl_up((int)incl, d);
                    if (ln >= (uint32_t)d) incl += v;
                }
                const uint32_t excl = base + incl - nt;
                const bool hit = tm >= excl && tm < excl + nt;
                if (hit) {
                    s_tile[0] = ee;
                    s_tile[1] = lo + (tm - excl) * kBM;
                    s_tile[2] = hi;
                }
                found = __ballot(hit) != 0ull;
                base += (uint32_t)__shfl((int)incl, 63);
            }
            if (!found && ln == 0) s_tile[0] = 0xFFFFFFFFu;
        }
        __syncthreads();
        e = s_tile[0];
        if (e == 0xFFFFFFFFu) return;
        row_lo = s_tile[1];
        row_hi = s_tile[2];
    } else {
        row_lo = tm * kBM;
    }
    const typename QF::W w0 = QF::expert(bank0, e), w1 = QF::expert(GATE_UP ? bank1 : bank0, e);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, r = lane & 31u, h = lane >> 5;
    const uint32_t n_base = tn * BN + wave * (GATE_UP ? 32 : kWaveN);
    // weight rows of the two MFMA column tiles of this wave (gate/up: same row in two matrices)
    uint32_t wrow[2];
    wrow[0] = n_base + r;
    wrow[1] = GATE_UP ? n_base + r : n_base + 32 + r;
    if (wrow[0] >= g.N) wrow[0] = g.N - 1;
    if (wrow[1] >= g.N) wrow[1] = g.N - 1;

    // A staging: thread loads 8 x 16 B: rows (tid/16) + 16 i, 16-byte column tid%16
    const uint32_t a_col = (tid & 15u) * 8u, a_row = tid >> 4;
    const half_t* a_src[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t row = row_lo + a_row + 16 * i;
        if (row >= row_hi) row = row_hi - 1;
        a_src[i] = g.A + (size_t)row * g.K + a_col;
    }
    const uint32_t n_chunks = g.K / kBK;
    constexpr bool PARTIAL = MODE != GEMM_DENSE;
    const uint32_t live_rows = row_hi - row_lo;
    const uint32_t mi = live_rows >= (uint32_t)kBM ? 4u : (live_rows + 31u) / 32u;

    float16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Software pipeline over K chunks: the weight words and the A rows of chunk c+1 are
    // fetched from global while chunk c is multiplied; the A rows go through registers in
    // two halves (rows 0..63 during steps 0-3, rows 64..127 during steps 4-7) into the
    // other LDS buffer.  The last chunk is peeled so the loop body has no conditionals.
    typename QF::Raw raw[2];
    raw[0] = QF::load(w0, wrow[0], 0, h);
    raw[1] = QF::load(w1, wrow[1], 0, h);
    {
        uint4 a0[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) a0[i] = *reinterpret_cast<const uint4*>(a_src[i]);
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(lds + (size_t)(a_row + 16 * i) * kPitch + a_col) = a0[i];
    }
    __syncthreads();

    for (uint32_t c = 0; c + 1 < n_chunks; ++c) {
        typename QF::Raw nxt[2];
        nxt[0] = QF::load(w0, wrow[0], c + 1, h);
        nxt[1] = QF::load(w1, wrow[1], c + 1, h);
        uint4 alo[4], ahi[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) alo[i] = *reinterpret_cast<const uint4*>(a_src[i] + (size_t)(c + 1) * kBK);
        typename QF::Dec dec[2];
        dec[0] = QF::prepare(raw[0], c, h);
        dec[1] = QF::prepare(raw[1], c, h);
        const half_t* a_lds = lds + (size_t)(c & 1u) * (kBM * kPitch);
        half_t* dst = lds + (size_t)((c + 1) & 1u) * (kBM * kPitch);
        mma_step<0, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<1, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<2, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<3, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(dst + (size_t)(a_row + 16 * i) * kPitch + a_col) = alo[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) ahi[i] = *reinterpret_cast<const uint4*>(a_src[4 + i] + (size_t)(c + 1) * kBK);
        mma_step<4, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<5, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<6, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<7, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(dst + (size_t)(a_row + 16 * (4 + i)) * kPitch + a_col) = ahi[i];
        raw[0] = nxt[0];
        raw[1] = nxt[1];
        __syncthreads();
    }
    {
        const uint32_t c = n_chunks - 1;
        typename QF::Dec dec[2];
        dec[0] = QF::prepare(raw[0], c, h);
        dec[1] = QF::prepare(raw[1], c, h);
        const half_t* a_lds = lds + (size_t)(c & 1u) * (kBM * kPitch);
        mma_step<0, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<1, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<2, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<3, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<4, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<5, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<6, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
        mma_step<7, QF, PARTIAL>(raw, dec, a_lds, r, h, acc, mi);
    }

    // ---- epilogue.  MFMA C layout: lane holds column n = lane%32, rows 8*(v/4) + 4*(lane/32) + v%4.
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t row = row_lo + 32 * i + 8 * (v / 4) + 4 * h + (v % 4);
            if (row >= row_hi) continue;
            if (GATE_UP) {
                const uint32_t n = n_base + r;
                if (n < g.N) g.Y[(size_t)row * g.N + n] = (half_t)silu_mul_f(acc[i][0][v], acc[i][1][v]);
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t n = n_base + 32 * j + r;
                    if (n >= g.N) continue;
                    float o = acc[i][j][v];
                    if (MODE == GEMM_MOE_DOWN) o *= (float)g.route_w[row];
                    g.Y[(size_t)row * g.N + n] = (half_t)o;
                }
            }
        }
}

// ---------------------------------------------------------------- host side
template <class QF, int MODE>
static int launch_gemm(mx_stream_t s, const typename QF::Bank& b0, const typename QF::Bank& b1, GemmArgs g, uint32_t rows_bound) {
    constexpr uint32_t BN = (MODE == GEMM_MOE_GATE_UP_SILU) ? 128 : 256;
    g.tiles_n = (g.N + BN - 1) / BN;
    g.tiles_m = (MODE == GEMM_DENSE) ? (g.M + kBM - 1) / kBM : (rows_bound + kBM - 1) / kBM + g.E;
    const uint64_t total = (uint64_t)g.tiles_m * g.tiles_n;
    const uint64_t grid = (total + 7) / 8 * 8;
    if (grid > 0x7FFFFFFFull) return MX_ERR_SHAPE;
    static bool attr_set = false;   // LDS above the 64 KB default needs the opt-in, once per kernel
    if (!attr_set) {
        const hipError_t er = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<QF, MODE>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemmLds);
        if (er != hipSuccess) {
            g_last_hip_error = (int)er;
            return MX_ERR_LAUNCH;
        }
        attr_set = true;
    }
    hipLaunchKernelGGL((gemm_kernel<QF, MODE>), dim3((uint32_t)grid), dim3(kGemmThreads), kGemmLds, as_stream(s), b0, b1, g);
    return launch_status();
}

static int check_gemm(const void* A, const void* W, const void* y, uint32_t M, uint32_t K, uint32_t N, uint32_t k_align) {
    MX_REQUIRE_PTR(A);
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_PTR(y);
    MX_REQUIRE_SHAPE(M > 0 && N > 0 && K > 0 && K % k_align == 0);
    MX_REQUIRE_ALIGN(A, 16);
    MX_REQUIRE_ALIGN(W, 16);
    return MX_OK;
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_gemm_q4_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    if (int rc = check_gemm(A, W, y, M, K, N, 256)) return rc;
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(A); g.Y = reinterpret_cast<half_t*>(y); g.M = M; g.K = K; g.N = N; g.E = 1;
    GemmQ4K::Bank b{static_cast<const uint8_t*>(W), 0, K / 256 * (uint32_t)kQ4KBytes};
    return launch_gemm<GemmQ4K, GEMM_DENSE>(s, b, b, g, M);
}

int mx_gemm_q8_0_soa(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    if (int rc = check_gemm(A, qs_W, y, M, K, N, 128)) return rc;
    MX_REQUIRE_PTR(d_W);
    MX_REQUIRE_ALIGN(d_W, 4);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(A); g.Y = reinterpret_cast<half_t*>(y); g.M = M; g.K = K; g.N = N; g.E = 1;
    GemmQ8Soa::Bank b{qs_W, d_W, 0, 0, K};
    return launch_gemm<GemmQ8Soa, GEMM_DENSE>(s, b, b, g, M);
}

int mx_moe_gemm_gate_up_silu_q8(mx_stream_t s, const uint16_t* x_packed, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                                const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets, uint16_t* h_packed,
                                uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    if (int rc = check_gemm(x_packed, g_qs, h_packed, total_rows, H, E_ffn, 128)) return rc;
    MX_REQUIRE_PTR(g_d); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_d); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && qs_stride % 16 == 0 && d_stride % 2 == 0);
    MX_REQUIRE_ALIGN(u_qs, 16); MX_REQUIRE_ALIGN(g_d, 4); MX_REQUIRE_ALIGN(u_d, 4);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(x_packed); g.Y = reinterpret_cast<half_t*>(h_packed); g.expert_offsets = expert_offsets;
    g.M = total_rows; g.K = H; g.N = E_ffn; g.E = E;
    GemmQ8Soa::Bank bg{g_qs, g_d, qs_stride, d_stride, H}, bu{u_qs, u_d, qs_stride, d_stride, H};
    return launch_gemm<GemmQ8Soa, GEMM_MOE_GATE_UP_SILU>(s, bg, bu, g, total_rows);
}

int mx_moe_gemm_down_q8(mx_stream_t s, const uint16_t* h_packed, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride, uint64_t d_stride,
                        const uint32_t* expert_offsets, const uint16_t* sorted_w, uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                        uint32_t total_rows) {
    if (int rc = check_gemm(h_packed, d_qs, out_packed, total_rows, E_ffn, H, 128)) return rc;
    MX_REQUIRE_PTR(d_d); MX_REQUIRE_PTR(expert_offsets); MX_REQUIRE_PTR(sorted_w);
    MX_REQUIRE_SHAPE(E > 0 && qs_stride % 16 == 0 && d_stride % 2 == 0);
    MX_REQUIRE_ALIGN(d_d, 4);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(h_packed); g.Y = reinterpret_cast<half_t*>(out_packed); g.expert_offsets = expert_offsets;
    g.route_w = reinterpret_cast<const half_t*>(sorted_w); g.M = total_rows; g.K = E_ffn; g.N = H; g.E = E;
    GemmQ8Soa::Bank b{d_qs, d_d, qs_stride, d_stride, E_ffn};
    return launch_gemm<GemmQ8Soa, GEMM_MOE_DOWN>(s, b, b, g, total_rows);
}

}  // extern "C"
