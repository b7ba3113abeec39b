// mxq_gemv_core.h — the bandwidth-bound int-dot GEMV core shared by the dense,
// fused gate/up and expert-indexed entry points.
//
// Work decomposition (wave64):
//   * a group of G lanes (G = 16, 32 or 64) owns R consecutive weight rows; lane l
//     of the group walks 64-weight units l, l+G, l+2G ... of each row, so one
//     wave-wide load instruction fetches consecutive 16-byte chunks of a row
//     (coalesced 128-bit loads of whole super-blocks);
//   * the T activation rows (block_q8_1x streams) are staged once per K-tile in
//     LDS as two planes — the int8 quants and a header plane holding the block
//     scale d8 (plus, for the K-quants, d8 * sum(q8) per 32 or per 16 elements) —
//     and every lane reads the 64 quants that face its unit with four
//     ds_read_b128;
//   * scale/min unpacking, the int8 dot (v_dot4_i32_i8) and the fp32 fold run in
//     registers; the per-row result is reduced across the group with DPP.
// No MFMA: at T <= 8 the kernel is a stream over the weight bytes.
#pragma once

#include "mxq_formats.h"

namespace mxq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;

// Header plane entry size per 32 activation elements:
//   SUM_GRAN 0  : float  d8                       (4 B / 32)
//   SUM_GRAN 32 : float2 {d8, d8*sum32}           (8 B / 32)
//   SUM_GRAN 16 : float2 {d8, d8*sum16} per 16    (16 B / 32)
//   SUM_GRAN 2  : float  d8; the quants of this layout are fp16 (MXFP4, see stage_act)   (4 B / 32)
__host__ __device__ constexpr uint32_t hdr_bytes_per32(int sum_gran) { return (sum_gran == 0 || sum_gran == 2) ? 4 : (sum_gran == 32 ? 8 : 16); }
__host__ __device__ constexpr uint32_t qs_bytes_per32(int sum_gran) { return sum_gran == 2 ? 64 : 32; }
__host__ __device__ constexpr uint32_t act_tile_bytes(uint32_t T, uint32_t KT, int sum_gran) {
    return T * (KT / 32) * (qs_bytes_per32(sum_gran) + hdr_bytes_per32(sum_gran));
}

struct ActTile {
    const uint4* qs;      // [T][KT/16] 16-quant chunks
    const uint8_t* hdr;   // [T][KT/32] entries, see hdr_bytes_per32
    uint32_t KT;
};

// Where 16-quant chunk q of a staged row lives.  A lane reads the chunks facing its 64-element unit, so lanes sit 64 B
// apart (units of consecutive elements) and the 16 lanes one ds_read_b128 pass serves would share four bank groups; the
// XOR spreads them over all sixteen.  Units of consecutive elements (every format but Q6_K) permute the four chunks inside
// a unit; Q6_K's units interleave two 128-element halves (K is a multiple of 256 there), so the bits one up are used.
// SUM_GRAN 2 (fp16 quants, 128 B per unit): eight chunks per unit, permuted by the bits above the pair of units that
// shares a 256-byte bank row.
template <int SUM_GRAN>
__device__ __forceinline__ uint32_t act_slot(uint32_t q) {
    if (SUM_GRAN == 2) return q ^ ((q >> 4) & 7u);
    return q ^ (((q >> 4) & 3u) << (SUM_GRAN == 16 ? 1 : 0));
}

// Four int8 of `lo` and of `hi` -> four fp16 pairs {half(lo[b]), half(hi[b])} (exact: |q| <= 127).
__device__ __forceinline__ uint4 q8_pairs_f16(uint32_t lo, uint32_t hi) {
    uint32_t o[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const half_t l = (half_t)(int)(int8_t)(lo >> (8 * b)), h = (half_t)(int)(int8_t)(hi >> (8 * b));
        o[b] = (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// Stage T q8_1 rows, elements [k0, k0+kt), into LDS.  `xrow(t)` -> pointer to
// the first block of activation row t.  All threads of the block call this.
// split = false: block_q8_1x {d, s, qs[32]} (40 B); the per-16 sums of SUM_GRAN 16 are
// recomputed from the quants.  split = true: block_q8_1s {d, s0, s1, pad, qs[32]} (48 B,
// include/ie/quant_blocks.hpp:174-181); the stored half sums are used as they are
// (src/ops/gemv_q8dot.cpp:483-597): per 16 they are the same numbers (s0 = d * float(sum of the
// half)); per 32 the sum s0 + s1 carries one more fp32 rounding than d * float(sum32).
struct NoHook {
    __device__ __forceinline__ void operator()() const {}
};
// `between`: called once by every thread after its first round of activation loads has been requested and before they
// are written to LDS.  Loads return in order, so weight words requested there stay in flight while the tile is built
// (requested before the activation loads, the tile would wait for them too).
template <int SUM_GRAN, int T, class RowFn, class Hook = NoHook>
__device__ __forceinline__ ActTile stage_act(uint8_t* lds, RowFn xrow, uint32_t k0, uint32_t kt, uint32_t KT_alloc, bool split = false,
                                             Hook between = Hook()) {
    uint4* qs = reinterpret_cast<uint4*>(lds);
    if constexpr (SUM_GRAN == 2) {
        // MXFP4: the matching weights are converted by v_cvt_scalef32_pk_f16_fp4, one byte (elements j and j + 16 of a
        // block) -> one fp16 pair, and summed by v_dot2_f32_f16; so the quants are staged as fp16 pairs
        // {x[j], x[j + 16]}, j = 0..15 per block (four 16-byte chunks), exact integers.
        uint8_t* hdr2 = lds + (size_t)T * KT_alloc * 2;
        const uint32_t blocks = (kt + 63) / 64 * 2;   // padded to whole 64-element units with zeros
        bool hooked2 = false;
        for (uint32_t i = threadIdx.x; i < (uint32_t)T * blocks; i += blockDim.x) {
            const uint32_t t = i / blocks, b = i - t * blocks;
            uint2 q[4] = {make_uint2(0, 0), make_uint2(0, 0), make_uint2(0, 0), make_uint2(0, 0)};
            float d = 0.f;
            if (b * 32 < kt) {
                const uint8_t* blk = xrow(t) + (size_t)(k0 / 32 + b) * (split ? kQ81sBytes : kQ81xBytes);
                const uint2* p = reinterpret_cast<const uint2*>(blk + (split ? 16 : 8));
#pragma unroll
                for (int j = 0; j < 4; ++j) q[j] = p[j];
                d = *reinterpret_cast<const float*>(blk);
            }
            if (!hooked2) {
                between();
                __builtin_amdgcn_sched_barrier(0);
                hooked2 = true;
            }
            const uint32_t lo[4] = {q[0].x, q[0].y, q[1].x, q[1].y}, hi[4] = {q[2].x, q[2].y, q[3].x, q[3].y};
#pragma unroll
            for (uint32_t c = 0; c < 4; ++c) qs[(size_t)t * (KT_alloc / 8) + act_slot<2>(4u * b + c)] = q8_pairs_f16(lo[c], hi[c]);
            reinterpret_cast<float*>(hdr2)[(size_t)t * (KT_alloc / 32) + b] = d;
        }
        if (!hooked2) between();
        return ActTile{qs, hdr2, KT_alloc};
    }
    uint8_t* hdr = lds + (size_t)T * KT_alloc;
    const uint32_t halves = (kt + 63) / 64 * 4;   // padded to whole 64-element units with zeros
    bool hooked = false;
    for (uint32_t i = threadIdx.x; i < (uint32_t)T * halves; i += blockDim.x) {
        const uint32_t t = i / halves, hb = i - t * halves;
        uint2 q0 = make_uint2(0, 0), q1 = q0;
        float2 ds = make_float2(0.f, 0.f);                          // {d, s = d * sum32}
        float s_half = 0.f;                                         // split: stored d * sum16 of this half
        if (hb * 16 < kt) {
            const uint8_t* blk = xrow(t) + (size_t)(k0 / 32 + (hb >> 1)) * (split ? kQ81sBytes : kQ81xBytes);
            const uint2* q = reinterpret_cast<const uint2*>(blk + (split ? 16 : 8) + (hb & 1u) * 16u);
            q0 = q[0];
            q1 = q[1];
            if (split) {
                const float4 h = *reinterpret_cast<const float4*>(blk);
                ds = make_float2(h.x, h.y + h.z);
                s_half = (hb & 1u) ? h.z : h.y;
            } else {
                ds = *reinterpret_cast<const float2*>(blk);
            }
        }
        if (!hooked) {
            between();
            __builtin_amdgcn_sched_barrier(0);
            hooked = true;
        }
        qs[(size_t)t * (KT_alloc / 16) + act_slot<SUM_GRAN>(hb)] = make_uint4(q0.x, q0.y, q1.x, q1.y);
        if (SUM_GRAN == 16) {
            float sh = s_half;
            if (!split) {
                int s = dot4(0x01010101u, q0.x, 0);
                s = dot4(0x01010101u, q0.y, s);
                s = dot4(0x01010101u, q1.x, s);
                s = dot4(0x01010101u, q1.y, s);
                sh = ds.x * (float)s;
            }
            reinterpret_cast<float2*>(hdr)[(size_t)t * (KT_alloc / 16) + hb] = make_float2(ds.x, sh);
        } else if ((hb & 1u) == 0) {
            if (SUM_GRAN == 32)
                reinterpret_cast<float2*>(hdr)[(size_t)t * (KT_alloc / 32) + (hb >> 1)] = ds;
            else
                reinterpret_cast<float*>(hdr)[(size_t)t * (KT_alloc / 32) + (hb >> 1)] = ds.x;
        }
    }
    if (!hooked) between();
    return ActTile{qs, hdr, KT_alloc};
}

// The same tile from fp16 rows, quantized on the way in: d = amax/127, q = round-half-away(v * 127/amax),
// s = d * float(sum q) per 32-element block, exactly quantize_q8_1 (src/ops/gemv_q8dot.cpp:94-124), so the
// staged tile is bit-identical to staging the quantizer's output.  A thread takes 16 elements; the two
// threads of a block (adjacent lanes) exchange their maxima and sums.  `hrow(t)` -> first element of row t.
template <int SUM_GRAN, int T, class RowFn, class Hook = NoHook>
__device__ __forceinline__ ActTile stage_act_f16(uint8_t* lds, RowFn hrow, uint32_t k0, uint32_t kt, uint32_t KT_alloc, Hook between = Hook()) {
    uint4* qs = reinterpret_cast<uint4*>(lds);
    uint8_t* hdr = lds + (size_t)T * KT_alloc;
    const uint32_t halves = (kt + 63) / 64 * 4;
    const uint32_t total = (uint32_t)T * halves, total_up = (total + blockDim.x - 1) / blockDim.x * blockDim.x;
    bool hooked = false;
    for (uint32_t i = threadIdx.x; i < total_up; i += blockDim.x) {   // whole passes: both threads of a block stay converged
        const bool in = i < total;
        const uint32_t t = in ? i / halves : 0, hb = in ? i - t * halves : 0;
        const bool live = in && hb * 16 < kt;
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = 0.f;
        uint4 a = make_uint4(0, 0, 0, 0), b = a;
        if (live) {
            const half_t* p = hrow(t) + k0 + hb * 16;
            a = reinterpret_cast<const uint4*>(p)[0];
            b = reinterpret_cast<const uint4*>(p)[1];
        }
        if (!hooked) {   // as in stage_act: behind the first pass's activation loads, in front of their use
            between();
            __builtin_amdgcn_sched_barrier(0);
            hooked = true;
        }
        if (live) {
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                v[2 * j] = h2f(w[j] & 0xFFFFu);
                v[2 * j + 1] = h2f(w[j] >> 16);
            }
        }
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(v[j]));
        amax = fmaxf(amax, __shfl_xor(amax, 1));
        const float d = amax / 127.0f, inv = amax > 0.f ? 127.0f / amax : 0.f;
        uint32_t q[4];
        int s16 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t pk = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int qi = (int)roundf(v[4 * j + b] * inv);
                s16 += qi;
                pk |= (uint32_t)(qi & 0xFF) << (8 * b);
            }
            q[j] = pk;
        }
        const int s32 = s16 + __shfl_xor(s16, 1);
        if constexpr (SUM_GRAN == 2) {
            // fp16 pairs {x[j], x[j + 16]}: the other half of the block sits in the neighbouring lane; the thread of the
            // first half writes pairs 0..7, the other one pairs 8..15
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (uint32_t)__shfl_xor((int)q[j], 1);
            if (!in) continue;
            const bool second = (hb & 1u) != 0;
            const uint32_t b = hb >> 1, c0 = second ? 2u : 0u;
            uint4* row = qs + (size_t)t * (KT_alloc / 8);
            row[act_slot<2>(4u * b + c0)] = second ? q8_pairs_f16(o[2], q[2]) : q8_pairs_f16(q[0], o[0]);
            row[act_slot<2>(4u * b + c0 + 1u)] = second ? q8_pairs_f16(o[3], q[3]) : q8_pairs_f16(q[1], o[1]);
            if (!second) reinterpret_cast<float*>(lds + (size_t)T * KT_alloc * 2)[(size_t)t * (KT_alloc / 32) + b] = d;
            continue;
        }
        if (!in) continue;
        qs[(size_t)t * (KT_alloc / 16) + act_slot<SUM_GRAN>(hb)] = make_uint4(q[0], q[1], q[2], q[3]);
        if (SUM_GRAN == 16) {
            reinterpret_cast<float2*>(hdr)[(size_t)t * (KT_alloc / 16) + hb] = make_float2(d, d * (float)s16);
        } else if ((hb & 1u) == 0) {
            if (SUM_GRAN == 32)
                reinterpret_cast<float2*>(hdr)[(size_t)t * (KT_alloc / 32) + (hb >> 1)] = make_float2(d, d * (float)s32);
            else
                reinterpret_cast<float*>(hdr)[(size_t)t * (KT_alloc / 32) + (hb >> 1)] = d;
        }
    }
    if constexpr (SUM_GRAN == 2) return ActTile{qs, lds + (size_t)T * KT_alloc * 2, KT_alloc};
    return ActTile{qs, hdr, KT_alloc};
}

__device__ __forceinline__ int dot16(const uint32_t (&w)[4], const uint4& x, int c) {
    c = dot4(w[0], x.x, c);
    c = dot4(w[1], x.y, c);
    c = dot4(w[2], x.z, c);
    return dot4(w[3], x.w, c);
}

// One step of the unit walk: R decoded units (one per row, same tile-local unit
// `ul`) against the T staged activation rows.
template <class F, int T, int R>
__device__ __forceinline__ void gemv_step(const typename F::Raw (&raw)[R], const typename F::Cursor (&cu)[R], uint32_t ul,
                                          const ActTile& act, float (&acc)[R][T]) {
    if constexpr (F::SUM_GRAN == 2) {
        // MXFP4 against fp16-pair activations: one v_cvt_scalef32_pk_f16_fp4 per weight byte (scale 2: the doubled E2M1
        // values 0..12, integers) and one v_dot2_f32_f16 per pair.  Every product and partial sum is an integer below
        // 2^24, so the fp32 sum equals the int8 dot of the other formats exactly and the fold is the same expression.
        typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
        const uint32_t e0 = F::elem_off(ul);
        uint32_t w[R][8];
        float c[R][2];
#pragma unroll
        for (int r = 0; r < R; ++r) F::fp4(raw[r], w[r], c[r]);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint4 x[8];
#pragma unroll
            for (uint32_t k = 0; k < 8; ++k) x[k] = act.qs[(size_t)t * (act.KT / 8) + act_slot<2>((e0 >> 3) + k)];
            const float* h = reinterpret_cast<const float*>(act.hdr) + (size_t)t * (act.KT / 32) + (e0 >> 5);
            const float d0 = h[0], d1 = h[1];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float f[2] = {0.f, 0.f};
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t ww = w[r][4 * b + k];
                        const uint4& xx = x[4 * b + k];
                        f[b] = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(ww, 2.0f, 0), __builtin_bit_cast(h2_t, xx.x), f[b], false);
                        f[b] = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(ww, 2.0f, 1), __builtin_bit_cast(h2_t, xx.y), f[b], false);
                        f[b] = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(ww, 2.0f, 2), __builtin_bit_cast(h2_t, xx.z), f[b], false);
                        f[b] = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(ww, 2.0f, 3), __builtin_bit_cast(h2_t, xx.w), f[b], false);
                    }
                acc[r][t] += c[r][0] * (d0 * f[0]) + c[r][1] * (d1 * f[1]);
            }
        }
        return;
    }
    Unit un[R];
#pragma unroll
    for (int r = 0; r < R; ++r) F::decode(raw[r], cu[r], un[r]);
    const uint32_t e0 = F::elem_off(ul);
#pragma unroll
    for (int t = 0; t < T; ++t) {
        uint4 x[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) x[g] = act.qs[(size_t)t * (act.KT / 16) + act_slot<F::SUM_GRAN>((e0 + g * F::GROUP_OFF) >> 4)];
        if (F::PAIRED) {
            // groups (0,1) and (2,3): one activation block and one weight scale each
            float d0, d1, s0 = 0.f, s1 = 0.f;
            if (F::SUM_GRAN == 32) {
                const float2* h = reinterpret_cast<const float2*>(act.hdr) + (size_t)t * (act.KT / 32) + (e0 >> 5);
                const float2 h0 = h[0], h1 = h[1];
                d0 = h0.x; s0 = h0.y; d1 = h1.x; s1 = h1.y;
            } else {
                const float* h = reinterpret_cast<const float*>(act.hdr) + (size_t)t * (act.KT / 32) + (e0 >> 5);
                d0 = h[0]; d1 = h[1];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int i0 = dot16(un[r].q[1], x[1], dot16(un[r].q[0], x[0], 0));
                const int i1 = dot16(un[r].q[3], x[3], dot16(un[r].q[2], x[2], 0));
                float v = un[r].c[0] * (d0 * (float)i0) + un[r].c[2] * (d1 * (float)i1);
                if (F::SUM_GRAN == 32) v -= un[r].m[0] * s0 + un[r].m[2] * s1;
                acc[r][t] += v;
            }
        } else if (F::SUM_GRAN == 0) {
            // four groups in four activation blocks, no min term: one scale pair per group
            float d8[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) d8[g] = reinterpret_cast<const float*>(act.hdr)[(size_t)t * (act.KT / 32) + ((e0 + g * F::GROUP_OFF) >> 5)];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float v = 0.f;
#pragma unroll
                for (int g = 0; g < 4; ++g) v += un[r].c[g] * (d8[g] * (float)dot16(un[r].q[g], x[g], 0));
                acc[r][t] += v;
            }
        } else {
            float2 h[4];
#pragma unroll
            for (int g = 0; g < 4; ++g)
                h[g] = reinterpret_cast<const float2*>(act.hdr)[(size_t)t * (act.KT / 16) + ((e0 + g * F::GROUP_OFF) >> 4)];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float v = 0.f;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ig = dot16(un[r].q[g], x[g], 0);
                    v += un[r].c[g] * (h[g].x * (float)ig) - un[r].m[g] * h[g].y;
                }
                acc[r][t] += v;
            }
        }
    }
}

// Walk one K-tile for R rows: lane `gl` of a G-lane group handles tile-local
// units gl, gl+G, ...  Full iterations (every lane live) run U at a time with
// all U*R loads issued before the first use; the ragged rest is predicated.
// cu[r] must point at unit (tile_first_unit + gl) of row r.  `n_units` counts
// 64-element units including a trailing half unit (`half_tail`: K % 64 == 32).
// `pre` (optional): the U*R units of the first full iteration, already requested by the caller (before it staged
// the activations, say); only used when there is a full iteration (n_whole / G >= U).
template <class F, int T, int R, int G, int U>
__device__ __forceinline__ void gemv_rows(const typename F::Cursor (&cu)[R], uint32_t n_units, bool half_tail, uint32_t gl,
                                          const ActTile& act, float (&acc)[R][T], const typename F::Raw (*pre)[R] = nullptr) {
    const uint32_t n_whole = half_tail ? n_units - 1 : n_units;
    const uint32_t full = n_whole / G;
    uint32_t it = 0;
    if (pre && U <= full) {
#pragma unroll
        for (int u = 0; u < U; ++u) gemv_step<F, T, R>(pre[u], cu, gl + u * G, act, acc);
        it = U;
    }
    for (; it + U <= full; it += U) {
        typename F::Raw raw[U][R];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r) raw[u][r] = load_unit<F, G>(cu[r], it + u, false);
#pragma unroll
        for (int u = 0; u < U; ++u) gemv_step<F, T, R>(raw[u], cu, gl + (it + u) * G, act, acc);
    }
    for (; it * G + gl < n_units; ++it) {
        typename F::Raw raw[R];
        const bool half_only = half_tail && (it * G + gl == n_units - 1);
#pragma unroll
        for (int r = 0; r < R; ++r) raw[r] = load_unit<F, G>(cu[r], it, half_only);
        gemv_step<F, T, R>(raw, cu, gl + it * G, act, acc);
    }
}

// ---------------------------------------------------------------- float activations
// Activations staged in LDS as fp32 plus per-16 sums; one unit folds as the reference's
//   acc += (d*sc) * sum(a*q) - (dmin*m) * sum(a)      (src/ops/gemv_q4k.cpp:119-146).
template <bool UNSIGNED>
__device__ __forceinline__ float code_to_f(uint32_t w, int j) {
    if (UNSIGNED) return (float)((w >> (8 * j)) & 0xFFu);
    return (float)(int)(int8_t)(w >> (8 * j));
}

// kt activations from A (zero up to the next multiple of 64) -> xa[], sums of 16 -> s16[].
// One thread per 16 elements, fetched with 128-bit loads where the row allows it.
__device__ __forceinline__ void load16(const half_t* p, float (&v)[16]) {
    if ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
        const uint4 a = reinterpret_cast<const uint4*>(p)[0], b = reinterpret_cast<const uint4*>(p)[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            v[2 * j] = h2f(w[j] & 0xFFFFu);
            v[2 * j + 1] = h2f(w[j] >> 16);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = (float)p[j];
    }
}
__device__ __forceinline__ void load16(const float* p, float (&v)[16]) {
    if ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 f = reinterpret_cast<const float4*>(p)[j];
            v[4 * j] = f.x; v[4 * j + 1] = f.y; v[4 * j + 2] = f.z; v[4 * j + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = p[j];
    }
}
// The staged row is kept in 16-byte slots, slot q stored at q ^ ((q >> 4) & 15).  A lane's unit is 64 consecutive
// floats, so without the permutation the 64 lanes of a ds_read_b128 all fall on the same four banks (lane stride 256 B);
// with it the 16 lanes served together read 16 different slots (Q4_K-style units) or 8 (Q6_K's interleaved units).
__device__ __forceinline__ uint32_t fact_slot(uint32_t q) { return q ^ ((q >> 4) & 15u); }
template <class ActT>
__device__ __forceinline__ void stage_fact(float* xa, float* s16, const ActT* A, uint32_t kt) {
    for (uint32_t i = threadIdx.x; i < (kt + 63) / 64 * 4; i += blockDim.x) {
        float v[16];
        if (i * 16 < kt) {
            load16(A + i * 16, v);
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) v[j] = 0.f;
        }
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) s += v[j];
#pragma unroll
        for (int j = 0; j < 4; ++j) reinterpret_cast<float4*>(xa)[fact_slot(i * 4 + j)] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
        s16[i] = s;
    }
}

template <class F>
__device__ __forceinline__ float fact_unit(const typename F::Raw& raw, const typename F::Cursor& cu, const float* xa, const float* s16, uint32_t e0) {
    Unit un;
    F::decode(raw, cu, un);
    float v = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t eg = e0 + g * F::GROUP_OFF;
        float dq = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 x = reinterpret_cast<const float4*>(xa)[fact_slot((eg >> 2) + i)];
            dq += x.x * code_to_f<F::CODES_UNSIGNED>(un.q[g][i], 0) + x.y * code_to_f<F::CODES_UNSIGNED>(un.q[g][i], 1) +
                  x.z * code_to_f<F::CODES_UNSIGNED>(un.q[g][i], 2) + x.w * code_to_f<F::CODES_UNSIGNED>(un.q[g][i], 3);
        }
        v += un.c[g] * dq;
        if (F::SUM_GRAN != 0 && F::SUM_GRAN != 2) v -= un.m[g] * s16[eg >> 4];
    }
    return v;
}

}  // namespace mxq
