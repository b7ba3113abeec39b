// mxq_gemv_core.h — the bandwidth-bound int-dot GEMV core shared by the dense,
// fused gate/up and expert-indexed entry points.
//
// Work decomposition (wave64):
//   * a group of G lanes (G = 32 or 64) owns R consecutive weight rows; lane l of
//     the group walks units l, l+G, l+2G ... of each row, so one wave-wide load
//     instruction fetches 64 consecutive 16-byte chunks of a row (coalesced
//     128-bit loads of whole super-blocks);
//   * the T activation rows (block_q8_1x streams) are staged once per K-tile in
//     LDS as three planes — int8 quants, fp32 block scales, fp32 per-16 sums —
//     and every lane reads the 2 x 16 quants that face its unit with two
//     ds_read_b128;
//   * scale/min unpacking, the int8 dot (v_dot4_i32_i8) and the fp32 fold run in
//     registers; the per-row result is reduced across the group with DPP.
// No MFMA: at T <= 8 the kernel is a stream over the weight bytes.
#pragma once

#include "mxq_formats.h"

namespace mxq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;

// LDS footprint of one activation tile.
__host__ __device__ constexpr uint32_t act_tile_bytes(uint32_t T, uint32_t KT, bool has_min) {
    return T * (KT + KT / 8 + (has_min ? KT / 4 : 0));
}

template <bool HAS_MIN>
struct ActTile {
    const uint4* qs;    // [T][KT/16] 16-quant chunks
    const float* d8;    // [T][KT/32]
    const float* s16;   // [T][KT/16]   (HAS_MIN only)
    uint32_t KT;
};

// Stage T q8_1x rows, elements [k0, k0+kt), into LDS.  `xrow(t)` -> pointer to
// the first block of activation row t.  All threads of the block call this.
template <bool HAS_MIN, int T, class RowFn>
__device__ __forceinline__ ActTile<HAS_MIN> stage_act(uint8_t* lds, RowFn xrow, uint32_t k0, uint32_t kt, uint32_t KT_alloc) {
    uint4* qs = reinterpret_cast<uint4*>(lds);
    float* d8 = reinterpret_cast<float*>(lds + (size_t)T * KT_alloc);
    float* s16 = d8 + (size_t)T * (KT_alloc / 32);
    const uint32_t halves = kt / 16;
    for (uint32_t i = threadIdx.x; i < (uint32_t)T * halves; i += blockDim.x) {
        const uint32_t t = i / halves, hb = i - t * halves;
        const uint8_t* blk = xrow(t) + (size_t)(k0 / 32 + (hb >> 1)) * kQ81xBytes;
        const uint2* q = reinterpret_cast<const uint2*>(blk + 8 + (hb & 1u) * 16u);
        const uint2 q0 = q[0], q1 = q[1];
        const float d = *reinterpret_cast<const float*>(blk);
        qs[(size_t)t * (KT_alloc / 16) + hb] = make_uint4(q0.x, q0.y, q1.x, q1.y);
        if ((hb & 1u) == 0) d8[(size_t)t * (KT_alloc / 32) + (hb >> 1)] = d;
        if (HAS_MIN) {
            int s = dot4(0x01010101u, q0.x, 0);
            s = dot4(0x01010101u, q0.y, s);
            s = dot4(0x01010101u, q1.x, s);
            s = dot4(0x01010101u, q1.y, s);
            s16[(size_t)t * (KT_alloc / 16) + hb] = d * (float)s;
        }
    }
    ActTile<HAS_MIN> a;
    a.qs = qs;
    a.d8 = d8;
    a.s16 = s16;
    a.KT = KT_alloc;
    return a;
}

// Accumulate one K-tile: units [u0, u0 + n_units) of rows `rows[r]` against the
// staged activations.  `gl` = lane index inside its G-lane group.
template <class F, int T, int R, int G>
__device__ __forceinline__ void gemv_tile(const typename F::W& w, const uint32_t (&rows)[R], uint32_t u0, uint32_t n_units,
                                          uint32_t gl, const ActTile<F::HAS_MIN>& act, float (&acc)[R][T]) {
    for (uint32_t ul = gl; ul < n_units; ul += G) {
        typename F::Raw raw[R];
#pragma unroll
        for (int r = 0; r < R; ++r) raw[r] = F::load(w, rows[r], u0 + ul);
        Unit un[R];
#pragma unroll
        for (int r = 0; r < R; ++r) F::decode(raw[r], u0 + ul, un[r]);
        const uint32_t ea = F::elem_off(ul), eb = ea + F::EB_OFF;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const uint4 xa = act.qs[(size_t)t * (act.KT / 16) + (ea >> 4)];
            const uint4 xb = act.qs[(size_t)t * (act.KT / 16) + (eb >> 4)];
            const float da = act.d8[(size_t)t * (act.KT / 32) + (ea >> 5)];
            const float db = act.d8[(size_t)t * (act.KT / 32) + (eb >> 5)];
            float sa = 0.f, sb = 0.f;
            if (F::HAS_MIN) {
                sa = act.s16[(size_t)t * (act.KT / 16) + (ea >> 4)];
                sb = act.s16[(size_t)t * (act.KT / 16) + (eb >> 4)];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                int ia = dot4(un[r].a[0], xa.x, 0);
                ia = dot4(un[r].a[1], xa.y, ia);
                ia = dot4(un[r].a[2], xa.z, ia);
                ia = dot4(un[r].a[3], xa.w, ia);
                int ib = dot4(un[r].b[0], xb.x, 0);
                ib = dot4(un[r].b[1], xb.y, ib);
                ib = dot4(un[r].b[2], xb.z, ib);
                ib = dot4(un[r].b[3], xb.w, ib);
                float v = un[r].ca * (da * (float)ia) + un[r].cb * (db * (float)ib);
                if (F::HAS_MIN) v -= un[r].ma * sa + un[r].mb * sb;
                acc[r][t] += v;
            }
        }
    }
}

}  // namespace mxq
