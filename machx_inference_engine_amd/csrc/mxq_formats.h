// mxq_formats.h — per-format "weight unit" decoders used by the GEMV kernels.
//
// A unit is the slice of one weight row that one lane handles per step: 32
// weights, delivered as two groups (A, B) of 16 int8 codes (4 dwords each) plus
// the fp32 coefficients of the fold
//     acc += ca * (d8[A] * idotA) - ma * s16[A] + cb * (d8[B] * idotB) - mb * s16[B]
// where idot = sum(code * q8), d8 = activation block scale, s16 = d8 * sum(q8)
// over the 16 activations of the group.  Consecutive units of a row are
// consecutive 16- or 32-byte chunks of the weight stream, so a wave's loads
// are fully coalesced 128-bit loads.
//
// Group A covers row elements [ea, ea+16), group B [ea + EB_OFF, +16) with
// ea = F::elem_off(u).
#pragma once

#include "mxq_device.h"

namespace mxq {

struct Unit {
    uint32_t a[4], b[4];
    float ca, ma, cb, mb;
};

// 128-bit load from a 2-byte aligned address (Q6_K and AoS Q8_0 blocks are only
// 2-byte aligned).  Global memory accepts unaligned vector loads on gfx950.
__device__ __forceinline__ uint4 load_u4_a2(const uint8_t* p) {
    struct __attribute__((packed, aligned(2))) U4 { uint32_t x, y, z, w; };
    const U4 v = *reinterpret_cast<const U4*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// ---------------------------------------------------------------- Q4_K (AoS GGUF blocks)
// Unit u = (block u/8, qs chunk c = u%8).  Chunk c holds qs[16c, 16c+16): low
// nibbles are elements 64g + 16h + [0,16) of sub-block 2g, high nibbles the same
// positions of sub-block 2g+1, g = c/2, h = c%2 (include/ie/dequant_ref.hpp:38-53).
struct FmtQ4K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Raw {
        uint4 qs, hdr;
    };
    static constexpr bool HAS_MIN = true;
    static constexpr uint32_t EB_OFF = 32;
    static constexpr uint32_t K_ALIGN = 256;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) {
        const uint32_t c = u & 7u;
        return (u >> 3) * 256u + (c >> 1) * 64u + (c & 1u) * 16u;
    }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t u) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)(u >> 3) * kQ4KBytes;
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qs = *reinterpret_cast<const uint4*>(blk + 16 + (u & 7u) * 16u);
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, uint32_t u, Unit& o) {
        const uint32_t q[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o.a[i] = q[i] & 0x0F0F0F0Fu;
            o.b[i] = (q[i] >> 4) & 0x0F0F0F0Fu;
        }
        uint32_t sc, mn;
        q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, (int)((u & 7u) >> 1), sc, mn);
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        o.ca = d * (float)(sc & 0xFFu);
        o.cb = d * (float)(sc >> 8);
        o.ma = dmin * (float)(mn & 0xFFu);
        o.mb = dmin * (float)(mn >> 8);
    }
};

// ---------------------------------------------------------------- Q6_K (AoS GGUF blocks)
// Unit u = (block u/8, ql chunk c = u%8), h = c/4, r = c%4.  Chunk c holds
// ql[16c, 16c+16) whose low nibbles are elements 128h + 32(r/2) + 16(r%2) + [0,16)
// and whose high nibbles are the elements 64 further on; the matching 2-bit
// planes sit in qh[32h + 16(r%2) + [0,16)] at bit 2(r/2) and 2(r/2)+4
// (include/ie/dequant_ref.hpp:78-96).  Codes are kept unsigned (0..63); the -32
// offset goes into the min term: ma = 32 * ca.
struct FmtQ6K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Raw {
        uint4 ql, qh;
        int sca, scb;
        uint32_t d;
    };
    static constexpr bool HAS_MIN = true;
    static constexpr uint32_t EB_OFF = 64;
    static constexpr uint32_t K_ALIGN = 256;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) {
        const uint32_t c = u & 7u;
        return (u >> 3) * 256u + (c >> 2) * 128u + ((c >> 1) & 1u) * 32u + (c & 1u) * 16u;
    }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t u) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)(u >> 3) * kQ6KBytes;
        const uint32_t c = u & 7u, h = c >> 2, r = c & 3u;
        Raw o;
        o.ql = load_u4_a2(blk + c * 16u);
        o.qh = load_u4_a2(blk + 128 + (h * 2u + (r & 1u)) * 16u);
        const int8_t* sc = reinterpret_cast<const int8_t*>(blk + 192 + h * 8u + (r >> 1) * 2u + (r & 1u));
        o.sca = sc[0];
        o.scb = sc[4];
        o.d = *reinterpret_cast<const uint16_t*>(blk + 208);
        return o;
    }
    __device__ static __forceinline__ void decode(const Raw& r, uint32_t u, Unit& o) {
        const uint32_t ql[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w}, qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        const uint32_t sh = ((u >> 1) & 1u) * 2u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t hsh = qh[i] >> sh;
            o.a[i] = (ql[i] & 0x0F0F0F0Fu) | ((hsh & 0x03030303u) << 4);
            o.b[i] = ((ql[i] >> 4) & 0x0F0F0F0Fu) | (hsh & 0x30303030u);
        }
        const float d = h2f(r.d);
        o.ca = d * (float)r.sca;
        o.cb = d * (float)r.scb;
        o.ma = 32.f * o.ca;
        o.mb = 32.f * o.cb;
    }
};

// ---------------------------------------------------------------- Q8_0, SoA planes
// qs[n*K + k] int8, d[n*(K/32) + b] fp16 bits (src/ops/gemv_q8dot.cpp:601-607).
// Unit u = block u: 32 bytes of qs, one scale.
struct FmtQ8Soa {
    struct W {
        const int8_t* qs;
        const uint16_t* d;
        uint32_t K;
    };
    struct Raw {
        uint4 lo, hi;
        uint32_t d;
    };
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t EB_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 32u; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t u) {
        const uint4* p = reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)u * 32u);
        Raw r;
        r.lo = p[0];
        r.hi = p[1];
        r.d = w.d[(size_t)n * (w.K >> 5) + u];
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, uint32_t, Unit& o) {
        o.a[0] = r.lo.x; o.a[1] = r.lo.y; o.a[2] = r.lo.z; o.a[3] = r.lo.w;
        o.b[0] = r.hi.x; o.b[1] = r.hi.y; o.b[2] = r.hi.z; o.b[3] = r.hi.w;
        o.ca = o.cb = h2f(r.d);
        o.ma = o.mb = 0.f;
    }
};

// ---------------------------------------------------------------- Q8_0, AoS GGUF blocks
// 34-byte blocks {fp16 d; int8 qs[32]}: one lane per block, quants read as two
// 128-bit loads at 2-byte alignment.
struct FmtQ8Aos {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    typedef FmtQ8Soa::Raw Raw;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t EB_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 32u; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t u) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)u * kQ8_0Bytes;
        Raw r;
        r.d = *reinterpret_cast<const uint16_t*>(blk);
        r.lo = load_u4_a2(blk + 2);
        r.hi = load_u4_a2(blk + 18);
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, uint32_t u, Unit& o) { FmtQ8Soa::decode(r, u, o); }
};

// ---------------------------------------------------------------- MXFP4, SoA planes
// qs_plane[n*(K/2) + 16b + j], e_plane[n*(K/32) + b] (src/ops/gemv_mxfp4.cpp:13-16).
// Unit u = block u: 16 bytes of codes (low nibbles = elements 0..15, high =
// 16..31), one E8M0 exponent.  Codes become doubled E2M1 values as int8; the
// block scale is 2^(e-128).
struct FmtMxfp4Soa {
    struct W {
        const uint8_t* qs;
        const uint8_t* e;
        uint32_t K;
    };
    struct Raw {
        uint4 qs;
        uint32_t e;
    };
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t EB_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 32u; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t u) {
        Raw r;
        r.qs = *reinterpret_cast<const uint4*>(w.qs + (size_t)n * (w.K >> 1) + (size_t)u * 16u);
        r.e = w.e[(size_t)n * (w.K >> 5) + u];
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, uint32_t, Unit& o) {
        mxfp4_decode_word(r.qs.x, o.a[0], o.b[0]);
        mxfp4_decode_word(r.qs.y, o.a[1], o.b[1]);
        mxfp4_decode_word(r.qs.z, o.a[2], o.b[2]);
        mxfp4_decode_word(r.qs.w, o.a[3], o.b[3]);
        o.ca = o.cb = e8m0_half(r.e);
        o.ma = o.mb = 0.f;
    }
};

}  // namespace mxq
