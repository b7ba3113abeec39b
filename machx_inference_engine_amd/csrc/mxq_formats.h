// mxq_formats.h — per-format "weight unit" decoders used by the GEMV kernels.
//
// A unit is the slice of one weight row that one lane handles per step: 64
// weights, delivered as four groups of 16 int8 codes (4 dwords each) plus the
// fp32 coefficients of the fold
//     acc += sum_g  c[g] * (d8[g] * idot[g]) - m[g] * s[g]
// where idot[g] = sum(code * q8) over the group, d8 = scale of the activation
// block the group lies in and s = d8 * sum(q8) over the group (the min / offset
// term of the K-quants).  Group g covers row elements
// [elem_off(u) + GROUP_OFF * g, +16).  Consecutive units of a row are
// consecutive chunks of the weight stream, so a wave's loads are coalesced
// 128-bit loads of whole super-blocks, and a block header is unpacked by four
// lanes only.
//
// PAIRED formats: groups (0,1) lie in one 32-element activation block and share
// one weight scale, likewise (2,3); their integer dots are accumulated in one
// chain and folded once.
//
// Addressing: a lane that walks units u, u+G, u+2G ... of a row keeps a Cursor
// (the address of its first unit); step i of the walk loads at
// cursor + i * G * bytes-per-unit, a compile-time offset in unrolled code.  The
// position of a unit inside its 256-element super-block (u % 4) is the same for
// every step of a lane because G is a multiple of 4.
#pragma once

#include "mxq_device.h"

namespace mxq {

struct Unit {
    uint32_t q[4][4];
    float c[4], m[4];
};

// Loads from 2-byte aligned addresses (Q6_K and AoS Q8_0 blocks are only 2-byte
// aligned).  Global memory accepts unaligned vector loads on gfx950.
__device__ __forceinline__ uint4 load_u4_a2(const uint8_t* p) {
    struct __attribute__((packed, aligned(2))) U4 { uint32_t x, y, z, w; };
    const U4 v = *reinterpret_cast<const U4*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_u2_a2(const uint8_t* p) {
    struct __attribute__((packed, aligned(2))) U2 { uint32_t x, y; };
    const U2 v = *reinterpret_cast<const U2*>(p);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t load_u1_a2(const uint8_t* p) {
    struct __attribute__((packed, aligned(2))) U1 { uint32_t x; };
    return reinterpret_cast<const U1*>(p)->x;
}

// A 16-byte load with the non-temporal hint, for weight words that one load instruction of a wave consumes whole cache
// lines of (a line that several instructions touch is fetched again by each of them under this hint).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_u4_stream(const void* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// ---------------------------------------------------------------- Q4_K (AoS GGUF blocks)
// Unit u = (block u/4, 64-element group g = u%4): the 32 bytes qs[32g, 32g+32),
// whose low nibbles are sub-block 2g and high nibbles sub-block 2g+1
// (include/ie/dequant_ref.hpp:38-53).  Groups: 0,1 = sub-block 2g (elements
// 0..15, 16..31), 2,3 = sub-block 2g+1.
struct FmtQ4K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Cursor {
        const uint8_t* blk;   // block of the lane's first unit
        uint32_t g;
    };
    struct Raw {
        uint4 hdr, q0, q1;
    };
    // expert bank: expert e at base + e * expert_stride_bytes (include/ie/ops.hpp:1027-1029)
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint32_t row_bytes;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.base + (size_t)e * b.expert_stride_bytes, b.row_bytes}; }
    static Bank bank(const void* base, uint64_t stride, uint32_t K, uint32_t) { return {static_cast<const uint8_t*>(base), stride, K / 256 * (uint32_t)kQ4KBytes}; }
    static constexpr uint32_t W_ALIGN = 16;
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {w.base + (size_t)n * w.row_bytes + (size_t)(u >> 2) * kQ4KBytes, u & 3u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const uint8_t* blk = cu.blk + (size_t)i * (G / 4 * kQ4KBytes);
        const uint4* q = reinterpret_cast<const uint4*>(blk + 16 + cu.g * 32u);
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) {
        const uint32_t q0[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w}, q1[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o.q[0][i] = q0[i] & 0x0F0F0F0Fu;
            o.q[1][i] = q1[i] & 0x0F0F0F0Fu;
            o.q[2][i] = (q0[i] >> 4) & 0x0F0F0F0Fu;
            o.q[3][i] = (q1[i] >> 4) & 0x0F0F0F0Fu;
        }
        uint32_t sc, mn;
        q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, (int)cu.g, sc, mn);
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        o.c[0] = o.c[1] = d * (float)(sc & 0xFFu);
        o.c[2] = o.c[3] = d * (float)(sc >> 8);
        o.m[0] = o.m[1] = dmin * (float)(mn & 0xFFu);
        o.m[2] = o.m[3] = dmin * (float)(mn >> 8);
    }
};

// ---------------------------------------------------------------- Q6_K (AoS GGUF blocks)
// Unit u = (block u/4, half h = (u/2)%2, j = u%2): ql[64h + 16j + [0,16)] (subs 0
// and 2 in its low / high nibbles), ql[64h + 32 + 16j + [0,16)] (subs 1 and 3) and
// qh[32h + 16j + [0,16)] whose four 2-bit fields are the high bits of subs 0..3
// (include/ie/dequant_ref.hpp:78-96).  Group s = sub s: elements
// 128h + 32s + 16j + [0,16), per-16 scale scales[8h + 2s + j].  Codes stay
// unsigned (0..63); the -32 offset goes into the min term: m = 32 * c.
struct FmtQ6K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Cursor {
        const uint8_t* blk;
        uint32_t hj;          // 2h + j
    };
    struct Raw {
        uint4 qla, qlb, qh;
        uint2 sc;             // scales[8h .. 8h+8)
        uint32_t d;
    };
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint32_t row_bytes;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.base + (size_t)e * b.expert_stride_bytes, b.row_bytes}; }
    static Bank bank(const void* base, uint64_t stride, uint32_t K, uint32_t) { return {static_cast<const uint8_t*>(base), stride, K / 256 * (uint32_t)kQ6KBytes}; }
    static constexpr uint32_t W_ALIGN = 2;
    static constexpr int SUM_GRAN = 16;
    static constexpr bool PAIRED = false;
    static constexpr uint32_t GROUP_OFF = 32;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) {
        return (u >> 2) * 256u + ((u >> 1) & 1u) * 128u + (u & 1u) * 16u;
    }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {w.base + (size_t)n * w.row_bytes + (size_t)(u >> 2) * kQ6KBytes, u & 3u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const uint8_t* blk = cu.blk + (size_t)i * (G / 4 * kQ6KBytes);
        const uint32_t h = cu.hj >> 1, j = cu.hj & 1u;
        Raw o;
        o.qla = load_u4_a2(blk + 64u * h + 16u * j);
        o.qlb = load_u4_a2(blk + 64u * h + 32u + 16u * j);
        o.qh = load_u4_a2(blk + 128 + 32u * h + 16u * j);
        o.sc = load_u2_a2(blk + 192 + 8u * h);
        o.d = *reinterpret_cast<const uint16_t*>(blk + 208);
        return o;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) {
        const uint32_t la[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w}, lb[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w};
        const uint32_t qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o.q[0][i] = (la[i] & 0x0F0F0F0Fu) | ((qh[i] << 4) & 0x30303030u);
            o.q[1][i] = (lb[i] & 0x0F0F0F0Fu) | ((qh[i] << 2) & 0x30303030u);
            o.q[2][i] = ((la[i] >> 4) & 0x0F0F0F0Fu) | (qh[i] & 0x30303030u);
            o.q[3][i] = ((lb[i] >> 4) & 0x0F0F0F0Fu) | ((qh[i] >> 2) & 0x30303030u);
        }
        const float d = h2f(r.d);
        const uint32_t j8 = (cu.hj & 1u) * 8u;   // scale of sub s = byte 2s + j of sc
        o.c[0] = d * (float)(int)(int8_t)(r.sc.x >> j8);
        o.c[1] = d * (float)(int)(int8_t)(r.sc.x >> (16u + j8));
        o.c[2] = d * (float)(int)(int8_t)(r.sc.y >> j8);
        o.c[3] = d * (float)(int)(int8_t)(r.sc.y >> (16u + j8));
#pragma unroll
        for (int g = 0; g < 4; ++g) o.m[g] = 32.f * o.c[g];
    }
};

// ---------------------------------------------------------------- Q4_K, per-region streams
// The blocks of one matrix (or of one expert region) split into three streams of the same
// bytes:  qs[128] x nb | scales[12] x nb | {d,dmin}[4] x nb,  nb = N * K/256
// (repack_q4_K_to_reorder, src/ops/gemv_q8dot.cpp:134-147; per expert region
// repack_moe_q4k_soa_host, include/ie/quant_soa.hpp:33-41,127-141).  Same units, same decode as
// the AoS form; only the load addresses differ.
struct FmtQ4KStr {
    struct W {
        const uint8_t* qs;
        const uint8_t* sc;
        const uint8_t* dm;
        uint32_t bpr;         // blocks per row
    };
    struct Cursor {
        const uint8_t* qs;    // the unit's 32 bytes of the lane's first block
        const uint8_t* sc;
        const uint8_t* dm;
        uint32_t g;
    };
    typedef FmtQ4K::Raw Raw;
    // expert e: region at base + e * expert_stride_bytes holding nb blocks as three streams
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint64_t nb;
        uint32_t bpr;
    };
    __host__ __device__ static __forceinline__ W view(const uint8_t* p, uint64_t nb, uint32_t bpr) { return {p, p + nb * 128u, p + nb * 140u, bpr}; }
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return view(b.base + (size_t)e * b.expert_stride_bytes, b.nb, b.bpr); }
    static Bank bank(const void* base, uint64_t stride, uint32_t K, uint32_t N) {
        return {static_cast<const uint8_t*>(base), stride, (uint64_t)N * (K / 256), K / 256};
    }
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    static constexpr uint32_t W_ALIGN = 16;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        const size_t ib = (size_t)n * w.bpr + (u >> 2);
        return {w.qs + ib * 128u + (u & 3u) * 32u, w.sc + ib * 12u, w.dm + ib * 4u, u & 3u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const size_t step = (size_t)i * (G / 4);
        const uint4* q = reinterpret_cast<const uint4*>(cu.qs + step * 128u);
        const uint32_t* sc = reinterpret_cast<const uint32_t*>(cu.sc + step * 12u);
        Raw r;
        r.hdr = make_uint4(*reinterpret_cast<const uint32_t*>(cu.dm + step * 4u), sc[0], sc[1], sc[2]);
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) { FmtQ4K::decode(r, FmtQ4K::Cursor{nullptr, cu.g}, o); }
};

// ---------------------------------------------------------------- Q6_K, per-region streams
// ql[128] x nb | qh[64] x nb | scales[16] x nb | d[2] x nb  (repack_moe_q6k_soa_host,
// include/ie/quant_soa.hpp:43-51,143-157).  Units and decode as FmtQ6K.
struct FmtQ6KStr {
    struct W {
        const uint8_t* ql;
        const uint8_t* qh;
        const uint8_t* sc;
        const uint8_t* d;
        uint32_t bpr;
    };
    struct Cursor {
        const uint8_t* ql;    // + 64h + 16j of the lane's first block
        const uint8_t* qh;    // + 32h + 16j
        const uint8_t* sc;    // + 8h
        const uint8_t* d;
        uint32_t hj;
    };
    typedef FmtQ6K::Raw Raw;
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint64_t nb;
        uint32_t bpr;
    };
    __host__ __device__ static __forceinline__ W view(const uint8_t* p, uint64_t nb, uint32_t bpr) {
        return {p, p + nb * 128u, p + nb * 192u, p + nb * 208u, bpr};
    }
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return view(b.base + (size_t)e * b.expert_stride_bytes, b.nb, b.bpr); }
    static Bank bank(const void* base, uint64_t stride, uint32_t K, uint32_t N) {
        return {static_cast<const uint8_t*>(base), stride, (uint64_t)N * (K / 256), K / 256};
    }
    static constexpr int SUM_GRAN = 16;
    static constexpr bool PAIRED = false;
    static constexpr uint32_t GROUP_OFF = 32;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    static constexpr uint32_t W_ALIGN = 2;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return FmtQ6K::elem_off(u); }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        const size_t ib = (size_t)n * w.bpr + (u >> 2);
        const uint32_t h = (u >> 1) & 1u, j = u & 1u;
        return {w.ql + ib * 128u + 64u * h + 16u * j, w.qh + ib * 64u + 32u * h + 16u * j, w.sc + ib * 16u + 8u * h, w.d + ib * 2u, u & 3u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const size_t step = (size_t)i * (G / 4);
        Raw o;
        o.qla = load_u4_a2(cu.ql + step * 128u);
        o.qlb = load_u4_a2(cu.ql + step * 128u + 32u);
        o.qh = load_u4_a2(cu.qh + step * 64u);
        o.sc = load_u2_a2(cu.sc + step * 16u);
        o.d = *reinterpret_cast<const uint16_t*>(cu.d + step * 2u);
        return o;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) { FmtQ6K::decode(r, FmtQ6K::Cursor{nullptr, cu.hj}, o); }
};

// ---------------------------------------------------------------- natural-order planes
// Eight natural-order nibbles of one dword -> two dwords of byte codes in element order.
__device__ __forceinline__ void nibbles_to_codes(uint32_t x, uint32_t& a, uint32_t& b) {
    const uint32_t ev = x & 0x0F0F0F0Fu, od = (x >> 4) & 0x0F0F0F0Fu;   // elements 0,2,4,6 / 1,3,5,7
    a = __builtin_amdgcn_perm(od, ev, 0x05010400u);                      // elements 0,1,2,3
    b = __builtin_amdgcn_perm(od, ev, 0x07030602u);                      // elements 4,5,6,7
}

// Q4_K repacked per row into natural element order (repack_q4_K_to_soa, src/ops/gemv_q4_soa.cpp:18-28,
// 115-151): q[n*(K/2) + k/2] nibble (k&1), per-32 unpacked 6-bit scale / min as int8, per-256 fp16
// d / dmin.  Unit u = elements [64u, 64u+64): 32 bytes of nibbles, two (scale, min) pairs.
struct FmtQ4KNat {
    struct W {
        const uint8_t* q;
        const int8_t* sc;
        const int8_t* mn;
        const uint16_t* d;
        const uint16_t* dmin;
        uint32_t K;
    };
    struct Cursor {
        const uint8_t* q;
        const uint8_t* sc;
        const uint8_t* mn;
        const uint8_t* d;
        const uint8_t* dmin;
    };
    struct Raw {
        uint4 q0, q1;
        uint32_t sc2, mn2, d, dmin;
    };
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        const size_t sb = (size_t)n * (w.K >> 5) + 2u * u, bb = (size_t)n * (w.K >> 8) + (u >> 2);
        return {w.q + (size_t)n * (w.K >> 1) + (size_t)u * 32u, reinterpret_cast<const uint8_t*>(w.sc + sb), reinterpret_cast<const uint8_t*>(w.mn + sb),
                reinterpret_cast<const uint8_t*>(w.d + bb), reinterpret_cast<const uint8_t*>(w.dmin + bb)};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const uint4* q = reinterpret_cast<const uint4*>(cu.q + (size_t)i * (G * 32));
        Raw r;
        r.q0 = q[0];
        r.q1 = q[1];
        r.sc2 = *reinterpret_cast<const uint16_t*>(cu.sc + (size_t)i * (G * 2));
        r.mn2 = *reinterpret_cast<const uint16_t*>(cu.mn + (size_t)i * (G * 2));
        r.d = *reinterpret_cast<const uint16_t*>(cu.d + (size_t)i * (G / 4 * 2));
        r.dmin = *reinterpret_cast<const uint16_t*>(cu.dmin + (size_t)i * (G / 4 * 2));
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
        const uint32_t w[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            nibbles_to_codes(w[2 * g], o.q[g][0], o.q[g][1]);
            nibbles_to_codes(w[2 * g + 1], o.q[g][2], o.q[g][3]);
        }
        const float d = h2f(r.d), dmin = h2f(r.dmin);
        o.c[0] = o.c[1] = d * (float)(r.sc2 & 0xFFu);
        o.c[2] = o.c[3] = d * (float)(r.sc2 >> 8);
        o.m[0] = o.m[1] = dmin * (float)(r.mn2 & 0xFFu);
        o.m[2] = o.m[3] = dmin * (float)(r.mn2 >> 8);
    }
};

// Q6_K repacked per row into natural element order (repack_q6_K_to_soa, src/ops/gemv_q6_soa.cpp:62-126):
// lo[n*(K/2) + k/2] nibble (k&1), hi[n*(K/4) + k/4] 2-bit field (k&3), per-16 int8 scale, per-256 fp16
// d.  Unit u = elements [64u, 64u+64): 32 bytes lo, 16 bytes hi, four scales.  Codes stay unsigned
// (0..63); the -32 goes into the min term as for the AoS form.
struct FmtQ6KNat {
    struct W {
        const uint8_t* lo;
        const uint8_t* hi;
        const int8_t* sc;
        const uint16_t* d;
        uint32_t K;
    };
    struct Cursor {
        const uint8_t* lo;
        const uint8_t* hi;
        const uint8_t* sc;
        const uint8_t* d;
    };
    struct Raw {
        uint4 l0, l1, h;
        uint32_t sc4, d;
    };
    static constexpr int SUM_GRAN = 16;
    static constexpr bool PAIRED = false;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {w.lo + (size_t)n * (w.K >> 1) + (size_t)u * 32u, w.hi + (size_t)n * (w.K >> 2) + (size_t)u * 16u,
                reinterpret_cast<const uint8_t*>(w.sc + (size_t)n * (w.K >> 4) + 4u * u),
                reinterpret_cast<const uint8_t*>(w.d + (size_t)n * (w.K >> 8) + (u >> 2))};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const uint4* l = reinterpret_cast<const uint4*>(cu.lo + (size_t)i * (G * 32));
        Raw r;
        r.l0 = l[0];
        r.l1 = l[1];
        r.h = *reinterpret_cast<const uint4*>(cu.hi + (size_t)i * (G * 16));
        r.sc4 = *reinterpret_cast<const uint32_t*>(cu.sc + (size_t)i * (G * 4));
        r.d = *reinterpret_cast<const uint16_t*>(cu.d + (size_t)i * (G / 4 * 2));
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
        const uint32_t w[8] = {r.l0.x, r.l0.y, r.l0.z, r.l0.w, r.l1.x, r.l1.y, r.l1.z, r.l1.w};
        const uint32_t hw[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
        const float d = h2f(r.d);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint32_t lo[4];
            nibbles_to_codes(w[2 * g], lo[0], lo[1]);
            nibbles_to_codes(w[2 * g + 1], lo[2], lo[3]);
            // 16 two-bit fields f0..f15 of one dword -> bits 4..5 of 16 byte codes: a 4x4 byte transpose
            const uint32_t t0 = hw[g] & 0x03030303u, t1 = (hw[g] >> 2) & 0x03030303u;      // f0,f4,f8,f12 / f1,f5,f9,f13
            const uint32_t t2 = (hw[g] >> 4) & 0x03030303u, t3 = (hw[g] >> 6) & 0x03030303u;
            const uint32_t p01a = __builtin_amdgcn_perm(t1, t0, 0x05010400u), p01b = __builtin_amdgcn_perm(t1, t0, 0x07030602u);
            const uint32_t p23a = __builtin_amdgcn_perm(t3, t2, 0x05010400u), p23b = __builtin_amdgcn_perm(t3, t2, 0x07030602u);
            o.q[g][0] = lo[0] | (__builtin_amdgcn_perm(p23a, p01a, 0x05040100u) << 4);       // f0..f3
            o.q[g][1] = lo[1] | (__builtin_amdgcn_perm(p23a, p01a, 0x07060302u) << 4);       // f4..f7
            o.q[g][2] = lo[2] | (__builtin_amdgcn_perm(p23b, p01b, 0x05040100u) << 4);       // f8..f11
            o.q[g][3] = lo[3] | (__builtin_amdgcn_perm(p23b, p01b, 0x07060302u) << 4);       // f12..f15
            o.c[g] = d * (float)(int)(int8_t)(r.sc4 >> (8 * g));
            o.m[g] = 32.f * o.c[g];
        }
    }
};

// ---------------------------------------------------------------- Q8_0, SoA planes
// qs[n*K + k] int8, d[n*(K/32) + b] fp16 bits (src/ops/gemv_q8dot.cpp:601-607).
// Unit u = blocks 2u, 2u+1: 64 bytes of qs, two scales.
struct FmtQ8Soa {
    struct W {
        const int8_t* qs;
        const uint16_t* d;
        uint32_t K;
    };
    // expert e: qs + e*qs_stride (elements), d + e*d_stride (fp16 entries) (include/ie/moe_q8.hpp:8-10)
    struct Bank {
        const int8_t* qs;
        const uint16_t* d;
        uint64_t qs_stride, d_stride;
        uint32_t K;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.qs + (size_t)e * b.qs_stride, b.d + (size_t)e * b.d_stride, b.K}; }
    struct Cursor {
        const uint4* qs;
        const uint8_t* d;
    };
    struct Raw {
        uint4 q[4];
        uint32_t d2;   // d of block 2u | d of block 2u+1 << 16
    };
    static constexpr int SUM_GRAN = 0;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    static constexpr bool CODES_UNSIGNED = false;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)u * 64u),
                reinterpret_cast<const uint8_t*>(w.d + (size_t)n * (w.K >> 5) + 2u * u)};
    }
    // `half_only`: the row ends after the unit's first block (K % 64 == 32)
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool half_only = false) {
        const uint4* p = cu.qs + (size_t)i * (G * 4);
        Raw r;
        r.q[0] = p[0];
        r.q[1] = p[1];
        if (half_only) {
            r.q[2] = r.q[3] = make_uint4(0, 0, 0, 0);
            r.d2 = *reinterpret_cast<const uint16_t*>(cu.d + (size_t)i * (G * 4));
        } else {
            r.q[2] = p[2];
            r.q[3] = p[3];
            r.d2 = load_u1_a2(cu.d + (size_t)i * (G * 4));
        }
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            o.q[g][0] = r.q[g].x; o.q[g][1] = r.q[g].y; o.q[g][2] = r.q[g].z; o.q[g][3] = r.q[g].w;
            o.m[g] = 0.f;
        }
        o.c[0] = o.c[1] = h2f(r.d2 & 0xFFFFu);
        o.c[2] = o.c[3] = h2f(r.d2 >> 16);
    }
};

// ---------------------------------------------------------------- Q8_0, SoA planes, interleaved units
// The same planes, read so that one load instruction of a wave covers whole cache lines.  With units of 64 consecutive
// bytes a lane's four 16-byte loads sit 64 bytes from its neighbour's, and the memory pipeline serves such a load at
// about 18 bytes per clock and CU (measured on L2-resident data; 35 / 50 / 62 when two / four / eight neighbouring lanes
// read adjacent 16-byte pieces).  Here eight consecutive units share a 512-element span of the row and unit 8 U + m
// takes its 16-byte pieces m, m + 8, m + 16, m + 24: eight lanes read 128 contiguous bytes per load, and a line is
// consumed by a single instruction, so the loads carry the non-temporal hint.  Group g of a unit = elements
// 512 U + 16 m + 128 g .. + 15 = half of Q8_0 block 16 U + (m >> 1) + 4 g: four blocks, so four weight scales (each lane
// loads two of the span's sixteen, the eight lanes exchange them) and four activation scales per unit.  K % 512 == 0.
struct FmtQ8SoaW {
    typedef FmtQ8Soa::W W;
    typedef FmtQ8Soa::Bank Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ8Soa::expert(b, e); }
    struct Cursor {
        const uint4* qs;
        const uint8_t* d;
        uint32_t m;
    };
    struct Raw {
        uint4 q[4];
        uint32_t d2;   // scales 2 m, 2 m + 1 of the span's sixteen: the eight lanes of a span hold all of them
    };
    static constexpr int SUM_GRAN = 0;
    static constexpr bool PAIRED = false;
    static constexpr uint32_t GROUP_OFF = 128;
    static constexpr uint32_t K_ALIGN = 512;
    static constexpr bool CODES_UNSIGNED = false;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return (u >> 3) * 512u + (u & 7u) * 16u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)(u >> 3) * 512u + (u & 7u) * 16u),
                reinterpret_cast<const uint8_t*>(w.d + (size_t)n * (w.K >> 5) + (size_t)(u >> 3) * 16u + (u & 7u) * 2u), u & 7u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool = false) {
        static_assert(G % 8 == 0, "a lane keeps its place in the span from step to step");
        const uint4* p = cu.qs + (size_t)i * (G * 4);
        Raw r;
#pragma unroll
        for (int g = 0; g < 4; ++g) r.q[g] = load_u4_stream(p + 8 * g);
        r.d2 = load_u1_a2(cu.d + (size_t)i * (G * 4));
        return r;
    }
    // The lanes of a span sit in eight consecutive lanes of the wave (units 8 U .. 8 U + 7), all live or all idle together
    // (unit counts are multiples of 8).  Group g needs scale (m >> 1) + 4 g: the dword of span lane (m >> 2) + 2 g, half
    // (m >> 1) & 1, fetched across lanes.
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) {
        const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        const uint32_t src = ((lane & ~7u) + (cu.m >> 2)) * 4u, sh = (cu.m & 2u) * 8u;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            o.q[g][0] = r.q[g].x; o.q[g][1] = r.q[g].y; o.q[g][2] = r.q[g].z; o.q[g][3] = r.q[g].w;
            const uint32_t w = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(src + 8u * g), (int)r.d2);
            o.c[g] = h2f((w >> sh) & 0xFFFFu);
            o.m[g] = 0.f;
        }
    }
};

// ---------------------------------------------------------------- Q8_0, AoS GGUF blocks
// 34-byte blocks {fp16 d; int8 qs[32]}: one lane per block pair (68 bytes),
// quants read as four 128-bit loads at 2-byte alignment.
struct FmtQ8Aos {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Cursor {
        const uint8_t* blk;
    };
    typedef FmtQ8Soa::Raw Raw;
    static constexpr int SUM_GRAN = 0;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    static constexpr bool CODES_UNSIGNED = false;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {w.base + (size_t)n * w.row_bytes + (size_t)u * (2 * kQ8_0Bytes)};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool half_only = false) {
        const uint8_t* blk = cu.blk + (size_t)i * (G * 2 * kQ8_0Bytes);
        Raw r;
        r.d2 = *reinterpret_cast<const uint16_t*>(blk);
        r.q[0] = load_u4_a2(blk + 2);
        r.q[1] = load_u4_a2(blk + 18);
        if (half_only) {
            r.q[2] = r.q[3] = make_uint4(0, 0, 0, 0);
        } else {
            r.d2 |= (uint32_t)*reinterpret_cast<const uint16_t*>(blk + 34) << 16;
            r.q[2] = load_u4_a2(blk + 36);
            r.q[3] = load_u4_a2(blk + 52);
        }
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
        FmtQ8Soa::decode(r, FmtQ8Soa::Cursor{}, o);
    }
};

// ---------------------------------------------------------------- Q4_0
// {fp16 d; u8 qs[16]} per 32 elements, element j in the low and j + 16 in the high nibble of qs[j],
// w = d * (q - 8) (include/ie/quant_blocks.hpp:32-43).  Codes stay unsigned; the -8 goes into the
// min term against the activation block's sum: acc += d * (d8 * idot - 8 * s), the reference's fold
// (src/ops/gemv_q4_0.cpp:194-197).  Unit u = blocks 2u, 2u+1.
// SoA planes: q4_qs[n*(K/2) + 16b + j], q4_d[n*(K/32) + b] (repack_q4_0_to_soa, :179-192).
struct FmtQ40Soa {
    struct W {
        const uint8_t* qs;
        const uint16_t* d;
        uint32_t K;
    };
    // expert e: qs + e*qs_stride bytes, d + e*d_stride fp16 entries (include/ie/ops.hpp:179-190)
    struct Bank {
        const uint8_t* qs;
        const uint16_t* d;
        uint64_t qs_stride, d_stride;
        uint32_t K;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.qs + (size_t)e * b.qs_stride, b.d + (size_t)e * b.d_stride, b.K}; }
    struct Cursor {
        const uint4* qs;
        const uint8_t* d;
    };
    struct Raw {
        uint4 qa, qb;
        uint32_t d2;
    };
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {reinterpret_cast<const uint4*>(w.qs + (size_t)n * (w.K >> 1) + (size_t)u * 32u),
                reinterpret_cast<const uint8_t*>(w.d + (size_t)n * (w.K >> 5) + 2u * u)};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool half_only = false) {
        const uint4* p = cu.qs + (size_t)i * (G * 2);
        const uint8_t* d = cu.d + (size_t)i * (G * 4);
        Raw r;
        r.qa = p[0];
        if (half_only) {
            r.qb = make_uint4(0, 0, 0, 0);
            r.d2 = *reinterpret_cast<const uint16_t*>(d);
        } else {
            r.qb = p[1];
            r.d2 = load_u1_a2(d);
        }
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
        const uint32_t a[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w}, b[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o.q[0][i] = a[i] & 0x0F0F0F0Fu;
            o.q[1][i] = (a[i] >> 4) & 0x0F0F0F0Fu;
            o.q[2][i] = b[i] & 0x0F0F0F0Fu;
            o.q[3][i] = (b[i] >> 4) & 0x0F0F0F0Fu;
        }
        o.c[0] = o.c[1] = h2f(r.d2 & 0xFFFFu);
        o.c[2] = o.c[3] = h2f(r.d2 >> 16);
#pragma unroll
        for (int g = 0; g < 4; ++g) o.m[g] = 8.f * o.c[g];
    }
};

// Q4_0 as GGUF blocks (18 B, 2-byte aligned): one lane per block pair, 36 contiguous bytes.
struct FmtQ40Aos {
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
    struct Cursor {
        const uint8_t* blk;
    };
    typedef FmtQ40Soa::Raw Raw;
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) { return {w.base + (size_t)n * w.row_bytes + (size_t)u * 36u}; }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool half_only = false) {
        const uint8_t* blk = cu.blk + (size_t)i * (G * 36);
        Raw r;
        r.d2 = *reinterpret_cast<const uint16_t*>(blk);
        r.qa = load_u4_a2(blk + 2);
        if (half_only) {
            r.qb = make_uint4(0, 0, 0, 0);
        } else {
            r.d2 |= (uint32_t)*reinterpret_cast<const uint16_t*>(blk + 18) << 16;
            r.qb = load_u4_a2(blk + 20);
        }
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) { FmtQ40Soa::decode(r, FmtQ40Soa::Cursor{}, o); }
};

// ---------------------------------------------------------------- Q5_K (AoS GGUF blocks)
// {d, dmin, scales[12], qh[32], qs[128]} (176 B; include/ie/quant_blocks.hpp:79-85): Q4_K plus a fifth
// bit, bit 2g + hi of qh[l] for element 64g + 32hi + l (include/ie/dequant_ref.hpp:55-75).  Units, scales
// and fold as Q4_K; the unit also reads the whole qh (32 bytes) and picks its two bit planes.
struct FmtQ5K {
    struct W {
        const uint8_t* base;
        uint32_t row_bytes;
    };
    struct Cursor {
        const uint8_t* blk;
        uint32_t g;
    };
    struct Raw {
        uint4 hdr, h0, h1, q0, q1;
    };
    static constexpr int SUM_GRAN = 32;
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr bool CODES_UNSIGNED = true;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {w.base + (size_t)n * w.row_bytes + (size_t)(u >> 2) * 176u, u & 3u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i) {
        const uint8_t* blk = cu.blk + (size_t)i * (G / 4 * 176);
        const uint4* h = reinterpret_cast<const uint4*>(blk + 16);
        const uint4* q = reinterpret_cast<const uint4*>(blk + 48 + cu.g * 32u);
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.h0 = h[0];
        r.h1 = h[1];
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor& cu, Unit& o) {
        const uint32_t q0[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w}, q1[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t h0[4] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w}, h1[4] = {r.h1.x, r.h1.y, r.h1.z, r.h1.w};
        const uint32_t sh = 2u * cu.g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // bit (2g) of each qh byte -> bit 4 of the low-nibble code, bit (2g+1) -> of the high-nibble code
            o.q[0][i] = (q0[i] & 0x0F0F0F0Fu) | (((h0[i] >> sh) & 0x01010101u) << 4);
            o.q[1][i] = (q1[i] & 0x0F0F0F0Fu) | (((h1[i] >> sh) & 0x01010101u) << 4);
            o.q[2][i] = ((q0[i] >> 4) & 0x0F0F0F0Fu) | (((h0[i] >> (sh + 1u)) & 0x01010101u) << 4);
            o.q[3][i] = ((q1[i] >> 4) & 0x0F0F0F0Fu) | (((h1[i] >> (sh + 1u)) & 0x01010101u) << 4);
        }
        uint32_t sc, mn;
        q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, (int)cu.g, sc, mn);
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        o.c[0] = o.c[1] = d * (float)(sc & 0xFFu);
        o.c[2] = o.c[3] = d * (float)(sc >> 8);
        o.m[0] = o.m[1] = dmin * (float)(mn & 0xFFu);
        o.m[2] = o.m[3] = dmin * (float)(mn >> 8);
    }
};

// ---------------------------------------------------------------- MXFP4, SoA planes
// qs_plane[n*(K/2) + 16b + j], e_plane[n*(K/32) + b] (src/ops/gemv_mxfp4.cpp:13-16).
// Unit u = blocks 2u, 2u+1: 32 bytes of codes (per block: low nibbles = elements
// 0..15, high = 16..31), two E8M0 exponents.  Codes become doubled E2M1 values as
// int8; the block scale is 2^(e-128).
struct FmtMxfp4Soa {
    struct W {
        const uint8_t* qs;
        const uint8_t* e;
        uint32_t K;
    };
    // expert x: qs + x*qs_stride, e + x*e_stride bytes (src/model/gptoss.cpp:183-195)
    struct Bank {
        const uint8_t* qs;
        const uint8_t* e;
        uint64_t qs_stride, e_stride;
        uint32_t K;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t x) { return {b.qs + (size_t)x * b.qs_stride, b.e + (size_t)x * b.e_stride, b.K}; }
    struct Cursor {
        const uint4* qs;
        const uint8_t* e;
    };
    struct Raw {
        uint4 qa, qb;
        uint32_t e2;
    };
    static constexpr int SUM_GRAN = 2;   // int-dot GEMVs: fp16-pair activations, codes converted by the FP4 convert instruction (fp4())
    static constexpr bool PAIRED = true;
    static constexpr uint32_t GROUP_OFF = 16;
    static constexpr uint32_t K_ALIGN = 32;
    static constexpr bool CODES_UNSIGNED = false;
    __device__ static __forceinline__ uint32_t elem_off(uint32_t u) { return u * 64u; }
    __device__ static __forceinline__ Cursor cursor(const W& w, uint32_t n, uint32_t u) {
        return {reinterpret_cast<const uint4*>(w.qs + (size_t)n * (w.K >> 1) + (size_t)u * 32u), w.e + (size_t)n * (w.K >> 5) + 2u * u};
    }
    template <int G>
    __device__ static __forceinline__ Raw load(const Cursor& cu, uint32_t i, bool half_only = false) {
        const uint4* p = cu.qs + (size_t)i * (G * 2);
        const uint8_t* e = cu.e + (size_t)i * (G * 2);
        Raw r;
        r.qa = p[0];
        if (half_only) {
            r.qb = make_uint4(0, 0, 0, 0);
            r.e2 = e[0];
        } else {
            r.qb = p[1];
            struct __attribute__((packed, aligned(1))) E2 { uint16_t v; };   // one request for both exponents (any byte address)
            r.e2 = reinterpret_cast<const E2*>(e)->v;
        }
        return r;
    }
    // the unit as the convert instruction takes it: eight code words (two blocks) and the two half-scaled block scales
    __device__ static __forceinline__ void fp4(const Raw& r, uint32_t (&w)[8], float (&c)[2]) {
        w[0] = r.qa.x; w[1] = r.qa.y; w[2] = r.qa.z; w[3] = r.qa.w;
        w[4] = r.qb.x; w[5] = r.qb.y; w[6] = r.qb.z; w[7] = r.qb.w;
        c[0] = e8m0_half(r.e2 & 0xFFu);
        c[1] = e8m0_half(r.e2 >> 8);
    }
    // doubled E2M1 values as int8 (the float-activation GEMV)
    __device__ static __forceinline__ void decode(const Raw& r, const Cursor&, Unit& o) {
        mxfp4_decode_word(r.qa.x, o.q[0][0], o.q[1][0]);
        mxfp4_decode_word(r.qa.y, o.q[0][1], o.q[1][1]);
        mxfp4_decode_word(r.qa.z, o.q[0][2], o.q[1][2]);
        mxfp4_decode_word(r.qa.w, o.q[0][3], o.q[1][3]);
        mxfp4_decode_word(r.qb.x, o.q[2][0], o.q[3][0]);
        mxfp4_decode_word(r.qb.y, o.q[2][1], o.q[3][1]);
        mxfp4_decode_word(r.qb.z, o.q[2][2], o.q[3][2]);
        mxfp4_decode_word(r.qb.w, o.q[2][3], o.q[3][3]);
        o.c[0] = o.c[1] = e8m0_half(r.e2 & 0xFFu);
        o.c[2] = o.c[3] = e8m0_half(r.e2 >> 8);
#pragma unroll
        for (int g = 0; g < 4; ++g) o.m[g] = 0.f;
    }
};

// K-quant loads never run past a row (K % 256 == 0), so they ignore half_only.
template <class F, int G>
__device__ __forceinline__ typename F::Raw load_unit(const typename F::Cursor& cu, uint32_t i, bool half_only) {
    if constexpr (F::K_ALIGN == 256) {
        return F::template load<G>(cu, i);
    } else {
        return F::template load<G>(cu, i, half_only);
    }
}

}  // namespace mxq
