// mxq_mmq.h — int-dot on the matrix cores: q8 activation rows x block-quantized weights with
// v_mfma_i32_32x32x32_i8, one 32-element block per instruction.
//
// The arithmetic is the reference's int-dot chain, block by block
//     acc[t][n] += d_w[n][b] * (d_x[t][b] * float(sum_k q_w[n][k] q_x[t][k]))  (- m_w[n][b] * s_x[t][b] for Q4_K)
// (src/ops/gemv_q8dot.cpp:328-350,646-653, src/ops/gemv_q6k.cpp:412-438, src/ops/gemv_mxfp4.cpp:120-141): the
// integer dot of a block is exact, so only the fp32 fold order differs from the vector-ALU kernels.  One MFMA
// covers exactly one block of 32 k-values for 32 tokens x 32 weight rows, i.e. the 8 x T dot4 instructions per lane
// and block of the vector path become one matrix instruction per 32 rows, and what is left per block is the
// fold (convert, two multiplies per live output).  That makes batches of 2 .. 32 rows a stream over the weight
// bytes again (the vector path is issue-bound from T = 4 on).
//
// Operand layout (wave64): the A operand holds tokens, lane (i = lane % 32, h = lane / 32) the 16 quants
// x[i][32 b + 16 h ..], read from the staged activation plane in LDS; the B operand holds weights, lane (j, h) the
// 16 codes w[n0 + j][32 b + 16 h ..], produced in registers from the lane's own global loads.  Both operands use
// the same (h, byte) -> k map, which is all the instruction needs.  Result: lane (j, h) holds column j (weight
// row n0 + j) and token rows 8 (v / 4) + 4 h + v % 4, v = 0 .. 15; with T <= 8 tokens only v = 0 .. 3 are live
// (TV = 4), T <= 16: v < 8, T <= 32: all 16.
//
// Work split: a workgroup of NW x WR x WK waves owns 32 WR weight rows (of NW matrices: gate and up) and a K
// range; wave (m, wr, wk) walks its share of the range's 256-element groups with one group of weight words in
// flight behind the one being multiplied.  The activation rows of the range are staged once per
// workgroup.  Partial sums of the WK waves meet in LDS; K ranges of different workgroups (dense launches with
// few rows) meet in a scratch plane that a second launch reduces.
#pragma once

#include <type_traits>

#include "mxq_formats.h"

namespace mxq {

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef int v16i_t __attribute__((ext_vector_type(16)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

// producers that feed the scaled FP8 x FP4 matrix instruction declare NATIVE_FP4
template <class P, class = void> struct mmq_native : std::false_type {};
template <class P> struct mmq_native<P, std::void_t<decltype(P::NATIVE_FP4)>> : std::true_type {};

__device__ __forceinline__ v4i_t as_v4i(const uint4& u) {
    v4i_t r;
    r.x = (int)u.x; r.y = (int)u.y; r.z = (int)u.z; r.w = (int)u.w;
    return r;
}
__device__ __forceinline__ uint4 load_u4_a1(const uint8_t* p) {
    struct __attribute__((packed, aligned(1))) U4 { uint32_t x, y, z, w; };
    const U4 v = *reinterpret_cast<const U4*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_u2_a1(const uint8_t* p) {
    struct __attribute__((packed, aligned(1))) U2 { uint32_t x, y; };
    const U2 v = *reinterpret_cast<const U2*>(p);
    return make_uint2(v.x, v.y);
}

// ---------------------------------------------------------------- weight operand producers
// A group = 8 consecutive blocks of 32 (one 256-element super-block of the K-quants).  load() fetches what lane
// (row n, half h) needs of group g; `nb` = blocks per row, groups past the row end re-read valid bytes and get
// scale 0.  operand<S>() = the 16 int8 codes of block S of the group for this lane half; scale<S>() the fp32
// factor of that block (SUBS = 2: one factor per 16-element half, Q6_K).
struct MmqQ8Soa {
    using W = FmtQ8Soa::W;
    using Bank = FmtQ8Soa::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ8Soa::expert(b, e); }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t K_ALIGN = 32;
    struct Raw {
        uint4 q[8];
        uint32_t d[4];   // 8 fp16 block scales
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t nb) {
        const uint8_t* p = reinterpret_cast<const uint8_t*>(w.qs) + (size_t)n * w.K + 16u * h + (size_t)g * 256u;
        const uint8_t* d = reinterpret_cast<const uint8_t*>(w.d + (size_t)n * nb);
        Raw r;
#pragma unroll
        for (int s = 0; s < 8; ++s) r.q[s] = *reinterpret_cast<const uint4*>(p + s * 32);
        const uint4 dd = load_u4_a2(d + 16u * g);
        r.d[0] = dd.x; r.d[1] = dd.y; r.d[2] = dd.z; r.d[3] = dd.w;
        return r;
    }
    // the last group of a row whose block count is not a multiple of 8
    __device__ static __forceinline__ Raw load_tail(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t nb) {
        const uint8_t* p = reinterpret_cast<const uint8_t*>(w.qs) + (size_t)n * w.K + 16u * h;
        const uint16_t* d = w.d + (size_t)n * nb;
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t b = 8u * g + s, bc = b < nb ? b : nb - 1u;
            r.q[s] = *reinterpret_cast<const uint4*>(p + (size_t)bc * 32u);
            ds[s] = b < nb ? (uint32_t)d[bc] : 0u;   // fp16 +0: the block contributes nothing
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t) { return as_v4i(r.q[S]); }
    struct Dec {
        float c[8];
    };
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t) {
        Dec o;
#pragma unroll
        for (int s = 0; s < 8; ++s) o.c[s] = h2f((s & 1) ? r.d[s >> 1] >> 16 : r.d[s >> 1] & 0xFFFFu);
        return o;
    }
};

// Q8_0 GGUF blocks (34 B: fp16 d, 32 int8; 2-byte aligned): lane half h reads the 16 quants at byte 2 + 16 h of each
// block and the block's d.  Same operands and fold as the planes, so both layouts give the same bits.
struct MmqQ8Aos {
    using W = FmtQ8Aos::W;
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint32_t row_bytes;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.base + (size_t)e * b.expert_stride_bytes, b.row_bytes}; }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t K_ALIGN = 32;
    using Raw = MmqQ8Soa::Raw;
    using Dec = MmqQ8Soa::Dec;
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes + (size_t)g * (8 * kQ8_0Bytes);
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            r.q[s] = load_u4_a2(p + s * kQ8_0Bytes + 2 + 16u * h);
            ds[s] = *reinterpret_cast<const uint16_t*>(p + s * kQ8_0Bytes);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    __device__ static __forceinline__ Raw load_tail(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t nb) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes;
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t b = 8u * g + s, bc = b < nb ? b : nb - 1u;
            r.q[s] = load_u4_a2(p + (size_t)bc * kQ8_0Bytes + 2 + 16u * h);
            ds[s] = b < nb ? (uint32_t) * reinterpret_cast<const uint16_t*>(p + (size_t)bc * kQ8_0Bytes) : 0u;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t) { return as_v4i(r.q[S]); }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t h) { return MmqQ8Soa::prepare(r, h); }
};

// MXFP4 SoA planes: qs_plane[n*(K/2) + 16 b + j] (element j in the low, 16 + j in the high nibble), e_plane[n*(K/32) + b]
// (src/ops/gemv_mxfp4.cpp:13-16).  Both lane halves read the block's 16 bytes; half h decodes nibble h of each.
struct MmqMxfp4Soa {
    using W = FmtMxfp4Soa::W;
    using Bank = FmtMxfp4Soa::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtMxfp4Soa::expert(b, e); }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t K_ALIGN = 32;
    struct Raw {
        uint4 q[8];
        uint32_t e[2];
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t nb) {
        const uint8_t* p = w.qs + (size_t)n * (w.K >> 1) + (size_t)g * 128u;
        Raw r;
#pragma unroll
        for (int s = 0; s < 8; ++s) r.q[s] = *reinterpret_cast<const uint4*>(p + s * 16);
        const uint2 ee = load_u2_a1(w.e + (size_t)n * nb + 8u * g);
        r.e[0] = ee.x; r.e[1] = ee.y;
        return r;
    }
    // the last group of a row whose block count is not a multiple of 8: a dead block gets exponent 0 and cleared
    // codes (code 0 is the value 0)
    __device__ static __forceinline__ Raw load_tail(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t nb) {
        const uint8_t* p = w.qs + (size_t)n * (w.K >> 1);
        const uint8_t* e = w.e + (size_t)n * nb;
        Raw r;
        uint32_t es[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t b = 8u * g + s, bc = b < nb ? b : nb - 1u;
            const uint4 q = *reinterpret_cast<const uint4*>(p + (size_t)bc * 16u);
            r.q[s] = b < nb ? q : make_uint4(0, 0, 0, 0);
            es[s] = b < nb ? (uint32_t)e[bc] : 0u;
        }
        r.e[0] = es[0] | (es[1] << 8) | (es[2] << 16) | (es[3] << 24);
        r.e[1] = es[4] | (es[5] << 8) | (es[6] << 16) | (es[7] << 24);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t h) {
        const uint32_t sh = 4u * h;
        const uint32_t w[4] = {r.q[S].x >> sh, r.q[S].y >> sh, r.q[S].z >> sh, r.q[S].w >> sh};
        v4i_t o;
        o.x = (int)mxfp4_lut4(w[0] & 0x07070707u, ((w[0] >> 1) & 0x04040404u) | 0x03020100u);
        o.y = (int)mxfp4_lut4(w[1] & 0x07070707u, ((w[1] >> 1) & 0x04040404u) | 0x03020100u);
        o.z = (int)mxfp4_lut4(w[2] & 0x07070707u, ((w[2] >> 1) & 0x04040404u) | 0x03020100u);
        o.w = (int)mxfp4_lut4(w[3] & 0x07070707u, ((w[3] >> 1) & 0x04040404u) | 0x03020100u);
        return o;
    }
    struct Dec {
        float c[8];
    };
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t) {
        Dec o;
#pragma unroll
        for (int s = 0; s < 8; ++s) o.c[s] = e8m0_half((r.e[s >> 2] >> (8 * (s & 3))) & 0xFFu);
        return o;
    }
};

// MXFP4 planes fed to the matrix cores as they lie in memory: v_mfma_scale_f32_32x32x64_f8f6f4 takes E2M1 codes and one
// E8M0 scale per lane and 32 k-values, which is exactly a block of this format (include/ie/quant_blocks.hpp:46-54), so
// there is no code -> integer conversion at all.  The q8 activation codes go in as two FP8 (E4M3) operands, q = 16 hi + lo
// with hi = q >> 4 in -8..7 and lo = q & 15, both exact in E4M3; the hi instruction runs with the scale 2^4 and both
// accumulate into the same registers, so the instruction pair returns 2^(e-127) * sum_k e2m1(w_k) * q_k exactly (every
// partial sum is a small multiple of 2^(e-128)), the same number as weight-scale x integer dot of the vector kernels.
// What the fold still does per block is the multiplication by the activation block scale d_x, which is not a power of two.
//
// Operand geometry (measured on gfx950 with one-hot operands): the instruction sums K = 64 in four groups of 16; an FP4
// lane (column j, half h) holds groups 2h and 2h+1 as 32 consecutive nibbles (low nibble first), an FP8 lane (row i, half
// h) holds group h in bytes 0..15 and group 2 + h in bytes 16..31.  So lane half h of the weight operand carries the whole
// block 2 s + h of pair s, and the token rows are arranged so that the two blocks of a pair land in different result rows:
// rows 0..15 = up to 16 tokens against block 2 s (bytes 16..31 of their operand are zero), rows 16..31 = the same tokens
// against block 2 s + 1 (bytes 0..15 zero).  Result registers v < 8 of lane (j, h) are then tokens 8 (v / 4) + 4 h + v % 4
// for block 2 s and registers 8 + v the same tokens for block 2 s + 1.
struct MmqMxfp4Native {
    using W = FmtMxfp4Soa::W;
    using Bank = FmtMxfp4Soa::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtMxfp4Soa::expert(b, e); }
    static constexpr bool NATIVE_FP4 = true;
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t K_ALIGN = 32;
    struct Raw {
        uint4 q[4];       // blocks h, 2 + h, 4 + h, 6 + h of the group
        uint32_t e[2];    // the eight exponents of the group; lane half h uses bytes h and 2 + h of e[s / 2]
    };
    // Nothing is computed on the loaded words here (that would make the request wait for them).  A partial last group
    // (block count not a multiple of 8) re-reads the row's last block for its dead blocks and takes the eight exponent
    // bytes that end at the row end; the staged activations of dead blocks are zero, so whatever they hold adds nothing.
    // live = false: every lane reads the same valid bytes (the loads of a pipeline slot past the end of the walk).
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t nb, bool live = true) {
        const uint8_t* row = w.qs + (size_t)n * (w.K >> 1);
        const uint32_t last = nb - 1u, e_at = 8u * g + 8u <= nb ? 8u * g : nb - 8u;
        const uint8_t* e = live ? w.e + (size_t)n * nb + e_at : w.e;
        Raw r;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint32_t b = 8u * g + 2u * s + h;
            r.q[s] = *reinterpret_cast<const uint4*>(live ? row + (size_t)(b < last ? b : last) * 16u : w.qs);
        }
        const uint2 ee = load_u2_a1(e);
        r.e[0] = ee.x;
        r.e[1] = ee.y;
        return r;
    }
    // exponent byte of pair S for lane half h (block 2 S + h of group g), moved to byte 0
    template <int S>
    __device__ static __forceinline__ int scale_word(const Raw& r, uint32_t g, uint32_t h, uint32_t nb) {
        const uint32_t skew = 8u * g + 8u <= nb ? 0u : 8u * g + 8u - nb;   // bytes the partial group's exponent window was moved down
        const uint64_t all = ((uint64_t)r.e[1] << 32) | r.e[0];
        const uint32_t at = skew + 2u * S + h;                             // past the window for a dead block: any valid byte will do
        return (int)(uint32_t)(all >> (8u * (at < 7u ? at : 7u)));
    }
};

// Q4_K AoS blocks: group g = block g of the row; sub-block s = nibble (s & 1) of qs[32 (s / 2) + l], l = 0..31
// (include/ie/dequant_ref.hpp:38-53); lane half h owns l = 16 h .. 16 h + 15.  Codes stay unsigned (0..15); the min
// term folds on the stored block sum of the activation row.
struct MmqQ4K {
    using W = FmtQ4K::W;
    using Bank = FmtQ4K::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ4K::expert(b, e); }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = true;
    static constexpr uint32_t K_ALIGN = 256;
    struct Raw {
        uint4 hdr, q[4];
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)g * kQ4KBytes;
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
#pragma unroll
        for (int i = 0; i < 4; ++i) r.q[i] = *reinterpret_cast<const uint4*>(blk + 16 + 32 * i + 16u * h);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t) {
        const uint4 w = r.q[S >> 1];
        constexpr int sh = (S & 1) * 4;
        v4i_t o;
        o.x = (int)((w.x >> sh) & 0x0F0F0F0Fu); o.y = (int)((w.y >> sh) & 0x0F0F0F0Fu);
        o.z = (int)((w.z >> sh) & 0x0F0F0F0Fu); o.w = (int)((w.w >> sh) & 0x0F0F0F0Fu);
        return o;
    }
    struct Dec {
        float c[8], m[8];
    };
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t) {
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        Dec o;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint32_t sc, mn;
            q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, g, sc, mn);
            o.c[2 * g] = d * (float)(sc & 0xFFu);
            o.c[2 * g + 1] = d * (float)(sc >> 8);
            o.m[2 * g] = dmin * (float)(mn & 0xFFu);
            o.m[2 * g + 1] = dmin * (float)(mn >> 8);
        }
        return o;
    }
};

// Q4_0 (32-element blocks: fp16 d, 16 bytes with element j in the low and j + 16 in the high nibble of byte j;
// include/ie/quant_blocks.hpp:32-43): value = d (q - 8), so the codes stay unsigned and the -8 d folds on the stored
// block sum of the activation row, like Q4_K's min term.  Lane half h takes the low (h = 0) or high nibbles of all 16
// bytes, so both halves load the block's bytes.  Planes: qs[N][K/2], d[N][K/32]; GGUF blocks: 18 bytes, 2-byte aligned.
struct MmqQ40Soa {
    using W = FmtQ40Soa::W;
    using Bank = FmtQ40Soa::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ40Soa::expert(b, e); }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = true;
    static constexpr uint32_t K_ALIGN = 32;
    struct Raw {
        uint4 q[8];
        uint32_t d[4];   // 8 fp16 block scales
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t nb) {
        const uint8_t* p = w.qs + (size_t)n * (w.K >> 1) + (size_t)g * 128u;
        Raw r;
#pragma unroll
        for (int s = 0; s < 8; ++s) r.q[s] = *reinterpret_cast<const uint4*>(p + s * 16);
        const uint4 dd = load_u4_a2(reinterpret_cast<const uint8_t*>(w.d + (size_t)n * nb) + 16u * g);
        r.d[0] = dd.x; r.d[1] = dd.y; r.d[2] = dd.z; r.d[3] = dd.w;
        return r;
    }
    __device__ static __forceinline__ Raw load_tail(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t nb) {
        const uint8_t* p = w.qs + (size_t)n * (w.K >> 1);
        const uint16_t* d = w.d + (size_t)n * nb;
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t b = 8u * g + s, bc = b < nb ? b : nb - 1u;
            r.q[s] = *reinterpret_cast<const uint4*>(p + (size_t)bc * 16u);
            ds[s] = b < nb ? (uint32_t)d[bc] : 0u;   // fp16 +0: the block contributes nothing (its activation sum is zero as well)
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t h) {
        const uint32_t sh = 4u * h;
        v4i_t o;
        o.x = (int)((r.q[S].x >> sh) & 0x0F0F0F0Fu); o.y = (int)((r.q[S].y >> sh) & 0x0F0F0F0Fu);
        o.z = (int)((r.q[S].z >> sh) & 0x0F0F0F0Fu); o.w = (int)((r.q[S].w >> sh) & 0x0F0F0F0Fu);
        return o;
    }
    struct Dec {
        float c[8], m[8];
    };
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t) {
        Dec o;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            o.c[s] = h2f((s & 1) ? r.d[s >> 1] >> 16 : r.d[s >> 1] & 0xFFFFu);
            o.m[s] = 8.f * o.c[s];
        }
        return o;
    }
};
struct MmqQ40Aos {
    using W = FmtQ40Aos::W;
    using Bank = FmtQ40Aos::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ40Aos::expert(b, e); }
    static constexpr int SUBS = 1;
    static constexpr bool HAS_MIN = true;
    static constexpr uint32_t K_ALIGN = 32;
    using Raw = MmqQ40Soa::Raw;
    using Dec = MmqQ40Soa::Dec;
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes + (size_t)g * (8u * 18u);
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            r.q[s] = load_u4_a2(p + 18 * s + 2);
            ds[s] = *reinterpret_cast<const uint16_t*>(p + 18 * s);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    __device__ static __forceinline__ Raw load_tail(const W& w, uint32_t n, uint32_t g, uint32_t, uint32_t nb) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes;
        Raw r;
        uint32_t ds[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t b = 8u * g + s, bc = b < nb ? b : nb - 1u;
            r.q[s] = load_u4_a2(p + (size_t)bc * 18u + 2);
            ds[s] = b < nb ? (uint32_t)*reinterpret_cast<const uint16_t*>(p + (size_t)bc * 18u) : 0u;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) r.d[s] = ds[2 * s] | (ds[2 * s + 1] << 16);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t h) { return MmqQ40Soa::operand<S>(r, h); }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t h) { return MmqQ40Soa::prepare(r, h); }
};

// Q6_K AoS blocks (210 B, 2-byte aligned): element 128 hf + 32 sub + l has its low nibble in nibble (sub >> 1) of
// ql[64 hf + 32 (sub & 1) + l] and its two high bits at 2 sub of qh[32 hf + l]; scale scales[8 hf + 2 sub + l / 16]
// (include/ie/dequant_ref.hpp:78-96).  Lane half h owns l = 16 h .. +15, which is exactly the 16-element scale
// group l / 16 = h, so a block needs two matrix instructions, each with the activations of one lane half only
// (SUBS = 2), and folds per 16 elements as the reference does.  Codes go in signed (code - 32).
struct MmqQ6K {
    using W = FmtQ6K::W;
    using Bank = FmtQ6K::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ6K::expert(b, e); }
    static constexpr int SUBS = 2;
    static constexpr bool HAS_MIN = false;
    static constexpr uint32_t K_ALIGN = 256;
    struct Raw {
        uint4 ql[4], qh[2], sc;
        uint32_t d;
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)g * kQ6KBytes;
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r.ql[i] = load_u4_a2(blk + 32 * i + 16u * h);     // i = 2 hf + (sub & 1)
        r.qh[0] = load_u4_a2(blk + 128 + 16u * h);
        r.qh[1] = load_u4_a2(blk + 160 + 16u * h);
        r.sc = load_u4_a2(blk + 192);
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
        return r;
    }
    template <int S>
    __device__ static __forceinline__ v4i_t operand(const Raw& r, uint32_t) {
        constexpr int hf = S >> 2, sub = S & 3;
        const uint4 l = r.ql[2 * hf + (sub & 1)], q = r.qh[hf];
        constexpr int ls = (sub >> 1) * 4, hs = 2 * sub;
        auto one = [&](uint32_t lw, uint32_t hw) {
            const uint32_t code = ((lw >> ls) & 0x0F0F0F0Fu) | (((hw >> hs) & 0x03030303u) << 4);
            return (int)(((code | 0x80808080u) - 0x20202020u) ^ 0x80808080u);        // per byte: code - 32
        };
        v4i_t o;
        o.x = one(l.x, q.x); o.y = one(l.y, q.y); o.z = one(l.z, q.z); o.w = one(l.w, q.w);
        return o;
    }
    struct Dec {
        float c[16];   // c[2 S + half]
    };
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t) {
        const float d = h2f(r.d);
        const uint32_t s[4] = {r.sc.x, r.sc.y, r.sc.z, r.sc.w};
        Dec o;
#pragma unroll
        for (int i = 0; i < 16; ++i) o.c[i] = d * (float)(int)(int8_t)(s[i >> 2] >> (8 * (i & 3)));
        return o;
    }
};

// The per-field stream forms of the K-quants (qs | scales | {d, dmin} and ql | qh | scales | d per matrix or per
// expert region, include/ie/quant_soa.hpp:33-51): the same words from other addresses, the same operands and fold.
struct MmqQ4KStr : MmqQ4K {
    using W = FmtQ4KStr::W;
    using Bank = FmtQ4KStr::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ4KStr::expert(b, e); }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t) {
        const size_t ib = (size_t)n * w.bpr + g;
        const uint32_t* sc = reinterpret_cast<const uint32_t*>(w.sc + ib * 12u);
        Raw r;
        r.hdr = make_uint4(*reinterpret_cast<const uint32_t*>(w.dm + ib * 4u), sc[0], sc[1], sc[2]);
#pragma unroll
        for (int i = 0; i < 4; ++i) r.q[i] = *reinterpret_cast<const uint4*>(w.qs + ib * 128u + 32 * i + 16u * h);
        return r;
    }
};
struct MmqQ6KStr : MmqQ6K {
    using W = FmtQ6KStr::W;
    using Bank = FmtQ6KStr::Bank;
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return FmtQ6KStr::expert(b, e); }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t g, uint32_t h, uint32_t) {
        const size_t ib = (size_t)n * w.bpr + g;
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r.ql[i] = load_u4_a2(w.ql + ib * 128u + 32 * i + 16u * h);
        r.qh[0] = load_u4_a2(w.qh + ib * 64u + 16u * h);
        r.qh[1] = load_u4_a2(w.qh + ib * 64u + 32u + 16u * h);
        r.sc = load_u4_a2(w.sc + ib * 16u);
        r.d = *reinterpret_cast<const uint16_t*>(w.d + ib * 2u);
        return r;
    }
};

// ---------------------------------------------------------------- activation staging
// LDS image of T q8 rows over the k range [k0, k0 + kr) (kr a multiple of 256, the tail of the row zero padded):
//   plane  [T][kr + 32]        int8 quants (the 32-byte pad spreads the rows over the banks)
//   dx     [kr / 32][TP]       fp32 block scales d           TP = 2 TV token slots per block
//   sx     [kr / 32][TP]       fp32 block sums s = d * sum q (HAS_MIN formats only)
// Blocks past the end of the row get d = s = 0 and zero quants.  Rows are block_q8_1x (40 B) or block_q8_1s
// (48 B, s = s0 + s1) streams.
struct MmqAct {
    const uint8_t* plane;
    const float* dx;
    const float* sx;
    uint32_t stride;   // plane row pitch in bytes
};
__host__ __device__ constexpr uint32_t mmq_row_pitch(uint32_t kr, bool native) { return native ? 2u * kr + 16u : kr + 32u; }
__host__ __device__ constexpr uint32_t mmq_lds_bytes(uint32_t T, uint32_t kr, int TV, bool has_min, bool native = false) {
    return T * mmq_row_pitch(kr, native) + (kr / 32u) * (uint32_t)(2 * TV) * 4u * (has_min ? 2u : 1u);
}

// Four 4-bit values (one per byte) through a 16-entry byte table: two byte permutes over the table halves, a third one
// takes byte i from the low or the high result.
__device__ __forceinline__ uint32_t mmq_lut16(uint32_t n, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t sel = n & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    return __builtin_amdgcn_perm(hi, lo, ((n >> 1) & 0x04040404u) | 0x03020100u);
}

// The 32 codes of one activation block into the staged image.  Int8 plane: as they are (32 B at 32 b).  FP8 image of
// the native FP4 path (64 B at 64 b): [hi chunk 0][hi chunk 1][lo chunk 0][lo chunk 1], hi = q >> 4 and lo = q & 15 as
// E4M3 bytes (0, 1, .. 15 -> 00 38 40 44 48 4A 4C 4E 50 .. 57; -8 .. -1 -> D0 CE CC CA C8 C4 C0 B8); chunk h holds, at
// byte p, element ((16 h + p) >> 1) + 16 ((16 h + p) & 1), the order of the nibbles of an MXFP4 block (byte m = elements
// m and m + 16).
template <bool NATIVE>
__device__ __forceinline__ void mmq_store_codes(uint8_t* row, uint32_t b, const uint4& q0, const uint4& q1) {
    if constexpr (!NATIVE) {
        uint4* dst = reinterpret_cast<uint4*>(row + 32u * b);
        dst[0] = q0;
        dst[1] = q1;
    } else {
        const uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            lo[j] = mmq_lut16(w[j] & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0x53525150u, 0x57565554u);
            hi[j] = mmq_lut16((w[j] >> 4) & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0xCACCCED0u, 0xB8C0C4C8u);
        }
        // dwords j and j + 4 hold elements 4j.. and 16 + 4j..: interleave them byte by byte
        auto il0 = [](uint32_t a, uint32_t c) { return __builtin_amdgcn_perm(c, a, 0x05010400u); };
        auto il1 = [](uint32_t a, uint32_t c) { return __builtin_amdgcn_perm(c, a, 0x07030602u); };
        uint4* dst = reinterpret_cast<uint4*>(row + 64u * b);
        dst[0] = make_uint4(il0(hi[0], hi[4]), il1(hi[0], hi[4]), il0(hi[1], hi[5]), il1(hi[1], hi[5]));
        dst[1] = make_uint4(il0(hi[2], hi[6]), il1(hi[2], hi[6]), il0(hi[3], hi[7]), il1(hi[3], hi[7]));
        dst[2] = make_uint4(il0(lo[0], lo[4]), il1(lo[0], lo[4]), il0(lo[1], lo[5]), il1(lo[1], lo[5]));
        dst[3] = make_uint4(il0(lo[2], lo[6]), il1(lo[2], lo[6]), il0(lo[3], lo[7]), il1(lo[3], lo[7]));
    }
}

template <int TV, bool HAS_MIN, bool NATIVE, class RowFn>
__device__ __forceinline__ MmqAct mmq_stage(uint8_t* lds, RowFn xrow, uint32_t T, uint32_t k0, uint32_t kr, uint32_t K, bool split) {
    constexpr uint32_t TP = 2 * TV;
    const uint32_t stride = mmq_row_pitch(kr, NATIVE), nblk = kr / 32u;
    float* dx = reinterpret_cast<float*>(lds + (size_t)T * stride);
    float* sx = dx + (size_t)nblk * TP;
    const uint32_t bsz = split ? kQ81sBytes : kQ81xBytes, hsz = split ? 16u : 8u;
    // four (token, block) pairs per thread and round: all their loads are requested before the first LDS write
    const uint32_t total = T * nblk;
    for (uint32_t base = threadIdx.x; base < total; base += 4u * blockDim.x) {
        uint4 q0[4], q1[4];
        float d[4], sm[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = base + (uint32_t)u * blockDim.x;
            q0[u] = make_uint4(0, 0, 0, 0);
            q1[u] = q0[u];
            d[u] = 0.f;
            sm[u] = 0.f;
            if (i < total) {
                const uint32_t t = i / nblk, b = i - t * nblk;
                if (k0 + 32u * b < K) {
                    const uint8_t* blk = xrow(t) + (size_t)(k0 / 32u + b) * bsz;
                    const uint2* q = reinterpret_cast<const uint2*>(blk + hsz);
                    const uint2 a0 = q[0], a1 = q[1], a2 = q[2], a3 = q[3];
                    q0[u] = make_uint4(a0.x, a0.y, a1.x, a1.y);
                    q1[u] = make_uint4(a2.x, a2.y, a3.x, a3.y);
                    if (split) {
                        const float4 hd = *reinterpret_cast<const float4*>(blk);
                        d[u] = hd.x;
                        sm[u] = hd.y + hd.z;
                    } else {
                        const float2 hd = *reinterpret_cast<const float2*>(blk);
                        d[u] = hd.x;
                        sm[u] = hd.y;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = base + (uint32_t)u * blockDim.x;
            if (i < total) {
                const uint32_t t = i / nblk, b = i - t * nblk;
                mmq_store_codes<NATIVE>(lds + (size_t)t * stride, b, q0[u], q1[u]);
                dx[(size_t)b * TP + t] = d[u];
                if (HAS_MIN) sx[(size_t)b * TP + t] = sm[u];
            }
        }
    }
    return MmqAct{lds, dx, sx, stride};
}

// The same image from fp16 rows, quantized on the way in: d = amax / 127, q = round-half-away(v * 127 / amax),
// s = d * float(sum q) per 32-element block, exactly quantize_q8_1 (src/ops/gemv_q8dot.cpp:94-124), so the staged
// image is bit-identical to staging the quantizer's output.  One thread per (token, block).  `hrow(t)` -> row t.
template <int TV, bool HAS_MIN, bool NATIVE, class RowFn>
__device__ __forceinline__ MmqAct mmq_stage_f16(uint8_t* lds, RowFn hrow, uint32_t T, uint32_t k0, uint32_t kr, uint32_t K) {
    constexpr uint32_t TP = 2 * TV;
    const uint32_t stride = mmq_row_pitch(kr, NATIVE), nblk = kr / 32u;
    float* dx = reinterpret_cast<float*>(lds + (size_t)T * stride);
    float* sx = dx + (size_t)nblk * TP;
    const uint32_t total = T * nblk;
    for (uint32_t i = threadIdx.x; i < total; i += blockDim.x) {
        const uint32_t t = i / nblk, b = i - t * nblk;
        uint32_t q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        float d = 0.f, sm = 0.f;
        if (k0 + 32u * b < K) {
            const uint4* p = reinterpret_cast<const uint4*>(hrow(t) + k0 + 32u * b);
            const uint4 r0 = p[0], r1 = p[1], r2 = p[2], r3 = p[3];
            const uint32_t w[16] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w, r2.x, r2.y, r2.z, r2.w, r3.x, r3.y, r3.z, r3.w};
            float v[32];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                v[2 * j] = h2f(w[j] & 0xFFFFu);
                v[2 * j + 1] = h2f(w[j] >> 16);
            }
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(v[j]));
            d = amax / 127.0f;
            const float inv = amax > 0.f ? 127.0f / amax : 0.f;
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                uint32_t pk = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int qi = (int)roundf(v[4 * j + c] * inv);
                    sum += qi;
                    pk |= (uint32_t)(qi & 0xFF) << (8 * c);
                }
                q[j] = pk;
            }
            sm = d * (float)sum;
        }
        mmq_store_codes<NATIVE>(lds + (size_t)t * stride, b, make_uint4(q[0], q[1], q[2], q[3]), make_uint4(q[4], q[5], q[6], q[7]));
        dx[(size_t)b * TP + t] = d;
        if (HAS_MIN) sx[(size_t)b * TP + t] = sm;
    }
    return MmqAct{lds, dx, sx, stride};
}

// ---------------------------------------------------------------- one group of 8 blocks
template <int TV>
__device__ __forceinline__ void mmq_fold(const v16i_t& I, const float (&dxv)[TV], float c, float (&acc)[TV]) {
#pragma unroll
    for (int v = 0; v < TV; ++v) acc[v] += c * (dxv[v] * (float)I[v]);
}

template <int TV>
__device__ __forceinline__ void mmq_read4(const float* p, uint32_t h, float (&o)[TV]) {
    // token slots of lane half h: 8 q + 4 h + (0..3), q = 0 .. TV/4 - 1
#pragma unroll
    for (int q = 0; q < TV / 4; ++q) {
        const float4 f = *reinterpret_cast<const float4*>(p + 8 * q + 4 * h);
        o[4 * q] = f.x; o[4 * q + 1] = f.y; o[4 * q + 2] = f.z; o[4 * q + 3] = f.w;
    }
}

// Block S of group `gl` (group index inside the staged range).  The matrix instruction of block S + 1 is issued
// before the fold of block S, so the fold never waits on the instruction it depends on alone.
template <class P, int TV, int S>
__device__ __forceinline__ void mmq_block(const typename P::Raw& raw, const typename P::Dec& dec, const MmqAct& act, uint32_t a_off, uint32_t gl,
                                          uint32_t h, float (&acc)[TV], v16i_t (&I)[2][P::SUBS]) {
    constexpr uint32_t TP = 2 * TV;
    if constexpr (S < 8) {
        constexpr int cur = S & 1, nxt = cur ^ 1;
        if constexpr (S + 1 < 8) {
            const v4i_t a = as_v4i(*reinterpret_cast<const uint4*>(act.plane + a_off + (8u * gl + S + 1) * 32u));
            const v4i_t b = P::template operand<S + 1>(raw, h);
            const v16i_t z = {};
            if constexpr (P::SUBS == 1) {
                I[nxt][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, z, 0, 0, 0);
            } else {
                const v4i_t zero = {};
                I[nxt][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(h ? zero : a, b, z, 0, 0, 0);
                I[nxt][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(h ? a : zero, b, z, 0, 0, 0);
            }
        }
        float dxv[TV];
        mmq_read4<TV>(act.dx + (size_t)(8u * gl + S) * TP, h, dxv);
        if constexpr (P::SUBS == 1) {
            mmq_fold<TV>(I[cur][0], dxv, dec.c[S], acc);
        } else {
            mmq_fold<TV>(I[cur][0], dxv, dec.c[2 * S], acc);
            mmq_fold<TV>(I[cur][1], dxv, dec.c[2 * S + 1], acc);
        }
        if constexpr (P::HAS_MIN) {
            float sxv[TV];
            mmq_read4<TV>(act.sx + (size_t)(8u * gl + S) * TP, h, sxv);
#pragma unroll
            for (int v = 0; v < TV; ++v) acc[v] -= dec.m[S] * sxv[v];
        }
        mmq_block<P, TV, S + 1>(raw, dec, act, a_off, gl, h, acc, I);
    }
}

template <class P, int TV>
__device__ __forceinline__ void mmq_group(const typename P::Raw& raw, const MmqAct& act, uint32_t a_off, uint32_t gl, uint32_t h, float (&acc)[TV]) {
    const typename P::Dec dec = P::prepare(raw, h);
    v16i_t I[2][P::SUBS];
    {
        const v4i_t a = as_v4i(*reinterpret_cast<const uint4*>(act.plane + a_off + (8u * gl) * 32u));
        const v4i_t b = P::template operand<0>(raw, h);
        const v16i_t z = {};
        if constexpr (P::SUBS == 1) {
            I[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, z, 0, 0, 0);
        } else {
            const v4i_t zero = {};
            I[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(h ? zero : a, b, z, 0, 0, 0);
            I[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(h ? a : zero, b, z, 0, 0, 0);
        }
    }
    mmq_block<P, TV, 0>(raw, dec, act, a_off, gl, h, acc, I);
}

// Groups [g_lo, g_hi) of weight row `n` (row-relative group numbers) against the staged range that starts at group
// `g_base`.  One group of weight words is in flight while the previous one is multiplied (two register sets, never
// copied, no load under a branch that a later iteration depends on).  Measured on this part: a wave streams best
// with about eight 16-byte loads outstanding; deeper per-wave prefetch loses to more waves (a 58.7 MB read as 1792
// walks of 32 rows x 1 KB: everything requested up front 13.0 us, one group ahead 11.7 us).
template <class P, int TV>
struct MmqWalk {
    typename P::Raw raw[2];
    // the first group, requested by the caller before it stages the activations (it does not depend on them)
    __device__ __forceinline__ void prefetch(const typename P::W& w, uint32_t n, uint32_t g_lo, uint32_t, uint32_t h, uint32_t nb) { raw[0] = P::load(w, n, g_lo, h, nb); }
    // the partial last group of a row (block count not a multiple of 8), outside the pipeline
    __device__ __forceinline__ void tail(const typename P::W& w, uint32_t n, uint32_t g, uint32_t g_base, uint32_t h, uint32_t nb, const MmqAct& act,
                                         uint32_t a_off, float (&acc)[TV]) {
        if constexpr (P::K_ALIGN != 256) {
            const typename P::Raw r = P::load_tail(w, n, g, h, nb);
            mmq_group<P, TV>(r, act, a_off, g - g_base, h, acc);
        }
    }
    __device__ __forceinline__ void run(const typename P::W& w, uint32_t n, uint32_t g_lo, uint32_t g_hi, uint32_t g_base, uint32_t h, uint32_t nb,
                                        const MmqAct& act, uint32_t a_off, float (&acc)[TV]) {
        uint32_t g = g_lo;
        while (g + 2 < g_hi) {   // at least three groups left: both loads of the round are real
            raw[1] = P::load(w, n, g + 1, h, nb);
            __builtin_amdgcn_sched_barrier(0);   // the loads stay ahead of the arithmetic
            mmq_group<P, TV>(raw[0], act, a_off, g - g_base, h, acc);
            raw[0] = P::load(w, n, g + 2, h, nb);
            __builtin_amdgcn_sched_barrier(0);
            mmq_group<P, TV>(raw[1], act, a_off, g + 1 - g_base, h, acc);
            g += 2;
        }
        if (g + 1 < g_hi) {
            raw[1] = P::load(w, n, g + 1, h, nb);
            __builtin_amdgcn_sched_barrier(0);
            mmq_group<P, TV>(raw[0], act, a_off, g - g_base, h, acc);
            mmq_group<P, TV>(raw[1], act, a_off, g + 1 - g_base, h, acc);
        } else {
            mmq_group<P, TV>(raw[0], act, a_off, g - g_base, h, acc);
        }
    }
};

// ---------------------------------------------------------------- native FP4: one group = four block pairs
// `a_off` = row_a * pitch + 64 * (j / 16) + 16 h for token row_a = min(j % 16, live rows - 1): the lane's hi chunk of block
// 2 s + j / 16 of the pair; the lo chunk lies 32 bytes on.  keep_lo / keep_hi: all ones in the lanes whose data belongs in
// bytes 0..15 / 16..31 of the operand (j < 16 / j >= 16).
template <class P, int TV, int S>
__device__ __forceinline__ void mmq_pair_issue(const typename P::Raw& raw, const MmqAct& act, uint32_t a_off, uint32_t gl, uint32_t g, uint32_t nb,
                                               uint32_t keep_lo, uint32_t keep_hi, v16f_t& C) {
    const uint8_t* ap = act.plane + a_off + (8u * gl + 2u * S) * 64u;
    const uint4 xh = *reinterpret_cast<const uint4*>(ap), xl = *reinterpret_cast<const uint4*>(ap + 32);
    const v8i_t ah = {(int)(xh.x & keep_lo), (int)(xh.y & keep_lo), (int)(xh.z & keep_lo), (int)(xh.w & keep_lo),
                      (int)(xh.x & keep_hi), (int)(xh.y & keep_hi), (int)(xh.z & keep_hi), (int)(xh.w & keep_hi)};
    const v8i_t al = {(int)(xl.x & keep_lo), (int)(xl.y & keep_lo), (int)(xl.z & keep_lo), (int)(xl.w & keep_lo),
                      (int)(xl.x & keep_hi), (int)(xl.y & keep_hi), (int)(xl.z & keep_hi), (int)(xl.w & keep_hi)};
    const v8i_t b = {(int)raw.q[S].x, (int)raw.q[S].y, (int)raw.q[S].z, (int)raw.q[S].w, 0, 0, 0, 0};
    const v16f_t z = {};
    constexpr int sa = 0x7F83;              // byte 0: 2^4 for the hi operand, byte 1: 2^0 for the lo operand
    const int sb = P::template scale_word<S>(raw, g, (threadIdx.x >> 5) & 1u, nb);   // the block exponent of this lane half in byte 0
    C = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ah, b, z, 0, 4, 0, sa, 0, sb);
    C = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(al, b, C, 0, 4, 1, sa, 0, sb);
}

template <class P, int TV, int S>
__device__ __forceinline__ void mmq_pair(const typename P::Raw& raw, const MmqAct& act, uint32_t a_off, uint32_t gl, uint32_t g, uint32_t nb, uint32_t h,
                                         uint32_t keep_lo, uint32_t keep_hi, float (&acc)[TV], v16f_t (&C)[2]) {
    constexpr uint32_t TP = 2 * TV;
    if constexpr (S < 4) {
        constexpr int cur = S & 1, nxt = cur ^ 1;
        if constexpr (S + 1 < 4) mmq_pair_issue<P, TV, S + 1>(raw, act, a_off, gl, g, nb, keep_lo, keep_hi, C[nxt]);
        float dx0[TV], dx1[TV];
        mmq_read4<TV>(act.dx + (size_t)(8u * gl + 2u * S) * TP, h, dx0);
        mmq_read4<TV>(act.dx + (size_t)(8u * gl + 2u * S + 1u) * TP, h, dx1);
        {
            // each product is rounded on its own before it is added (the fold of the other kernels: acc += c * (d_x * idot))
#pragma clang fp contract(off)
#pragma unroll
            for (int v = 0; v < TV; ++v) {
                const float p0 = dx0[v] * C[cur][v];
                acc[v] += p0;
            }
#pragma unroll
            for (int v = 0; v < TV; ++v) {
                const float p1 = dx1[v] * C[cur][8 + v];
                acc[v] += p1;
            }
        }
        mmq_pair<P, TV, S + 1>(raw, act, a_off, gl, g, nb, h, keep_lo, keep_hi, acc, C);
    }
}

template <class P, int TV>
__device__ __forceinline__ void mmq_group_native(const typename P::Raw& raw, const MmqAct& act, uint32_t a_off, uint32_t g, uint32_t g_base, uint32_t nb,
                                                 uint32_t h, float (&acc)[TV]) {
    static_assert(TV <= 8, "a pass of the native FP4 path holds at most 16 tokens");
    const uint32_t keep_lo = (threadIdx.x & 16u) ? 0u : 0xFFFFFFFFu, keep_hi = ~keep_lo;
    v16f_t C[2];
    mmq_pair_issue<P, TV, 0>(raw, act, a_off, g - g_base, g, nb, keep_lo, keep_hi, C[0]);
    mmq_pair<P, TV, 0>(raw, act, a_off, g - g_base, g, nb, h, keep_lo, keep_hi, acc, C);
}

// The walk of the native path: a group is 18 registers, so three groups are in flight behind the one being multiplied.
// Slots past the end of the walk load one broadcast address (no load sits under a branch).
template <class P, int TV>
struct MmqWalkNative {
    typename P::Raw raw[4];
    __device__ __forceinline__ void prefetch(const typename P::W& w, uint32_t n, uint32_t g_lo, uint32_t g_hi, uint32_t h, uint32_t nb) {
#pragma unroll
        for (int u = 0; u < 3; ++u) raw[u] = P::load(w, n, g_lo + u, h, nb, g_lo + u < g_hi);
    }
    // partial groups run through the pipeline like whole ones
    __device__ __forceinline__ void tail(const typename P::W&, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, const MmqAct&, uint32_t, float (&)[TV]) {}
    __device__ __forceinline__ void run(const typename P::W& w, uint32_t n, uint32_t g_lo, uint32_t g_hi, uint32_t g_base, uint32_t h, uint32_t nb,
                                        const MmqAct& act, uint32_t a_off, float (&acc)[TV]) {
        for (uint32_t g = g_lo; g < g_hi; g += 4) {
            raw[3] = P::load(w, n, g + 3, h, nb, g + 3 < g_hi);
            __builtin_amdgcn_sched_barrier(0);
            mmq_group_native<P, TV>(raw[0], act, a_off, g, g_base, nb, h, acc);
            raw[0] = P::load(w, n, g + 4, h, nb, g + 4 < g_hi);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 < g_hi) mmq_group_native<P, TV>(raw[1], act, a_off, g + 1, g_base, nb, h, acc);
            raw[1] = P::load(w, n, g + 5, h, nb, g + 5 < g_hi);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 2 < g_hi) mmq_group_native<P, TV>(raw[2], act, a_off, g + 2, g_base, nb, h, acc);
            raw[2] = P::load(w, n, g + 6, h, nb, g + 6 < g_hi);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 3 < g_hi) mmq_group_native<P, TV>(raw[3], act, a_off, g + 3, g_base, nb, h, acc);
        }
    }
};


// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global load of the
// wave (its fence covers global memory), which would drain the weight words requested ahead of the barrier; here only the
// LDS counter is waited for, so those loads stay in flight across the barrier.
__device__ __forceinline__ void mmq_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---------------------------------------------------------------- kernel
enum { MMQ_STORE = 0, MMQ_SILU = 1, MMQ_OAI = 2, MMQ_DOWN_WEIGHTED = 3, MMQ_DOWN_BIAS = 4 };

template <class P>
struct MmqArgs {
    typename P::Bank bank0, bank1;    // NW = 2: gate and up
    const uint8_t* xq8;               // q8 rows (block_q8_1x, or block_q8_1s when q8_split)
    const half_t* act_f16;            // when set: the rows arrive as fp16 [rows][K] and are quantized while they are staged
    const uint32_t* expert_offsets;   // grouped: rows [off[e], off[e+1]) belong to expert e = blockIdx.y; NULL: one matrix, rows [0, M)
    half_t* out;                      // [rows][N] fp16
    float* part;                      // dense K ranges across workgroups (gridDim.z > 1): part[(z * M + row) * N + n]
    const float* bias0;               // [E][N] or NULL
    const float* bias1;
    const half_t* route_w;            // MMQ_DOWN_WEIGHTED: [rows]
    float alpha, limit;
    uint32_t M, K, N, E;
    uint32_t q8_split;
    uint32_t kr;                      // staged k range per pass (multiple of 256 WK)
    uint32_t red_off;                 // byte offset of the partial-sum exchange area in LDS: behind the staged image, or 0 = over it
    uint32_t deal_rows;               // one matrix with many rows [0, M): gridDim.z deals the token tiles (no K ranges, no `part`)
};

__device__ __forceinline__ float mmq_silu_mul(float g, float u) { return (g / (1.f + __expf(-g))) * u; }
__device__ __forceinline__ float mmq_swiglu_oai(float g, float u, float alpha, float limit) {
    const float x = fminf(g, limit), z = fmaxf(fminf(u, limit), -limit);
    return (x / (1.f + __expf(alpha * -x))) * (z + 1.f);
}

// Grid: x = workgroups per expert (each takes the blocks of 32 WR weight rows x, x + gridDim.x, ...), y = expert (grouped)
// or 1, z = K range (dense, with `part`) or token tile dealing (grouped).  Workgroup = NW x WR x WK waves.  A pass covers
// up to 2 TV token rows: T <= 8 (TV = 4), 16 (TV = 8), 32 (TV = 16); an expert with more rows runs several passes over
// its weights.  When one staged image covers the whole K range (the usual case) it is built once per token tile and every
// row block of the workgroup runs against it; the first weight words of the next row block are requested before the
// partial sums of the current one meet, so a workgroup with several row blocks streams without gaps.
// LDS: the staged image, then `red` [waves][TV][64] floats where the partial sums of the WK waves (and the NW matrices) meet.
template <class P, int TV, int NW, int WR, int WK, int EPI>
__global__ __launch_bounds__(64 * NW * WR * WK, 2) void mmq_kernel(MmqArgs<P> a) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr uint32_t TT = 2 * TV;   // token rows per pass
    constexpr bool NATIVE = mmq_native<P>::value;
    const uint32_t lane = threadIdx.x & 63u, j = lane & 31u, h = lane >> 5;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t wk = wave % WK, wr = (wave / WK) % WR, wm = wave / (WK * WR);
    uint32_t e = 0, r_begin = 0, r_end = a.M;
    if (a.expert_offsets) {
        e = blockIdx.y;
        r_begin = a.expert_offsets[e];
        r_end = a.expert_offsets[e + 1];
        if (r_begin >= r_end) return;   // empty expert (src/ops/moe_q8.cpp:211)
    }
    const typename P::W w = P::expert((NW == 2 && wm) ? a.bank1 : a.bank0, e);
    const uint32_t nb = a.K / 32u, n_groups = (nb + 7u) / 8u;
    const uint32_t n_rb = (a.N + 32u * WR - 1u) / (32u * WR);
    // gridDim.z: dense launches split K into ranges (partial sums to `part`); grouped launches deal the token tiles of an
    // expert round-robin, so that an expert with many rows is spread over many workgroups
    const bool grouped = a.expert_offsets != nullptr || a.deal_rows != 0;
    const uint32_t kz = grouped ? 1u : gridDim.z, kzi = grouped ? 0u : blockIdx.z;
    const uint32_t gz = (n_groups + kz - 1u) / kz;
    const uint32_t G0 = kzi * gz, G1 = G0 + gz < n_groups ? G0 + gz : n_groups;
    const uint32_t t_step = grouped ? gridDim.z * 2u * TV : 2u * TV, t_first = grouped ? blockIdx.z * 2u * TV : 0u;
    const uint32_t gp = a.kr / 256u;                     // groups per pass (multiple of WK)
    const bool single = G1 - G0 <= gp && a.red_off != 0; // one image covers the K range and is not overlaid by the exchange area
    const size_t q8_row_bytes = (size_t)nb * (a.q8_split ? kQ81sBytes : kQ81xBytes);
    float* red = reinterpret_cast<float*>(lds + a.red_off);

    for (uint32_t t0 = r_begin + t_first; t0 < r_end; t0 += t_step) {
        const uint32_t nt = r_end - t0 < TT ? r_end - t0 : TT;
        auto xrow = [&](uint32_t t) { return a.xq8 + (size_t)(t0 + t) * q8_row_bytes; };
        auto hrow = [&](uint32_t t) { return a.act_f16 + (size_t)(t0 + t) * a.K; };
        // token rows past the tile re-read its last row (their results are dropped)
        const uint32_t jt = NATIVE ? (j & 15u) : j, row_a = jt < nt ? jt : nt - 1u;
        typename std::conditional<NATIVE, MmqWalkNative<P, TV>, MmqWalk<P, TV>>::type walk;
        MmqAct act{};
        bool staged = false, requested = false;
        // what the epilogue reads from global memory is requested ahead of the weight walk: a load issued in the epilogue
        // would have to wait for the whole queue of weight words requested for the next row block before it
        float rw[TV];
#pragma unroll
        for (int v = 0; v < TV; ++v) {
            const uint32_t t = 8u * (v / 4) + 4u * h + (v % 4);
            rw[v] = (EPI == MMQ_DOWN_WEIGHTED) ? (float)a.route_w[t0 + (t < nt ? t : nt - 1u)] : 0.f;
        }
        for (uint32_t rb = blockIdx.x; rb < n_rb; rb += gridDim.x) {
            const uint32_t n0 = (rb * WR + wr) * 32u;
            const uint32_t n = n0 + j < a.N ? n0 + j : a.N - 1u;
            // MMQ_OAI: the bias of this wave's matrix joins its partial sum before the exchange (wave wk = 0 of each matrix);
            // MMQ_DOWN_BIAS: added after the fp16 rounding of the sum, in the epilogue
            float bias_a = 0.f;
            if (EPI == MMQ_OAI || EPI == MMQ_DOWN_BIAS) {
                const float* bp = (NW == 2 && wm) ? a.bias1 : a.bias0;
                if (bp) bias_a = bp[(size_t)e * a.N + n];
            }
            float acc[TV];
#pragma unroll
            for (int v = 0; v < TV; ++v) acc[v] = 0.f;
            for (uint32_t gb = G0; gb < G1; gb += gp) {
                const uint32_t ge = gb + gp < G1 ? gb + gp : G1;          // groups [gb, ge) of this pass
                const uint32_t per = (ge - gb + WK - 1u) / WK;
                const uint32_t g_lo = gb + wk * per < ge ? gb + wk * per : ge, g_hi = g_lo + per < ge ? g_lo + per : ge;
                // the pipeline takes whole groups and a partial last group follows it, except where the producer loads both alike
                const uint32_t g_full = (NATIVE || g_hi < nb / 8u) ? g_hi : nb / 8u;
                if (!requested && g_lo < g_full) walk.prefetch(w, n, g_lo, g_full, h, nb);
                requested = false;
                if (!staged) {
                    mmq_lds_barrier();                                        // the image of the previous pass is no longer read
                    act = a.act_f16 ? mmq_stage_f16<TV, P::HAS_MIN, NATIVE>(lds, hrow, nt, gb * 256u, (ge - gb) * 256u, a.K)
                                    : mmq_stage<TV, P::HAS_MIN, NATIVE>(lds, xrow, nt, gb * 256u, (ge - gb) * 256u, a.K, a.q8_split != 0);
                    mmq_lds_barrier();
                    staged = single;
                }
                const uint32_t a_off = row_a * act.stride + 16u * h + (NATIVE ? 64u * (j >> 4) : 0u);
                if (g_lo < g_full) walk.run(w, n, g_lo, g_full, gb, h, nb, act, a_off, acc);
                if (g_hi > g_full && g_lo <= g_full) walk.tail(w, n, g_full, gb, h, nb, act, a_off, acc);
                // the epilogue's operands are made to arrive here, while nothing else is outstanding: otherwise the wait for
                // them would sit in the epilogue, behind the weight words requested just below
                asm volatile("" : "+v"(bias_a));
#pragma unroll
                for (int v = 0; v < TV; ++v) asm volatile("" : "+v"(rw[v]));
                if (EPI == MMQ_OAI && ge == G1 && wk == 0) {
#pragma unroll
                    for (int v = 0; v < TV; ++v) acc[v] += bias_a;
                }
                if (single && rb + gridDim.x < n_rb && g_lo < g_full) {
                    // the next row block's first weight words, requested before the partial sums of this one meet
                    const uint32_t nn0 = ((rb + gridDim.x) * WR + wr) * 32u;
                    walk.prefetch(w, nn0 + j < a.N ? nn0 + j : a.N - 1u, g_lo, g_full, h, nb);
                    requested = true;
                }
            }
            // ---- partial sums of the WK waves (and the NW matrices) meet in LDS
            mmq_lds_barrier();
#pragma unroll
            for (int v = 0; v < TV; ++v) red[((size_t)wave * TV + v) * 64u + lane] = acc[v];
            mmq_lds_barrier();
            if (wk == 0 && wm == 0) {
#pragma unroll
                for (int v = 0; v < TV; ++v) {
                    const uint32_t t = 8u * (v / 4) + 4u * h + (v % 4);
                    float s0 = 0.f, s1 = 0.f;
#pragma unroll
                    for (int k = 0; k < WK; ++k) {
                        s0 += red[((size_t)((0 * WR + wr) * WK + k) * TV + v) * 64u + lane];
                        if (NW == 2) s1 += red[((size_t)((1 * WR + wr) * WK + k) * TV + v) * 64u + lane];
                    }
                    if (t >= nt || n0 + j >= a.N) continue;
                    const uint32_t row = t0 + t, col = n0 + j;
                    if (a.part) {
                        a.part[((size_t)kzi * a.M + row) * a.N + col] = s0;
                        continue;
                    }
                    float o;
                    if (EPI == MMQ_SILU) {
                        o = mmq_silu_mul(s0, s1);                                          // src/ops/moe_q8.cpp:94-97
                    } else if (EPI == MMQ_OAI) {
                        // rounding points of the reference chain: half(acc + bias) per projection, then the fp16 activation
                        const float g = (float)(half_t)s0, u = (float)(half_t)s1;   // sums with their biases
                        o = mmq_swiglu_oai(g, u, a.alpha, a.limit);
                    } else if (EPI == MMQ_DOWN_WEIGHTED) {
                        o = rw[v] * s0;                                                   // src/ops/moe_q8.cpp:143-144
                    } else if (EPI == MMQ_DOWN_BIAS) {
                        o = (float)(half_t)s0;                                            // gemv out, then add_bias (elementwise.cpp:782-793)
                        if (a.bias0) o += bias_a;
                    } else {
                        o = s0;
                    }
                    a.out[(size_t)row * a.N + col] = (half_t)o;
                }
            }
        }
    }
}

// reduction of the K ranges of a dense launch, in range order
static __global__ __launch_bounds__(256) void mmq_reduce_kernel(half_t* y, const float* part, uint32_t mn, uint32_t n_split) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= mn) return;
    float v = 0.f;
    for (uint32_t k = 0; k < n_split; ++k) v += part[(size_t)k * mn + i];
    y[i] = (half_t)v;
}

}  // namespace mxq
