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
//   tokens    : the fp16 A chunk [128 x 128] is staged in LDS (double buffered, unpadded
//               256-byte rows whose 16-byte columns are XOR-swizzled by the row number, so a
//               fragment read is bank-conflict free) and shared by the four waves;
//   weights   : lane (r = lane%32, h = lane/32) of a wave owns weight row r of a tile
//               and the 64 consecutive elements [64h, 64h+64) of the chunk: it loads
//               them from global as 128-bit words (32 B of Q4_K nibbles or 64 B of
//               Q8_0 quants), unpacks scale/min once per chunk and emits, for MFMA
//               step s, the 8 halfs of elements 64h + 8s .. +7 — exactly the MFMA
//               operand layout (lane%32 = row, lane/32 = k group), so no LDS round
//               trip and no redundant dequantisation inside a workgroup.
// The k order inside a chunk is (lanes 0-31: 8s.., lanes 32-63: 64+8s..); the
// A fragments are read from LDS with the same order, so the products pair up.
#include <type_traits>

#include "mxq_formats.h"
#include "mxq_host.h"

namespace mxq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float2_t __attribute__((ext_vector_type(2)));

constexpr int kBK = 128;            // K chunk
constexpr int kWaveN = 64;          // weight rows per wave (2 MFMA tiles)
constexpr int kGemmThreads = 256;
// One A chunk in LDS: BM rows x 256 B, unpadded, 16-byte columns XOR-swizzled by row.

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const float2_t f = {a, b};
    const half2_t h = __builtin_convertvector(f, half2_t);   // v_cvt_pk_f16_f32, RNE
    return __builtin_bit_cast(uint32_t, h);
}

// Two consecutive weights of a fragment from integer codes held as fp16 subnormals: the bits
// 0x0000 | u (u < 1024) read as fp16 are exactly u * 2^-24, so half(fma(u * 2^-24, scale * 2^24, off))
// is the dequantized weight with the integer -> float conversion folded into the operand
// (v_fma_mix_f32: fp16 source, fp32 scale/offset, fused fp32 multiply-add), then one RNE pack to
// fp16 (v_cvt_pk_f16_f32).  The power-of-two rescale of `scale` is exact, so the value is
// bit-identical to converting the code to float first.  Left to itself the compiler fuses
// convert + fma + convert into v_fma_mixlo/mixhi_f16, which measures about half the rate of the
// other VALU ops next to MFMA work on this chip; spelling the pack as an instruction keeps the two
// halves apart.
__device__ __forceinline__ uint32_t mix_pair(_Float16 x0, _Float16 x1, float scale, float off) {
    const float f0 = __builtin_fmaf((float)x0, scale, off), f1 = __builtin_fmaf((float)x1, scale, off);
    uint32_t r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(f0), "v"(f1));
    return r;
}
__device__ __forceinline__ half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// Four int8 of a dword to four fp16 (sub-dword addressed converts with sign extension: exact, |q| <= 128), then times a
// packed fp16 scale: half(d * q) with one rounding of the exact product, which is what rounding the fp32 product d * q
// (exact in fp32: 11 + 8 bits) to fp16 gives.  Six instructions for four weights (bias flip, two byte permutes, four
// mixed-precision multiply-adds and two packs before).
__device__ __forceinline__ void q8x4_scaled(uint32_t w, uint32_t d2, uint32_t& o01, uint32_t& o23) {
    uint32_t lo, hi;
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(lo) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1" : "+v"(lo) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(hi) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3" : "+v"(hi) : "v"(w));
    o01 = __builtin_bit_cast(uint32_t, as_h2(lo) * as_h2(d2));
    o23 = __builtin_bit_cast(uint32_t, as_h2(hi) * as_h2(d2));
}

union Frag {
    half8_t v;
    uint32_t u[4];
    uint4 q;
};

// ---------------------------------------------------------------- weight fragment producers
// Q4_K: chunk kc of a row = half c = kc%2 of block kc/2; lane half h owns the 32 bytes
// qs[32g, 32g+32), g = 2c + h: low nibbles = sub-block 2g, high = sub-block 2g+1.
// value = half(fma(d*sc, q, -(dmin*m))): the products are exact in fp32, so this is the single
// fp32 rounding of the reference expression followed by one RNE to fp16.  A low nibble is the
// subnormal q * 2^-24, a high nibble stays in place as q * 2^-20.
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
        float d1[2], c1[2];
    };
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr uint32_t H_COL = 8;                                   // 16-byte A column of lane half h at step 0
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }   // A column offset of step S
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
        o.d1[0] = d * (float)(sc & 0xFFu) * 16777216.f;   // x 2^24
        o.d1[1] = d * (float)(sc >> 8) * 1048576.f;       // x 2^20
        o.c1[0] = -(dmin * (float)(mn & 0xFFu));
        o.c1[1] = -(dmin * (float)(mn >> 8));
        return o;
    }
    // Half HF of the fragment of step S: elements 4 HF .. 4 HF + 3 (words u[2 HF], u[2 HF + 1]).
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int sub = S / 4, p = S % 4;
        const uint32_t w = HF == 0 ? (p == 0 ? r.q0.x : p == 1 ? r.q0.z : p == 2 ? r.q1.x : r.q1.z)
                                   : (p == 0 ? r.q0.y : p == 1 ? r.q0.w : p == 2 ? r.q1.y : r.q1.w);
        constexpr uint32_t mask = sub ? 0x00F000F0u : 0x000F000Fu;
        const half2_t ev = as_h2(w & mask), od = as_h2((w >> 8) & mask);   // bytes (0,2), (1,3)
        const float d1 = dc.d1[sub], c1 = dc.c1[sub];
        f.u[2 * HF] = mix_pair(ev.x, od.x, d1, c1);
        f.u[2 * HF + 1] = mix_pair(ev.y, od.y, d1, c1);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// Q8_0 SoA planes: lane half h owns quants [128 kc + 64h, +64) of the row and the two
// block scales.  value = half(d * q) (exact product, one RNE to fp16): the byte is converted to fp16
// where it sits (q8x4_scaled) and multiplied by the fp16 scale in packed fp16.
struct GemmQ8SoaLds;
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
        uint32_t dh[2];   // the two block scales, each in both halves of a dword
    };
    static constexpr uint32_t K_ALIGN = 128;
    static constexpr uint32_t H_COL = 8;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint4* p = reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)kc * 128u + 64u * h);
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r.q[i] = p[i];
        r.d2 = *reinterpret_cast<const uint32_t*>(w.d + (size_t)n * (w.K >> 5) + kc * 4u + 2u * h);
        return r;
    }
    __device__ static __forceinline__ Dec dec_of(uint32_t d2) {
        Dec o;
        o.dh[0] = __builtin_amdgcn_perm(0u, d2, 0x01000100u);
        o.dh[1] = __builtin_amdgcn_perm(0u, d2, 0x03020302u);
        return o;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t) { return dec_of(r.d2); }
    using LdsScales = GemmQ8SoaLds;   // the producer of expert-grouped tiles whose scale table fits in LDS
    template <int S, int HF, class RawT>
    __device__ static __forceinline__ void frag_half(const RawT& r, const Dec& dc, Frag& f) {
        constexpr int blk = S / 4, i = (S * 2) / 4, e = (S * 2) % 4;
        const uint32_t w = HF == 0 ? (e == 0 ? r.q[i].x : r.q[i].z) : (e == 0 ? r.q[i].y : r.q[i].w);
        q8x4_scaled(w, dc.dh[blk], f.u[2 * HF], f.u[2 * HF + 1]);
    }
    template <int S, class RawT>
    __device__ static __forceinline__ void frag(const RawT& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// The same planes with the scales of the workgroup's 256 weight rows copied into an LDS table at the start of the tile
// (every K chunk of them, 2 K / 32 bytes per row).  Read per chunk from global memory, the two scales a lane needs cost
// one cache line request per row and chunk, as many as the quants of the chunk (the line holds the scales of 16
// chunks, but the quants streaming through the L1 evict it before the next chunk), and a CU runs out of outstanding
// line requests long before it runs out of bytes: without the scale loads the expert-grouped launches are 10-16 %
// faster.  `Win` = the LDS byte address of the lane's row in the table.
struct GemmQ8SoaLds : GemmQ8Soa {
    struct Raw {
        uint4 q[4];
    };
    struct Win {
        uint32_t row;
    };
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint4* p = reinterpret_cast<const uint4*>(w.qs + (size_t)n * w.K + (size_t)kc * 128u + 64u * h);
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r.q[i] = p[i];
        return r;
    }
    // row pitch of the table: the scales of a row plus one dword, so that the 32 rows a wave reads at once fall into 32 banks
    __device__ __host__ static constexpr uint32_t table_pitch(uint32_t K) { return K / 16u + 4u; }
    __device__ static __forceinline__ const uint8_t* scales_of(const W& w, uint32_t n) { return reinterpret_cast<const uint8_t*>(w.d + (size_t)n * (w.K >> 5)); }
    __device__ static __forceinline__ Dec prepare(const Raw&, const Win& wn, uint32_t kc, uint32_t h) {
        typedef __attribute__((address_space(3))) const uint32_t lds_u32_t;
        return dec_of(*reinterpret_cast<lds_u32_t*>((uintptr_t)(wn.row + kc * 8u + 4u * h)));
    }
};

// Q8_0 AoS GGUF blocks (34 B: fp16 d, 32 int8): lane half h owns blocks 4 kc + 2h and + 1, 68
// contiguous bytes at a 2-byte aligned address, fetched as 17 dwords.  The quants of the first
// block start 2 bytes into a dword and are realigned with one byte-align per word; those of
// the second block (byte 36) are dword aligned.  Same arithmetic as the SoA planes.
struct GemmQ8Aos {
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
        uint32_t w[17];
    };
    struct Dec {
        uint32_t dh[2];   // the two block scales, each in both halves of a dword
    };
    static constexpr uint32_t K_ALIGN = 128;
    static constexpr uint32_t H_COL = 8;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes + (size_t)(4u * kc + 2u * h) * kQ8_0Bytes;
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint4 v = load_u4_a2(p + 16 * i);
            r.w[4 * i] = v.x; r.w[4 * i + 1] = v.y; r.w[4 * i + 2] = v.z; r.w[4 * i + 3] = v.w;
        }
        r.w[16] = load_u1_a2(p + 64);
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t) {
        Dec o;
        o.dh[0] = __builtin_amdgcn_perm(0u, r.w[0], 0x01000100u);
        o.dh[1] = __builtin_amdgcn_perm(0u, r.w[8], 0x03020302u);
        return o;
    }
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int blk = S / 4, j = 2 * (S % 4) + HF;   // word j of the block's 8 quant words
        uint32_t w;
        if (blk == 0) w = __builtin_amdgcn_alignbyte(r.w[j + 1], r.w[j], 2);   // bytes 2 + 4j .. 5 + 4j
        else w = r.w[9 + j];
        q8x4_scaled(w, dc.dh[blk], f.u[2 * HF], f.u[2 * HF + 1]);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// Q4_0 AoS GGUF blocks (18 B: fp16 d, 16 bytes of nibbles; element j in the low, j + 16 in the high
// nibble of qs[j]; include/ie/quant_blocks.hpp:32-43): lane half h owns blocks 4 kc + 2h and + 1, 36
// contiguous bytes at a 2-byte aligned address, fetched as 9 dwords.  Step S covers elements
// 8 (S%4) .. +7 of block S/4: the low nibbles of quant words 2 (S%2), 2 (S%2) + 1 for S%4 < 2, their high
// nibbles otherwise.  value = half(d * (q - 8)) = fma(q * 2^-24, d * 2^24, -8 d), exact in fp32.
struct GemmQ40 {
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
        uint32_t w[9];
    };
    struct Dec {
        float d[2], o[2];
    };
    static constexpr uint32_t K_ALIGN = 128;
    static constexpr uint32_t H_COL = 8;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint8_t* p = w.base + (size_t)n * w.row_bytes + (size_t)(4u * kc + 2u * h) * 18u;
        Raw r;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4 v = load_u4_a2(p + 16 * i);
            r.w[4 * i] = v.x; r.w[4 * i + 1] = v.y; r.w[4 * i + 2] = v.z; r.w[4 * i + 3] = v.w;
        }
        r.w[8] = load_u1_a2(p + 32);
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t) {
        Dec o;
        o.d[0] = h2f(r.w[0] & 0xFFFFu);
        o.d[1] = h2f(r.w[4] >> 16);
        o.o[0] = -8.f * o.d[0];
        o.o[1] = -8.f * o.d[1];
        o.d[0] *= 16777216.f;
        o.d[1] *= 16777216.f;
        return o;
    }
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int blk = S / 4, j = 2 * (S % 2) + HF, hi = (S % 4) / 2;   // quant word j of the block, nibble half
        uint32_t w;
        if (blk == 0) w = __builtin_amdgcn_alignbyte(r.w[j + 1], r.w[j], 2);   // bytes 2 + 4j .. 5 + 4j
        else w = r.w[5 + j];                                                   // bytes 20 + 4j ..
        const uint32_t code = (hi ? w >> 4 : w) & 0x0F0F0F0Fu;
        const float d = dc.d[blk], o = dc.o[blk];
        const half2_t w01 = as_h2(__builtin_amdgcn_perm(0u, code, 0x0C010C00u)), w23 = as_h2(__builtin_amdgcn_perm(0u, code, 0x0C030C02u));
        f.u[2 * HF] = mix_pair(w01.x, w01.y, d, o);
        f.u[2 * HF + 1] = mix_pair(w23.x, w23.y, d, o);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// Q6_K (210-byte AoS blocks, 2-byte aligned): chunk kc = 128-element half c = kc%2 of block
// kc/2.  Lane half j = lane/32 owns the 16 "l" positions 16j .. 16j+15 of that half, i.e. the
// four 16-element groups 32s + 16j + [0,16), s = 0..3 (include/ie/dequant_ref.hpp:78-96):
// ql[64c + 16j + ..] (groups 0 and 2 in its low / high nibbles), ql[64c + 32 + 16j + ..]
// (groups 1 and 3), qh[32c + 16j + ..] (the 2-bit tops of all four) and the scales
// scales[8c + 2s + j].  Step S covers group S/2, elements 8 (S%2) .. +7 of it, so the A column
// of a step is 4 (S/2) + 2j + S%2.
// value = half((d*sc) * (code - 32)): every product is exact in fp32; evaluated as
// fma(code * 2^-24, d*sc * 2^24, -32 d*sc) on the 6-bit code held as an fp16 subnormal.
struct GemmQ6K {
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
        uint4 qla, qlb, qh;
        uint2 sc;
        uint32_t d;
    };
    struct Dec {
        float c[4], o[4];
    };
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr uint32_t H_COL = 2;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)(((S >> 1) << 2) | (S & 1)); }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t j) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)(kc >> 1) * kQ6KBytes;
        const uint32_t c = kc & 1u;
        Raw r;
        r.qla = load_u4_a2(blk + 64u * c + 16u * j);
        r.qlb = load_u4_a2(blk + 64u * c + 32u + 16u * j);
        r.qh = load_u4_a2(blk + 128u + 32u * c + 16u * j);
        r.sc = load_u2_a2(blk + 192u + 8u * c);
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t j) {
        const float d = h2f(r.d);
        const uint32_t j8 = j * 8u;
        Dec o;
        o.c[0] = d * (float)(int)(int8_t)(r.sc.x >> j8);
        o.c[1] = d * (float)(int)(int8_t)(r.sc.x >> (16u + j8));
        o.c[2] = d * (float)(int)(int8_t)(r.sc.y >> j8);
        o.c[3] = d * (float)(int)(int8_t)(r.sc.y >> (16u + j8));
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            o.o[s] = -32.f * o.c[s];
            o.c[s] *= 16777216.f;
        }
        return o;
    }
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int s = S / 2, i = 2 * (S % 2) + HF;   // group, dword of the 16-byte slices
        const uint32_t la = i == 0 ? r.qla.x : i == 1 ? r.qla.y : i == 2 ? r.qla.z : r.qla.w;
        const uint32_t lb = i == 0 ? r.qlb.x : i == 1 ? r.qlb.y : i == 2 ? r.qlb.z : r.qlb.w;
        const uint32_t qh = i == 0 ? r.qh.x : i == 1 ? r.qh.y : i == 2 ? r.qh.z : r.qh.w;
        uint32_t code;
        if (s == 0) code = (la & 0x0F0F0F0Fu) | ((qh << 4) & 0x30303030u);
        else if (s == 1) code = (lb & 0x0F0F0F0Fu) | ((qh << 2) & 0x30303030u);
        else if (s == 2) code = ((la >> 4) & 0x0F0F0F0Fu) | (qh & 0x30303030u);
        else code = ((lb >> 4) & 0x0F0F0F0Fu) | ((qh >> 2) & 0x30303030u);
        const float c = dc.c[s], o = dc.o[s];
        const half2_t w01 = as_h2(__builtin_amdgcn_perm(0u, code, 0x0C010C00u)), w23 = as_h2(__builtin_amdgcn_perm(0u, code, 0x0C030C02u));
        f.u[2 * HF] = mix_pair(w01.x, w01.y, c, o);
        f.u[2 * HF + 1] = mix_pair(w23.x, w23.y, c, o);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// Q5_K (176-byte blocks: d, dmin, scales[12], qh[32], qs[128]; include/ie/quant_blocks.hpp): Q4_K's nibbles plus one
// high bit per element, bit j of qh[l] for sub-block j and position l.  Same chunk / lane-half split as Q4_K (lane half h
// owns qs[32 g, 32 g + 32), g = 2 (kc % 2) + h: sub-blocks 2 g in the low and 2 g + 1 in the high nibbles); the lane also
// keeps all 32 bytes of qh.  value = half(fma(d*sc, q, -(dmin*m))), q the 5-bit code held as an fp16 subnormal.
struct GemmQ5K {
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
        uint4 hdr, h0, h1, q0, q1;
    };
    struct Dec {
        float d1[2], c1[2];
        uint32_t bit;   // sub-block number of the low nibbles = bit of qh
    };
    static constexpr uint32_t K_ALIGN = 256;
    static constexpr uint32_t H_COL = 8;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const uint8_t* blk = w.base + (size_t)n * w.row_bytes + (size_t)(kc >> 1) * 176u;
        const uint4* q = reinterpret_cast<const uint4*>(blk + 48 + (2u * (kc & 1u) + h) * 32u);
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.h0 = *reinterpret_cast<const uint4*>(blk + 16);
        r.h1 = *reinterpret_cast<const uint4*>(blk + 32);
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t kc, uint32_t h) {
        const uint32_t g = 2u * (kc & 1u) + h;
        uint32_t sc, mn;
        q4k_scale_pair(r.hdr.y, r.hdr.z, r.hdr.w, (int)g, sc, mn);
        const float d = h2f(r.hdr.x & 0xFFFFu), dmin = h2f(r.hdr.x >> 16);
        Dec o;
        o.d1[0] = d * (float)(sc & 0xFFu) * 16777216.f;
        o.d1[1] = d * (float)(sc >> 8) * 16777216.f;
        o.c1[0] = -(dmin * (float)(mn & 0xFFu));
        o.c1[1] = -(dmin * (float)(mn >> 8));
        o.bit = 2u * g;
        return o;
    }
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int sub = S / 4, p = S % 4, wi = 2 * p + HF;   // word wi of the 32-byte nibble slice and of qh
        const uint32_t w = wi == 0 ? r.q0.x : wi == 1 ? r.q0.y : wi == 2 ? r.q0.z : wi == 3 ? r.q0.w : wi == 4 ? r.q1.x : wi == 5 ? r.q1.y : wi == 6 ? r.q1.z : r.q1.w;
        const uint32_t qh = wi == 0 ? r.h0.x : wi == 1 ? r.h0.y : wi == 2 ? r.h0.z : wi == 3 ? r.h0.w : wi == 4 ? r.h1.x : wi == 5 ? r.h1.y : wi == 6 ? r.h1.z : r.h1.w;
        const uint32_t code = ((sub ? w >> 4 : w) & 0x0F0F0F0Fu) | (((qh >> (dc.bit + sub)) & 0x01010101u) << 4);
        const half2_t ev = as_h2(code & 0x00FF00FFu), od = as_h2((code >> 8) & 0x00FF00FFu);   // bytes (0,2), (1,3)
        const float d1 = dc.d1[sub], c1 = dc.c1[sub];
        f.u[2 * HF] = mix_pair(ev.x, od.x, d1, c1);
        f.u[2 * HF + 1] = mix_pair(ev.y, od.y, d1, c1);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// MXFP4 planes (E2M1 codes, element j in the low and j + 16 in the high nibble of byte j of a 16-byte block; one E8M0
// exponent per block; include/ie/quant_blocks.hpp:46-54): lane half h owns blocks 4 kc + 2 h and + 1.  A code goes
// through the byte table of the int-dot kernels (doubled E2M1 value as int8), is bias-flipped into an unsigned byte and
// then takes the Q8_0 route: half(fma((b ^ 0x80) * 2^-24, s * 2^24, -128 s)) = half(b * s) with s = 2^(e-128), which is
// half(e2m1 * 2^(e-127)), the reference's dequantized weight (src/ops/dequant_kernels.cpp:325-390), bit for bit.
// Rows may end half way through a chunk (K % 128 = 64, e.g. K = 2880): the dead lane half re-reads the live one's
// bytes and gets scale 0.
struct GemmMxfp4Soa {
    struct W {
        const uint8_t* qs;
        const uint8_t* e;
        uint32_t K;
    };
    struct Bank {
        const uint8_t* qs;
        const uint8_t* e;
        uint64_t qs_stride, e_stride;
        uint32_t K;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) { return {b.qs + (size_t)e * b.qs_stride, b.e + (size_t)e * b.e_stride, b.K}; }
    struct Raw {
        uint4 q[2];
        uint32_t e0, e1;
        uint32_t live;
    };
    struct Dec {
        float d[2], o[2];
    };
    static constexpr uint32_t K_ALIGN = 64;
    static constexpr uint32_t H_COL = 8;
    __device__ static constexpr uint32_t step_col(int S) { return (uint32_t)S; }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const bool live = 128u * kc + 64u * h < w.K;
        const uint32_t b0 = 4u * kc + (live ? 2u * h : 0u);
        const uint4* p = reinterpret_cast<const uint4*>(w.qs + (size_t)n * (w.K >> 1) + (size_t)b0 * 16u);
        const uint8_t* e = w.e + (size_t)n * (w.K >> 5) + b0;
        Raw r;
        r.q[0] = p[0];
        r.q[1] = p[1];
        r.e0 = e[0];
        r.e1 = e[1];
        r.live = live ? 1u : 0u;
        return r;
    }
    __device__ static __forceinline__ Dec prepare(const Raw& r, uint32_t, uint32_t) {
        const float s0 = r.live ? e8m0_half(r.e0) : 0.f, s1 = r.live ? e8m0_half(r.e1) : 0.f;
        Dec o;
        o.d[0] = s0 * 16777216.f;
        o.d[1] = s1 * 16777216.f;
        o.o[0] = -128.f * s0;
        o.o[1] = -128.f * s1;
        return o;
    }
    template <int S, int HF>
    __device__ static __forceinline__ void frag_half(const Raw& r, const Dec& dc, Frag& f) {
        constexpr int blk = S / 4, j = 2 * (S % 2) + HF, hi = (S % 4) / 2;   // word j of the block, nibble half
        const uint32_t w = j == 0 ? r.q[blk].x : j == 1 ? r.q[blk].y : j == 2 ? r.q[blk].z : r.q[blk].w;
        const uint32_t nib = hi ? w >> 4 : w;
        const uint32_t b = mxfp4_lut4(nib & 0x07070707u, ((nib >> 1) & 0x04040404u) | 0x03020100u) ^ 0x80808080u;
        const float d = dc.d[blk], o = dc.o[blk];
        const half2_t w01 = as_h2(__builtin_amdgcn_perm(0u, b, 0x0C010C00u)), w23 = as_h2(__builtin_amdgcn_perm(0u, b, 0x0C030C02u));
        f.u[2 * HF] = mix_pair(w01.x, w01.y, d, o);
        f.u[2 * HF + 1] = mix_pair(w23.x, w23.y, d, o);
    }
    template <int S>
    __device__ static __forceinline__ void frag(const Raw& r, const Dec& dc, Frag& f) {
        frag_half<S, 0>(r, dc, f);
        frag_half<S, 1>(r, dc, f);
    }
};

// K-quant expert regions stored as per-field streams (include/ie/quant_soa.hpp:33-51,127-157: Q4_K qs[128] x nb |
// scales[12] x nb | {d,dmin}[4] x nb; Q6_K ql[128] x nb | qh[64] x nb | scales[16] x nb | d[2] x nb): the same words as
// the AoS blocks from other addresses, so fragments, scales and arithmetic are inherited.
struct GemmQ4KStr : GemmQ4K {
    struct W {
        const uint8_t* qs;
        const uint8_t* sc;
        const uint8_t* dm;
        uint32_t bpr;
    };
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint64_t nb;
        uint32_t bpr;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) {
        const uint8_t* p = b.base + (size_t)e * b.expert_stride_bytes;
        return {p, p + b.nb * 128u, p + b.nb * 140u, b.bpr};
    }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t h) {
        const size_t ib = (size_t)n * w.bpr + (kc >> 1);
        const uint4* q = reinterpret_cast<const uint4*>(w.qs + ib * 128u + (2u * (kc & 1u) + h) * 32u);
        const uint32_t* sc = reinterpret_cast<const uint32_t*>(w.sc + ib * 12u);
        Raw r;
        r.hdr = make_uint4(*reinterpret_cast<const uint32_t*>(w.dm + ib * 4u), sc[0], sc[1], sc[2]);
        r.q0 = q[0];
        r.q1 = q[1];
        return r;
    }
};
struct GemmQ6KStr : GemmQ6K {
    struct W {
        const uint8_t* ql;
        const uint8_t* qh;
        const uint8_t* sc;
        const uint8_t* d;
        uint32_t bpr;
    };
    struct Bank {
        const uint8_t* base;
        uint64_t expert_stride_bytes;
        uint64_t nb;
        uint32_t bpr;
    };
    __device__ static __forceinline__ W expert(const Bank& b, uint32_t e) {
        const uint8_t* p = b.base + (size_t)e * b.expert_stride_bytes;
        return {p, p + b.nb * 128u, p + b.nb * 192u, p + b.nb * 208u, b.bpr};
    }
    __device__ static __forceinline__ Raw load(const W& w, uint32_t n, uint32_t kc, uint32_t j) {
        const size_t ib = (size_t)n * w.bpr + (kc >> 1);
        const uint32_t c = kc & 1u;
        Raw r;
        r.qla = load_u4_a2(w.ql + ib * 128u + 64u * c + 16u * j);
        r.qlb = load_u4_a2(w.ql + ib * 128u + 64u * c + 32u + 16u * j);
        r.qh = load_u4_a2(w.qh + ib * 64u + 32u * c + 16u * j);
        r.sc = load_u2_a2(w.sc + ib * 16u + 8u * c);
        r.d = *reinterpret_cast<const uint16_t*>(w.d + ib * 2u);
        return r;
    }
};

// ---------------------------------------------------------------- kernel
// GEMM_MOE_GATE_UP_OAI: gpt-oss gate/up, out = half(swiglu_oai(half(g + bias_g), half(u + bias_u))) (src/ops/elementwise.cpp:
// 468-492); GEMM_MOE_DOWN with `bias0`: out = half(half(acc) + bias) (gemv out, then add_bias, elementwise.cpp:782-793).
enum { GEMM_DENSE = 0, GEMM_MOE_GATE_UP_SILU = 1, GEMM_MOE_DOWN = 2, GEMM_MOE_GATE_UP_OAI = 3 };

struct GemmArgs {
    const half_t* A;                  // [M, K] fp16 (dense) or expert-sorted rows [TK, K]
    half_t* Y;                        // [M, N]
    const uint32_t* expert_offsets;   // grouped: [E+1]
    const half_t* route_w;            // GEMM_MOE_DOWN: [TK] fp16 row weights, or NULL for unweighted rows
    const int32_t* a_row_index;       // grouped gate/up, gather form: A row of sorted row r is a_row_index[r] (A = the unsorted [T, K] rows)
    const int32_t* row_token;         // GEMM_MOE_DOWN, accumulate form: token of each sorted row
    float* y_acc;                     //   and the fp32 [T, N] buffer w * acc is atomically added into (Y unused)
    uint32_t M, K, N, E;
    uint32_t tiles_m, tiles_n;        // dense tile grid; grouped: tiles_m is an upper bound
    uint32_t k_split;                 // dense only: K slices per output tile (above 1: fp32 partial sums go to split_acc)
    float* split_acc;                 // [k_split][M][N] partial sums of a K-sliced launch
    const float* bias0;               // [E][N] fp32 or NULL: gate bias (GEMM_MOE_GATE_UP_OAI), down bias (GEMM_MOE_DOWN)
    const float* bias1;               // [E][N] up bias
    float alpha, limit;               // swiglu_oai
};

__device__ __forceinline__ float silu_mul_f(float g, float u) { return (g / (1.f + __expf(-g))) * u; }
__device__ __forceinline__ float swiglu_oai_f(float g, float u, float alpha, float limit) {
    const float x = fminf(g, limit), z = fmaxf(fminf(u, limit), -limit);
    return (x / (1.f + __expf(alpha * -x))) * (z + 1.f);
}

// Dense launches with too few output tiles for the chip (a short batch against a narrow matrix) cut K into up to
// eight slices: every slice writes its fp32 partial sums to its own plane of a scratch buffer, and a last launch adds
// the planes in slice order and rounds to fp16 (so the result does not depend on which slice finished first).  The
// scratch is a caller's workspace (the *_ws entry points) or the file-scope device array below, which the library
// owns (no entry point allocates): one copy per device, keeping the last call's contents; every element the last
// launch reads was written by the slices in front of it.  Launches that overlap on one device would race on it, as
// with the reference's static per-device scratch buffers (src/model/dense_dispatch.hpp:547-560).
constexpr uint64_t kGemmSplitElems = 8ull << 20;   // slices * M * N <= 8 Mi partial sums (32 MB)
constexpr uint32_t kGemmSplitMax = 8;
static __device__ __align__(256) float g_gemm_splitk_acc[kGemmSplitElems];
static std::atomic<void*> g_gemm_splitk_addr[kMaxDevices];

int gemm_init_device() {
    void* p = nullptr;
    return scratch_address(HIP_SYMBOL(g_gemm_splitk_acc), g_gemm_splitk_addr, &p);
}

__global__ __launch_bounds__(256) void gemm_splitk_store_kernel(half_t* y, const float* acc, uint32_t n, uint32_t k_split) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = acc[i];
    for (uint32_t k = 1; k < k_split; ++k) v += acc[(size_t)k * n + i];
    y[i] = (half_t)v;
}

typedef __attribute__((address_space(3))) void lds_void_t;

// 16 bytes per lane from global memory straight into LDS, no registers in between
// (global_load_lds_dwordx4: lane L of the wave lands at lds_addr + 16 L).  `base` and
// `lds_addr` are wave-uniform.  The load counts on vmcnt like any other global load; the
// data is visible in LDS once vmcnt has drained, so every consumer sits behind an explicit
// vmcnt(0) + workgroup barrier.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is a reserved register; naming it as clobbered is the intent
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t byte_off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(base), "v"(byte_off), "s"(lds_addr) : "memory", "m0");
}
#pragma clang diagnostic pop

// One K chunk = 8 MFMA steps.  A fragment (token row R, 16-byte column c) sits at
// R * 256 + ((c ^ (R & 15)) << 4): the 16 lanes of a quarter wave then hit 16 different
// columns, i.e. all 64 banks once.  For step S the column is QF::H_COL * h + QF::step_col(S),
// so the address is the lane's step-0 address XOR-ed with step_col(S) << 4.
// `mi` = number of live 32-token tiles of this workgroup tile (4 unless PARTIAL: expert-grouped
// tiles are often mostly empty, and their dead token tiles skip both the LDS reads and the MFMAs).
template <int S, class QF, bool PARTIAL, int NI>
__device__ __forceinline__ void mma_step(const typename QF::Raw (&raw)[2], const typename QF::Dec (&dec)[2], const uint8_t* lds, uint32_t a_frag0,
                                         float16_t (&acc)[NI][2], uint32_t mi) {
    Frag af[NI], bf[2];
    const uint32_t a_s = a_frag0 ^ (QF::step_col(S) << 4);
#pragma unroll
    for (int i = 0; i < NI; ++i)
        if (!PARTIAL || (uint32_t)i < mi) af[i].q = *reinterpret_cast<const uint4*>(lds + a_s + i * 8192);
    QF::template frag<S>(raw[0], dec[0], bf[0]);
    QF::template frag<S>(raw[1], dec[1], bf[1]);
#pragma unroll
    for (int i = 0; i < NI; ++i)
        if (!PARTIAL || (uint32_t)i < mi) {
            acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i].v, bf[0].v, acc[i][0], 0, 0, 0);
            acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i].v, bf[1].v, acc[i][1], 0, 0, 0);
        }
}

// The chunk as one software pipeline over NI token tiles, all of them multiplied (no branch inside a chunk: a branch
// per token tile ends the scheduling region, and each step then runs as LDS read, wait, dequantisation, MFMAs one after
// the other).  A step is cut into NI segments, one per token tile: its 2 MFMAs, the LDS read that refills that A
// fragment for step S+1, and 4 / NI of the four half-fragment dequantisations of the weight fragments of step S+1
// into the other fragment pair.  The scheduling fences between segments keep that interleaving, so neither the VALU
// work nor the LDS latency ends up between two clusters of MFMAs.
template <int S, class QF, int NI>
__device__ __forceinline__ void mma_pipe(const typename QF::Raw (&raw)[2], const typename QF::Dec (&dec)[2], const uint8_t* lds, uint32_t a_frag0,
                                         float16_t (&acc)[NI][2], Frag (&af)[NI], Frag (&bf)[2][2]) {
    static_assert(NI == 1 || NI == 2 || NI == 4, "token tiles per pipelined chunk");
    if constexpr (S < 8) {
        constexpr int cur = S & 1, nxt = cur ^ 1, SN = (S + 1) & 7;
        constexpr bool more = S + 1 < 8;
        constexpr int per = 4 / NI;   // half fragments dequantized per segment
        const uint32_t a_n = a_frag0 ^ (QF::step_col(SN) << 4);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i].v, bf[cur][0].v, acc[i][0], 0, 0, 0);
            acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i].v, bf[cur][1].v, acc[i][1], 0, 0, 0);
            if (more) {
                af[i].q = *reinterpret_cast<const uint4*>(lds + a_n + i * 8192);
#pragma unroll
                for (int q = i * per; q < (i + 1) * per; ++q) {
                    if (q == 0) QF::template frag_half<SN, 0>(raw[0], dec[0], bf[nxt][0]);
                    if (q == 1) QF::template frag_half<SN, 1>(raw[0], dec[0], bf[nxt][0]);
                    if (q == 2) QF::template frag_half<SN, 0>(raw[1], dec[1], bf[nxt][1]);
                    if (q == 3) QF::template frag_half<SN, 1>(raw[1], dec[1], bf[nxt][1]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        mma_pipe<S + 1, QF, NI>(raw, dec, lds, a_frag0, acc, af, bf);
    }
}

template <class QF, bool PIPE, bool PARTIAL, int NI>
__device__ __forceinline__ void mma_chunk(const typename QF::Raw (&raw)[2], const typename QF::Dec (&dec)[2], const uint8_t* lds, uint32_t a_frag0,
                                          float16_t (&acc)[NI][2], uint32_t mi) {
    if constexpr (PIPE) {
        Frag af[NI], bf[2][2];
#pragma unroll
        for (int i = 0; i < NI; ++i) af[i].q = *reinterpret_cast<const uint4*>(lds + a_frag0 + i * 8192);
        QF::template frag<0>(raw[0], dec[0], bf[0][0]);
        QF::template frag<0>(raw[1], dec[1], bf[0][1]);
        __builtin_amdgcn_sched_barrier(0);   // prologue stays ahead of the pipelined steps
        mma_pipe<0, QF, NI>(raw, dec, lds, a_frag0, acc, af, bf);
    } else {
        mma_step<0, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<1, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<2, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<3, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<4, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<5, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<6, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
        mma_step<7, QF, PARTIAL, NI>(raw, dec, lds, a_frag0, acc, mi);
    }
}

// vmcnt(N) with every other counter left alone
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// Producers with a `Win` keep part of their per-block constants outside Raw (prepare takes the window as well).
template <class QF, class = void>
struct GemmWin {
    struct type {};
    static constexpr bool on = false;
};
template <class QF>
struct GemmWin<QF, std::void_t<typename QF::Win>> {
    using type = typename QF::Win;
    static constexpr bool on = true;
};
template <class QF>
__device__ __forceinline__ typename QF::Dec gemm_prepare(const typename QF::Raw& r, const typename GemmWin<QF>::type& wn, uint32_t kc, uint32_t h) {
    if constexpr (GemmWin<QF>::on) return QF::prepare(r, wn, kc, h);
    else return QF::prepare(r, kc, h);
}
// the producer a format uses for expert-grouped tiles when the scale table of the tile fits in LDS (itself if it names none)
template <class QF, class = void>
struct GemmLdsScales {
    using type = QF;
    static constexpr bool on = false;
};
template <class QF>
struct GemmLdsScales<QF, std::void_t<typename QF::LdsScales>> {
    using type = typename QF::LdsScales;
    static constexpr bool on = true;
};
constexpr uint32_t kGemmLdsScaleBytes = 16u * 1024u;   // LDS beyond the A buffers of a full tile, for launches of such formats

template <class QF, int NA>
struct TileCtx {
    typename QF::W w0, w1;
    uint32_t wrow0, wrow1, h;
    const uint8_t* a_glb;
    uint32_t a_dst;
    const uint8_t* lds_raw;
    uint32_t frag0, n_chunks, mi;
    uint32_t c0;   // first chunk of this K slice (chunk numbers below are slice-local)
    uint32_t tail_chunk;   // row-relative number of the chunk whose upper 64 columns lie past K (0xFFFFFFFF: none)
    uint32_t row_step;     // (BM / 4) * wave, for the A column of a lane
};

// The A rows of chunk `c` (slice-local) into the LDS buffer at `dst`.  In a chunk that ends half way (K % 128 = 64) a lane
// whose column lies past K reads the column 8 below instead (the same row, inside K): the weights of those columns are
// zero, so any finite value will do, and nothing is read past the row.
template <class QF, int NA>
__device__ __forceinline__ void a_rows_to_lds(const TileCtx<QF, NA>& t, const uint32_t (&a_off)[2 * NA], uint32_t c, uint32_t dst) {
    const uint8_t* src = t.a_glb + (size_t)c * (kBK * 2u);
    if (QF::K_ALIGN == 64 && t.c0 + c == t.tail_chunk) {
        const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
        for (int j = 0; j < 2 * NA; ++j) {
            const uint32_t R = t.row_step + 4u * j + (lane >> 4), col = (lane & 15u) ^ (R & 15u);
            load_to_lds16(src, a_off[j] - ((col & 8u) << 4), dst + 1024u * j);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2 * NA; ++j) load_to_lds16(src, a_off[j], dst + 1024u * j);
    }
}

// Chunk c out of register set P; meanwhile (`more`) the A rows of chunk c+1 and the weights of chunk c+DEPTH are requested.
// TAIL = one of the last chunks of the K loop, where chunk c+DEPTH may lie past the end: then no weight loads are issued
// (loads nobody reads may be dropped by the compiler, and the wait below counts on them) and the A rows are waited for
// with vmcnt(0).
template <class QF, bool PIPE, bool PARTIAL, int NA, int DEPTH, int P, bool TAIL>
__device__ __forceinline__ void gemm_chunk(const TileCtx<QF, NA>& t, const uint32_t (&a_off)[2 * NA], typename QF::Raw (&raw)[DEPTH + 1][2],
                                           const typename GemmWin<QF>::type (&win)[2], float16_t (&acc)[NA][2], uint32_t c, bool more) {
    constexpr int NSET = DEPTH + 1, PN = (P + DEPTH) % NSET;
    constexpr uint32_t ABUF = 32u * NA * kBK * 2u;
    constexpr int W_LOADS_MIN = 2 * (int)((sizeof(typename QF::Raw) + 15) / 16);
    const bool w_next = !TAIL || c + DEPTH < t.n_chunks;   // the weights of chunk c+DEPTH exist
    if (more) {
        a_rows_to_lds<QF, NA>(t, a_off, c + 1, t.a_dst + ((c + 1) & 1u) * ABUF);
        if (w_next) {
            raw[PN][0] = QF::load(t.w0, t.wrow0, t.c0 + c + DEPTH, t.h);
            raw[PN][1] = QF::load(t.w1, t.wrow1, t.c0 + c + DEPTH, t.h);
        }
        __builtin_amdgcn_sched_barrier(0);   // the scheduler must not sink these loads towards their uses
    }
    typename QF::Dec dec[2];
    dec[0] = gemm_prepare<QF>(raw[P][0], win[0], t.c0 + c, t.h);
    dec[1] = gemm_prepare<QF>(raw[P][1], win[1], t.c0 + c, t.h);
    mma_chunk<QF, PIPE, PARTIAL, NA>(raw[P], dec, t.lds_raw, (c & 1u) * ABUF + t.frag0, acc, t.mi);
    if (more) {
        // A rows of chunk c+1 are in LDS.  DEPTH > 1: the weight loads issued behind them in this chunk stay in flight
        // (memory returns in order, so at most that many outstanding loads means the A rows have landed).
        if (DEPTH > 1 && w_next) wait_vmcnt<W_LOADS_MIN>();
        else wait_vmcnt<0>();
        // A barrier that waits for the LDS traffic only: __syncthreads() carries a fence that waits for every
        // outstanding load, the weight words requested for later chunks included.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
}

// One output tile: accumulators, A staging, the K loop and the epilogue.  NA = 32-token tiles this instance
// keeps accumulators for and stages (the tile's live rows fit in 32 NA rows); PIPE = the hand-pipelined chunk
// (needs NA = 4 and a full tile); DEPTH = how many K chunks ahead the weight words are requested.
//
// Software pipeline over K chunks: at the top of chunk c the A rows of chunk c+1 start their way into the
// other LDS buffer, then the weight words of chunk c+DEPTH into registers.  Memory returns in order, the A
// rows come from L2 while the weights come from HBM.  With DEPTH = 1 both have one chunk of MFMAs to arrive,
// which covers the latency when a chunk carries 64 MFMAs per wave; a tile with one or two live token tiles
// finishes a chunk in a fraction of the memory latency, so it keeps two chunks of weights in flight.  At the
// end of chunk c the A rows of chunk c+1 must be in LDS: they are older than the weight loads issued after
// them in the same iteration, of which there are at least 2 ceil(sizeof(Raw) / 16) (a load instruction
// brings at most 16 bytes per lane), so waiting until at most that many loads are outstanding is enough
// whatever the compiler made of QF::load.
// KW = 2: a workgroup of eight waves, waves 4 - 7 walking the second half of K over A buffers of their own (`lds_raw` is
// then this half's buffer pair, `lds_red` the start of the workgroup's LDS); their sums meet the first half's in LDS
// before the epilogue.  Both halves run the same number of chunks, so their barriers pair up.
template <class QF, int MODE, bool PIPE, int NA, int DEPTH, int KW = 1>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, const typename QF::W& w0, const typename QF::W& w1, const uint32_t (&wrow)[2],
                                          uint32_t row_lo, uint32_t row_hi, uint32_t n_base, uint8_t* lds_raw, uint32_t c0 = 0,
                                          uint32_t n_chunks_slice = 0, uint32_t ks = 0, uint32_t e = 0, uint8_t* lds_red = nullptr) {
    static_assert(DEPTH == 1 || DEPTH == 2, "prefetch depth");
    static_assert(KW == 1 || (KW == 2 && MODE == GEMM_DENSE && NA == 4), "K halves inside a workgroup: dense full tiles only");
    static_assert(!PIPE || NA == 1 || NA == 2 || NA == 4, "the pipelined chunk is written for one, two or four token tiles");
    constexpr bool GATE_UP = MODE == GEMM_MOE_GATE_UP_SILU || MODE == GEMM_MOE_GATE_UP_OAI;
    constexpr bool PARTIAL = MODE != GEMM_DENSE && !PIPE;
    constexpr uint32_t BM = 32u * NA;
    constexpr int NL = 2 * NA;   // 1 KB loads per wave per chunk
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 31u, h = lane >> 5;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)((tid >> 6) & 3u));
    const uint32_t n_all = (g.K + kBK - 1) / kBK;                             // a row that ends half way through its last chunk counts it
    const uint32_t n_chunks = n_chunks_slice ? n_chunks_slice : n_all;       // chunks of this K slice (all of K unless split)
    const uint32_t live_rows = (row_hi - row_lo) >= BM ? BM : row_hi - row_lo;
    const uint32_t mi = (live_rows + 31u) / 32u;

    // A staging: wave w brings rows (BM/4) w .. of the chunk, 4 rows (1 KB) per load; lane L fills LDS slot
    // (row 4j + L/16, column L%16) of that 1 KB with global column (L%16) ^ (row & 15).  Rows past the end of
    // the tile re-read its last row (never used).
    // Gather form (grouped gate/up): the rows are read where they lie in the unsorted [T, K] matrix, through the sorted
    // row -> source row index, so no gathered copy is written and read back (moe_gather_rows folded into the A load).
    const bool gather = MODE != GEMM_DENSE && g.a_row_index != nullptr;
    uint32_t a_off[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const uint32_t R = (BM / 4u) * wave + 4u * j + (lane >> 4);
        const uint32_t Rc = R < live_rows ? R : live_rows - 1u;
        const uint32_t src = gather ? (uint32_t)g.a_row_index[row_lo + Rc] : Rc;
        a_off[j] = src * (g.K * 2u) + (((lane & 15u) ^ (R & 15u)) << 4);
    }
    const uint8_t* a_glb = reinterpret_cast<const uint8_t*>(g.A + (gather ? (size_t)0 : (size_t)row_lo * g.K)) + (size_t)c0 * (kBK * 2u);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t*)lds_raw;
    const uint32_t a_dst = lds_base + wave * (BM / 4u) * 256u;   // this wave's quarter of the rows inside an A buffer
    // step-0 fragment address of this lane inside an A buffer
    const uint32_t frag0 = r * 256u + (((QF::H_COL * h) ^ (r & 15u)) << 4);

    float16_t acc[NA][2];
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Weight words of DEPTH + 1 chunks live in registers: chunk c sits in set c % (DEPTH + 1).  The loop is unrolled
    // over the sets so that no set is ever copied into another (a register copy of loaded data waits for the load).
    constexpr int NSET = DEPTH + 1;
    typename QF::Raw raw[NSET][2];
    const TileCtx<QF, NA> ctx{w0, w1, wrow[0], wrow[1], h, a_glb, a_dst, lds_raw, frag0, n_chunks, mi, c0,
                              (g.K % kBK) ? n_all - 1u : 0xFFFFFFFFu, (BM / 4u) * wave};
    a_rows_to_lds<QF, NA>(ctx, a_off, 0, a_dst);
    raw[0][0] = QF::load(w0, wrow[0], c0, h);
    raw[0][1] = QF::load(w1, wrow[1], c0, h);
    typename GemmWin<QF>::type win[2];
    if constexpr (GemmWin<QF>::on) {
        // The scale table behind the A buffers: thread t copies table row t = 64 wave' + 32 tile + r', the scales of the
        // weight row that lane r' of wave' multiplies in its column tile `tile`, 16 bytes at a time.
        constexpr uint32_t ABUF2 = 2u * 32u * NA * kBK * 2u;
        const uint32_t pitch = QF::table_pitch(g.K), row_bytes = g.K / 16u;
        const uint32_t tw = tid >> 6, tj = (tid >> 5) & 1u, tr = tid & 31u;
        const uint32_t nb0 = n_base - wave * (GATE_UP ? 32u : kWaveN) + tw * (GATE_UP ? 32u : kWaveN);
        uint32_t tn_row = GATE_UP ? nb0 + tr : nb0 + 32u * tj + tr;
        if (tn_row >= g.N) tn_row = g.N - 1;
        const uint8_t* src = QF::scales_of((GATE_UP && tj) ? w1 : w0, tn_row);
        uint32_t* dst = reinterpret_cast<uint32_t*>(lds_raw + ABUF2 + tid * pitch);
        for (uint32_t b = 0; b < row_bytes; b += 64u) {
            uint4 v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {   // K is a multiple of 128: rows are whole 8-byte pieces
                const uint32_t at = b + 16u * i;
                if (at + 16u <= row_bytes) {
                    v[i] = load_u4_a2(src + at);
                } else if (at < row_bytes) {
                    const uint2 u = load_u2_a2(src + at);
                    v[i] = make_uint4(u.x, u.y, 0u, 0u);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t at = b + 16u * i;
                if (at < row_bytes) {
                    dst[at / 4u] = v[i].x;
                    dst[at / 4u + 1u] = v[i].y;
                    if (at + 16u <= row_bytes) {
                        dst[at / 4u + 2u] = v[i].z;
                        dst[at / 4u + 3u] = v[i].w;
                    }
                }
            }
        }
        win[0].row = lds_base + ABUF2 + (wave * 64u + r) * pitch;
        win[1].row = lds_base + ABUF2 + (wave * 64u + 32u + r) * pitch;
    }
    wait_vmcnt<0>();
    __syncthreads();
#pragma unroll
    for (int d = 1; d < DEPTH; ++d) {
        const uint32_t cd = (uint32_t)d < n_chunks ? (uint32_t)d : n_chunks - 1;
        raw[d][0] = QF::load(w0, wrow[0], c0 + cd, h);
        raw[d][1] = QF::load(w1, wrow[1], c0 + cd, h);
    }

#define CHUNK(P, c, more, tail) gemm_chunk<QF, PIPE, PARTIAL, NA, DEPTH, P, tail>(ctx, a_off, raw, win, acc, c, more)
    if constexpr (DEPTH == 1) {
        // two sets, and the set just loaded is copied into set 0 at the end of a chunk, where it has to have arrived anyway
        for (uint32_t c = 0; c + 1 < n_chunks; ++c) {
            CHUNK(0, c, true, false);
            raw[0][0] = raw[1][0];
            raw[0][1] = raw[1][1];
        }
        CHUNK(0, n_chunks - 1, false, true);
    } else {
        // three sets in rotation; inside the loop every chunk has its chunk c+2 (c + 4 < n_chunks), the last one to four
        // chunks check for it
        uint32_t c = 0;
        for (; c + 4 < n_chunks; c += 3) {
            CHUNK(0, c, true, false);
            CHUNK(1, c + 1, true, false);
            CHUNK(2, c + 2, true, false);
        }
        const uint32_t left = n_chunks - c;   // 1..4
        CHUNK(0, c, left > 1, true);
        if (left > 1) CHUNK(1, c + 1, left > 2, true);
        if (left > 2) CHUNK(2, c + 2, left > 3, true);
        if (left > 3) CHUNK(0, c + 3, false, true);
    }

#undef CHUNK
    if constexpr (KW == 2) {
        // The second K half hands its sums over through LDS (32 KB per wave, the whole allocation for four waves: both
        // halves are done with their A buffers behind the first barrier) and leaves; the first half adds them to its own.
        typedef float f32x4_t __attribute__((ext_vector_type(4)));
        const bool second = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 8)) != 0u;
        f32x4_t* red = reinterpret_cast<f32x4_t*>(lds_red) + (size_t)wave * (NA * 2 * 4) * 64u + lane;
        __syncthreads();
        if (second) {
#pragma unroll
            for (int i = 0; i < NA; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int v4 = 0; v4 < 4; ++v4)
                        red[((i * 2 + j) * 4 + v4) * 64] = f32x4_t{acc[i][j][4 * v4], acc[i][j][4 * v4 + 1], acc[i][j][4 * v4 + 2], acc[i][j][4 * v4 + 3]};
        }
        __syncthreads();
        if (second) return;
#pragma unroll
        for (int i = 0; i < NA; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) {
                    const f32x4_t t = red[((i * 2 + j) * 4 + v4) * 64];
                    acc[i][j][4 * v4] += t.x;
                    acc[i][j][4 * v4 + 1] += t.y;
                    acc[i][j][4 * v4 + 2] += t.z;
                    acc[i][j][4 * v4 + 3] += t.w;
                }
    }
    // ---- epilogue.  MFMA C layout: lane holds column n = lane%32, rows 8*(v/4) + 4*(lane/32) + v%4.
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t row = row_lo + 32 * i + 8 * (v / 4) + 4 * h + (v % 4);
            if (row >= row_hi) continue;
            if (GATE_UP) {
                const uint32_t n = n_base + r;
                if (n >= g.N) continue;
                if (MODE == GEMM_MOE_GATE_UP_OAI) {
                    const float gg = (float)(half_t)(acc[i][0][v] + (g.bias0 ? g.bias0[(size_t)e * g.N + n] : 0.f));
                    const float uu = (float)(half_t)(acc[i][1][v] + (g.bias1 ? g.bias1[(size_t)e * g.N + n] : 0.f));
                    g.Y[(size_t)row * g.N + n] = (half_t)swiglu_oai_f(gg, uu, g.alpha, g.limit);
                } else {
                    g.Y[(size_t)row * g.N + n] = (half_t)silu_mul_f(acc[i][0][v], acc[i][1][v]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t n = n_base + 32 * j + r;
                    if (n >= g.N) continue;
                    float o = acc[i][j][v];
                    if (MODE == GEMM_MOE_DOWN && g.route_w) o *= (float)g.route_w[row];
                    if (MODE == GEMM_MOE_DOWN && g.y_acc)
                        __hip_atomic_fetch_add(g.y_acc + (size_t)g.row_token[row] * g.N + n, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else if (MODE == GEMM_DENSE && g.k_split > 1)
                        g.split_acc[((size_t)ks * g.M + row) * g.N + n] = o;
                    else if (MODE == GEMM_MOE_DOWN && g.bias0)
                        g.Y[(size_t)row * g.N + n] = (half_t)((float)(half_t)o + g.bias0[(size_t)e * g.N + n]);
                    else
                        g.Y[(size_t)row * g.N + n] = (half_t)o;
                }
            }
        }
}

// Expert-grouped tile `tm` -> (expert, first row, end of the expert's rows), found by one wave.
// Tile order over all experts: every full BM-row tile first (expert by expert), then the experts' partial last tiles,
// those with the most live 32-row sub-tiles first.  A tile's cost grows with its live sub-tiles, so the workgroups
// dispatched last are the cheapest ones and the launch does not end with a few expensive tiles running alone (list
// scheduling, longest first).  The per-expert row counts are read 256 experts at a time, every load of a block issued
// before the first is used: with up to 256 experts the lookup costs one memory round trip (a loop that loads, scans
// and decides expert group by expert group and class by class pays one per step, several microseconds per tile).
// Returns false for a tile number past the last tile.
template <uint32_t BM, int NI>
__device__ __forceinline__ bool find_grouped_tile(const uint32_t* expert_offsets, uint32_t E, uint32_t tm, uint32_t ln, uint32_t (&out)[3]) {
    constexpr int JU = 4;   // expert groups of 64 per block
    struct Block {
        uint32_t lo[JU], hi[JU], full[JU], cls[JU];
    };
    auto load = [&](uint32_t e0, Block& b) {
#pragma unroll
        for (int j = 0; j < JU; ++j) {
            const uint32_t ee = e0 + 64u * j + ln;
            b.lo[j] = ee < E ? expert_offsets[ee] : 0u;
            b.hi[j] = ee < E ? expert_offsets[ee + 1] : 0u;
        }
#pragma unroll
        for (int j = 0; j < JU; ++j) {
            const uint32_t n = b.hi[j] - b.lo[j], rem = n % BM;
            b.full[j] = n / BM;
            b.cls[j] = (rem + 31u) / 32u;   // live sub-tiles of the partial tile, 0: none
        }
    };
    auto wave_sum = [&](uint32_t v) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) v += (uint32_t)__shfl_xor((int)v, d);
        return v;
    };
    uint32_t tot_full = 0, n_cls[NI + 1] = {};
    auto count = [&](const Block& b) {
#pragma unroll
        for (int j = 0; j < JU; ++j) {
            tot_full += wave_sum(b.full[j]);
#pragma unroll
            for (int k = 1; k <= NI; ++k) n_cls[k] += (uint32_t)__popcll(__ballot(b.cls[j] == (uint32_t)k));
        }
    };
    // locate state: the segment (full tiles, or class k) and the index inside it
    uint32_t seg = 0, idx = tm, seen = 0;
    bool found = false;
    auto locate = [&](uint32_t e0, const Block& b) {
#pragma unroll
        for (int j = 0; j < JU; ++j) {
            if (found) break;
            const uint32_t ee = e0 + 64u * j + ln;
            bool hit;
            uint32_t first;
            if (seg == 0) {
                uint32_t incl = b.full[j];
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) {
                    const uint32_t v = (uint32_t)__shfl_up((int)incl, d);
                    if (ln >= (uint32_t)d) incl += v;
                }
                const uint32_t excl = seen + incl - b.full[j];
                hit = idx >= excl && idx < excl + b.full[j];
                first = b.lo[j] + (idx - excl) * BM;
                seen += (uint32_t)__shfl((int)incl, 63);
            } else {
                const unsigned long long m = __ballot(b.cls[j] == seg);
                const uint32_t rank = (uint32_t)__popcll(m & ((1ull << ln) - 1ull));
                hit = ((m >> ln) & 1ull) && seen + rank == idx;
                first = b.lo[j] + b.full[j] * BM;
                seen += (uint32_t)__popcll(m);
            }
            if (hit) {
                out[0] = ee;
                out[1] = first;
                out[2] = b.hi[j];
            }
            found = __ballot(hit) != 0ull;
        }
    };
    auto pick_segment = [&]() {   // false: tm lies past the last tile
        if (idx < tot_full) return true;
        idx -= tot_full;
#pragma unroll
        for (int k = NI; k >= 1; --k) {
            if (idx < n_cls[k]) {
                seg = (uint32_t)k;
                return true;
            }
            idx -= n_cls[k];
        }
        return false;
    };
    Block b;
    if (E <= 64u * JU) {
        load(0, b);
        count(b);
        if (!pick_segment()) return false;
        locate(0, b);
    } else {
        for (uint32_t e0 = 0; e0 < E; e0 += 64u * JU) {
            load(e0, b);
            count(b);
        }
        if (!pick_segment()) return false;
        for (uint32_t e0 = 0; e0 < E && !found; e0 += 64u * JU) {
            load(e0, b);
            locate(e0, b);
        }
    }
    return found;
}

// NI = 32-token tiles per workgroup tile: 4 (128 tokens, two workgroups per CU), or 2 (64 tokens,
// three per CU) for dense launches whose 128-token tiles would leave CUs without work.
template <class QF, int MODE, int NI, int KW = 1>
__global__ __launch_bounds__(kGemmThreads * KW, KW == 2 ? 1 : NI == 2 ? 3 : 2) void gemm_kernel(typename QF::Bank bank0, typename QF::Bank bank1, GemmArgs g) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    constexpr uint32_t BM = 32u * NI;   // tokens per tile
    constexpr bool GATE_UP = MODE == GEMM_MOE_GATE_UP_SILU || MODE == GEMM_MOE_GATE_UP_OAI;
    constexpr uint32_t BN = GATE_UP ? 4 * 32 : 4 * kWaveN;   // output columns per workgroup

    // ---- which tile: XCD-aware order (workgroup i runs on XCD i % 8; each XCD walks a
    // contiguous range of tiles, 4 token tiles x consecutive column tiles at a time)
    // Expert-grouped tiles are uneven (dead tiles past the real count, 1-4 live token sub-tiles),
    // so they are dealt round-robin over the XCDs instead of in contiguous ranges.
    const uint32_t ksplit = (MODE == GEMM_DENSE) ? g.k_split : 1u;   // workgroups per output tile (K slices)
    const uint32_t total = g.tiles_m * g.tiles_n * ksplit;
    const uint32_t per_xcd = (total + 7) / 8;
    const uint32_t lin_ks = (MODE == GEMM_DENSE) ? (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    if ((MODE == GEMM_DENSE && (blockIdx.x >> 3) >= per_xcd) || lin_ks >= total) return;
    const uint32_t linear = lin_ks / ksplit, ks = lin_ks - linear * ksplit;
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
        // wave 0 finds the tile (find_grouped_tile) and leaves it at the head of the dynamic LDS, free until the tile starts
        uint32_t* s_tile = reinterpret_cast<uint32_t*>(lds_raw);
        if (threadIdx.x < 64) {
            uint32_t ent[3] = {0xFFFFFFFFu, 0u, 0u};
            const bool ok = find_grouped_tile<BM, NI>(g.expert_offsets, g.E, tm, threadIdx.x & 63u, ent);
            // the hit lane holds the entry; every other lane holds the "no tile" default
            const unsigned long long m = __ballot(ok && ent[0] != 0xFFFFFFFFu);
            if (m == 0ull) {
                if (threadIdx.x == 0) s_tile[0] = 0xFFFFFFFFu;
            } else if (ent[0] != 0xFFFFFFFFu) {
                s_tile[0] = ent[0];
                s_tile[1] = ent[1];
                s_tile[2] = ent[2];
            }
        }
        __syncthreads();
        e = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile[0]);
        if (e == 0xFFFFFFFFu) return;
        row_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile[1]);
        row_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile[2]);
        __syncthreads();   // every wave has read the entry before the first A rows land on it
    } else {
        row_lo = tm * BM;
    }
    const typename QF::W w0 = QF::expert(bank0, e), w1 = QF::expert(GATE_UP ? bank1 : bank0, e);

    const uint32_t tid = threadIdx.x, r = tid & 31u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)((tid >> 6) & 3u));
    const uint32_t n_base = tn * BN + wave * (GATE_UP ? 32 : kWaveN);
    // weight rows of the two MFMA column tiles of this wave (gate/up: same row in two matrices)
    uint32_t wrow[2];
    wrow[0] = n_base + r;
    wrow[1] = GATE_UP ? n_base + r : n_base + 32 + r;
    if (wrow[0] >= g.N) wrow[0] = g.N - 1;
    if (wrow[1] >= g.N) wrow[1] = g.N - 1;

    if constexpr (MODE == GEMM_DENSE) {
        const uint32_t n_all = (g.K + kBK - 1) / kBK, per = (n_all + ksplit - 1) / ksplit;
        const uint32_t c0 = ks * per, c1 = (c0 + per < n_all) ? c0 + per : n_all;
        if constexpr (KW == 2) {
            // the launcher takes this form for an even number of chunks and no K slices across workgroups
            const uint32_t kw = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 8)), half = n_all / 2u;
            gemm_tile<QF, MODE, true, 4, 1, 2>(g, w0, w1, wrow, row_lo, row_hi, n_base, lds_raw + kw * (2u * BM * kBK * 2u), kw * half, half, 0, 0, lds_raw);
        } else {
            gemm_tile<QF, MODE, NI == 4, NI, 1>(g, w0, w1, wrow, row_lo, row_hi, n_base, lds_raw, c0, c1 - c0, ks);
        }
    } else {
        (void)ks;
        // expert-grouped tiles: the pipelined chunk over as many 32-token tiles as the tile's live rows need (one, two,
        // or four; the token tiles past the live rows are multiplied too, on copies of the last live row, and dropped
        // by the epilogue).  A tile with at most 64 live rows keeps half (a quarter) of the accumulators and spends
        // the registers on a second chunk of weights in flight.
        const uint32_t live = row_hi - row_lo;
        using QL = typename GemmLdsScales<QF>::type;
        bool table4 = false, table2 = false, table1 = false;   // the scale table fits behind the A buffers of 4 / 2 / 1 token tiles
        if constexpr (GemmLdsScales<QF>::on) {
            const uint32_t need = 256u * QL::table_pitch(g.K), room = 2u * 128u * kBK * 2u + kGemmLdsScaleBytes;
            table4 = need <= room - 2u * 128u * kBK * 2u;
            table2 = need <= room - 2u * 64u * kBK * 2u;
            table1 = need <= room - 2u * 32u * kBK * 2u;
        }
#define MX_TILE(Q, na, depth) gemm_tile<Q, MODE, true, na, depth>(g, w0, w1, wrow, row_lo, row_hi, n_base, lds_raw, 0, 0, 0, e)
        if (live > 64u) {
            if (table4) MX_TILE(QL, 4, 1);
            else MX_TILE(QF, 4, 1);
        } else if (live > 32u) {
            if (table2) MX_TILE(QL, 2, 2);
            else MX_TILE(QF, 2, 2);
        } else {
            if (table1) MX_TILE(QL, 1, 2);
            else MX_TILE(QF, 1, 2);
        }
#undef MX_TILE
    }
}

// ---------------------------------------------------------------- host side
template <class QF, int MODE, int NI, int KW = 1>
static int launch_gemm_ni(mx_stream_t s, const typename QF::Bank& b0, const typename QF::Bank& b1, GemmArgs g, uint32_t rows_bound) {
    constexpr uint32_t BN = (MODE == GEMM_MOE_GATE_UP_SILU || MODE == GEMM_MOE_GATE_UP_OAI) ? 128 : 256, BM = 32u * NI;
    constexpr uint32_t lds = KW * 2u * BM * kBK * 2u + ((MODE != GEMM_DENSE && GemmLdsScales<QF>::on) ? kGemmLdsScaleBytes : 0u);
    g.tiles_n = (g.N + BN - 1) / BN;
    g.tiles_m = (MODE == GEMM_DENSE) ? (g.M + BM - 1) / BM : rows_bound / BM + g.E;   // grouped: an upper bound, workgroups past the real count leave at once
    if (MODE != GEMM_DENSE || g.k_split == 0) g.k_split = 1;
    const uint64_t total = (uint64_t)g.tiles_m * g.tiles_n * g.k_split;
    const uint64_t grid = (total + 7) / 8 * 8;
    if (grid > 0x7FFFFFFFull) return MX_ERR_SHAPE;
    static bool attr_set = false;   // LDS at the 64 KB default limit: opt in once per kernel
    if (!attr_set) {
        const hipError_t er = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<QF, MODE, NI, KW>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (er != hipSuccess) {
            g_last_hip_error = (int)er;
            return MX_ERR_LAUNCH;
        }
        attr_set = true;
    }
    hipLaunchKernelGGL((gemm_kernel<QF, MODE, NI, KW>), dim3((uint32_t)grid), dim3(kGemmThreads * KW), lds, as_stream(s), b0, b1, g);
    return launch_status();
}

static int gemm_cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    }
    return n;
}

// Dense launches whose 128-token tiles cover at most half of the CUs take 64-token tiles instead
// (twice the workgroups; measured: 64 tiles -> +20 %, 224 tiles -> -9 %); everything else runs
// 128-token tiles.
template <class QF, int MODE>
static int launch_gemm(mx_stream_t s, const typename QF::Bank& b0, const typename QF::Bank& b1, GemmArgs g, uint32_t rows_bound,
                       const SplitWs* caller_ws = nullptr) {
    if constexpr (MODE == GEMM_DENSE) {
        const uint64_t cus = (uint64_t)gemm_cu_count();
        const uint64_t tiles128 = (uint64_t)((g.M + 127) / 128) * ((g.N + 255) / 256);
        const uint64_t tiles64 = (uint64_t)((g.M + 63) / 64) * ((g.N + 255) / 256);
        const uint64_t mn = (uint64_t)g.M * g.N, n_chunks = (g.K + kBK - 1) / kBK;
        const uint64_t cap = caller_ws ? caller_ws->elems : kGemmSplitElems;   // partial sums the scratch holds
        // K slices a tiling could take: until every CU has a workgroup, each slice at least 8 chunks deep, the partial
        // sums within the scratch
        auto slices = [&](uint64_t tiles) {
            uint64_t k = tiles ? cus / tiles : 1;
            if (k > kGemmSplitMax) k = kGemmSplitMax;
            if (k > n_chunks / 8) k = n_chunks / 8;
            if (k * mn > cap) k = cap / mn;
            return k < 1 ? (uint64_t)1 : k;
        };
        bool ni2 = false;
        uint64_t k_split = 1;
        if (2 * tiles128 <= cus) {
            // 128-token tiles would leave half the CUs idle.  They stay (they do twice the matrix work per dequantized
            // weight) when K slices alone fill three quarters of the chip; otherwise 64-token tiles, sliced as well.
            // Measured at K = 14336, N = 4096: T = 128 94 -> 39 us, T = 512 162 -> 111 us.
            const uint64_t k4 = slices(tiles128);
            if (4 * tiles128 * k4 >= 3 * cus || g.M <= 64) {
                k_split = k4;
            } else {
                ni2 = true;
                k_split = slices(tiles64);
            }
        }
        if (2 * tiles128 > cus && tiles128 <= cus && n_chunks % 2 == 0 && n_chunks >= 16) {
            // One workgroup per CU would leave every SIMD with a single wave: eight-wave workgroups instead, each half of
            // the waves walking half of K (no scratch, no second launch).  T = 512, K = 4096, N = 14336: 224 tiles.
            return launch_gemm_ni<QF, MODE, 4, 2>(s, b0, b1, g, rows_bound);
        }
        if (k_split >= 2) {
            const uint32_t per = (uint32_t)((n_chunks + k_split - 1) / k_split);
            g.k_split = (uint32_t)((n_chunks + per - 1) / per);   // no empty slice
            if (caller_ws) {
                g.split_acc = caller_ws->ptr;
            } else {
                void* p = nullptr;
                if (int rc = scratch_address(HIP_SYMBOL(g_gemm_splitk_acc), g_gemm_splitk_addr, &p)) return rc;
                g.split_acc = static_cast<float*>(p);
            }
            const int rc = ni2 ? launch_gemm_ni<QF, MODE, 2>(s, b0, b1, g, rows_bound) : launch_gemm_ni<QF, MODE, 4>(s, b0, b1, g, rows_bound);
            if (rc != MX_OK) return rc;
            hipLaunchKernelGGL(gemm_splitk_store_kernel, dim3((uint32_t)((mn + 255) / 256)), dim3(256), 0, as_stream(s), g.Y, g.split_acc, (uint32_t)mn, g.k_split);
            return launch_status();
        }
        if (ni2) return launch_gemm_ni<QF, MODE, 2>(s, b0, b1, g, rows_bound);
    }
    return launch_gemm_ni<QF, MODE, 4>(s, b0, b1, g, rows_bound);
}

static int check_gemm(const void* A, const void* W, const void* y, uint32_t M, uint32_t K, uint32_t N, uint32_t k_align, uint32_t w_align = 16) {
    MX_REQUIRE_PTR(A);
    MX_REQUIRE_PTR(W);
    MX_REQUIRE_PTR(y);
    MX_REQUIRE_SHAPE(M > 0 && N > 0 && K > 0 && K % k_align == 0 && K <= (1u << 22));   // a 128-row A tile is addressed with 32-bit byte offsets
    MX_REQUIRE_ALIGN(A, 16);
    MX_REQUIRE_ALIGN(W, w_align);
    return MX_OK;
}

// AoS expert bank entry points (Q4_K, Q6_K): shared argument checks and GemmArgs
template <class QF, int MODE>
static int moe_gemm_aos(mx_stream_t s, const uint16_t* rows, const void* W0, const void* W1, uint64_t expert_stride_bytes, const uint32_t* expert_offsets,
                        const uint16_t* sorted_w, uint16_t* out, uint32_t E, uint32_t K, uint32_t N, uint32_t total_rows, uint32_t block_bytes,
                        uint32_t w_align, const int32_t* row_token = nullptr, float* y_acc = nullptr, const int32_t* a_row_index = nullptr) {
    if (int rc = check_gemm(rows, W0, y_acc ? static_cast<const void*>(y_acc) : out, total_rows, K, N, 256, w_align)) return rc;
    MX_REQUIRE_PTR(W1); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && expert_stride_bytes % w_align == 0);
    MX_REQUIRE_ALIGN(W1, w_align);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(rows); g.Y = reinterpret_cast<half_t*>(out); g.expert_offsets = expert_offsets;
    g.route_w = reinterpret_cast<const half_t*>(sorted_w); g.M = total_rows; g.K = K; g.N = N; g.E = E;
    g.row_token = row_token; g.y_acc = y_acc; g.a_row_index = a_row_index;
    if constexpr (std::is_same<QF, GemmQ4KStr>::value || std::is_same<QF, GemmQ6KStr>::value) {
        const uint64_t nb = (uint64_t)N * (K / 256);
        typename QF::Bank b0{static_cast<const uint8_t*>(W0), expert_stride_bytes, nb, K / 256}, b1{static_cast<const uint8_t*>(W1), expert_stride_bytes, nb, K / 256};
        return launch_gemm<QF, MODE>(s, b0, b1, g, total_rows);
    } else {
        const uint32_t row_bytes = K / 256 * block_bytes;
        typename QF::Bank b0{static_cast<const uint8_t*>(W0), expert_stride_bytes, row_bytes}, b1{static_cast<const uint8_t*>(W1), expert_stride_bytes, row_bytes};
        return launch_gemm<QF, MODE>(s, b0, b1, g, total_rows);
    }
}

// Dense entry points.  ws = NULL: K-sliced launches keep their partial sums in the library's per-device scratch.
template <class QF>
static int gemm_dense_aos(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, uint32_t k_align,
                          uint32_t w_align, uint32_t row_bytes, const SplitWs* ws) {
    if (int rc = check_gemm(A, W, y, M, K, N, k_align, w_align)) return rc;
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(A); g.Y = reinterpret_cast<half_t*>(y); g.M = M; g.K = K; g.N = N; g.E = 1;
    typename QF::Bank b{static_cast<const uint8_t*>(W), 0, row_bytes};
    return launch_gemm<QF, GEMM_DENSE>(s, b, b, g, M, ws);
}
static int gemm_dense_q8_soa(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M, uint32_t K,
                             uint32_t N, const SplitWs* ws) {
    if (int rc = check_gemm(A, qs_W, y, M, K, N, 128)) return rc;
    MX_REQUIRE_PTR(d_W);
    MX_REQUIRE_ALIGN(d_W, 4);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(A); g.Y = reinterpret_cast<half_t*>(y); g.M = M; g.K = K; g.N = N; g.E = 1;
    GemmQ8Soa::Bank b{qs_W, d_W, 0, 0, K};
    return launch_gemm<GemmQ8Soa, GEMM_DENSE>(s, b, b, g, M, ws);
}
// A caller's workspace: any size is accepted, the number of K slices adapts to what it holds (none below 2 M N floats).
static int gemm_ws(void* ws, uint64_t ws_bytes, SplitWs* out) {
    if (ws_bytes) {
        MX_REQUIRE_PTR(ws);
        MX_REQUIRE_ALIGN(ws, 16);
    }
    *out = SplitWs{static_cast<float*>(ws), ws_bytes / 4, true};
    return MX_OK;
}

}  // namespace mxq

using namespace mxq;

extern "C" {

int mx_gemm_q4_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_aos<GemmQ4K>(s, A, W, y, M, K, N, 256, 16, K / 256 * (uint32_t)kQ4KBytes, nullptr);
}
int mx_gemm_q6_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_aos<GemmQ6K>(s, A, W, y, M, K, N, 256, 2, K / 256 * (uint32_t)kQ6KBytes, nullptr);
}
int mx_gemm_q8_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_aos<GemmQ8Aos>(s, A, W, y, M, K, N, 128, 2, K / 32 * (uint32_t)kQ8_0Bytes, nullptr);
}
int mx_gemm_q4_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_aos<GemmQ40>(s, A, W, y, M, K, N, 128, 2, K / 32 * 18u, nullptr);
}
int mx_gemm_q8_0_soa(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_q8_soa(s, A, qs_W, d_W, y, M, K, N, nullptr);
}

// ---- caller-workspace forms: K-sliced launches keep their partial sums in `ws`, so calls on different streams can overlap
int mx_gemm_ws_bytes(uint32_t M, uint32_t K, uint32_t N, uint64_t* bytes) {
    MX_REQUIRE_PTR(bytes);
    MX_REQUIRE_SHAPE(M > 0 && K > 0 && N > 0);
    // K is sliced only when the 128-token tiles cover at most half of the CUs; then up to kGemmSplitMax planes of M x N floats
    const uint64_t tiles128 = (uint64_t)((M + 127) / 128) * ((N + 255) / 256);
    *bytes = (2 * tiles128 <= (uint64_t)gemm_cu_count() && K / kBK >= 16) ? (uint64_t)kGemmSplitMax * M * N * sizeof(float) : 0;
    return MX_OK;
}
int mx_gemm_q4_K_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws, uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = gemm_ws(ws, ws_bytes, &w)) return rc;
    return gemm_dense_aos<GemmQ4K>(s, A, W, y, M, K, N, 256, 16, K / 256 * (uint32_t)kQ4KBytes, &w);
}
int mx_gemm_q6_K_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws, uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = gemm_ws(ws, ws_bytes, &w)) return rc;
    return gemm_dense_aos<GemmQ6K>(s, A, W, y, M, K, N, 256, 2, K / 256 * (uint32_t)kQ6KBytes, &w);
}
int mx_gemm_q8_0_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws, uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = gemm_ws(ws, ws_bytes, &w)) return rc;
    return gemm_dense_aos<GemmQ8Aos>(s, A, W, y, M, K, N, 128, 2, K / 32 * (uint32_t)kQ8_0Bytes, &w);
}
int mx_gemm_q8_0_soa_ws(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N,
                        void* ws, uint64_t ws_bytes) {
    SplitWs w;
    if (int rc = gemm_ws(ws, ws_bytes, &w)) return rc;
    return gemm_dense_q8_soa(s, A, qs_W, d_W, y, M, K, N, &w);
}

// gather form: x = the unsorted rows [n_tokens, H], sorted_idx[r] = source row of sorted row r (NULL: x is already sorted)
static int check_gather(const int32_t* sorted_idx, uint32_t n_tokens, uint32_t H) {
    if (!sorted_idx) return MX_OK;
    MX_REQUIRE_ALIGN(sorted_idx, 4);
    MX_REQUIRE_SHAPE(n_tokens > 0 && (uint64_t)n_tokens * H * 2u < (1ull << 32));   // the A loads address rows with 32-bit byte offsets
    return MX_OK;
}
static int moe_gemm_gate_up_silu_q8(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens, const int8_t* g_qs, const uint16_t* g_d,
                                    const int8_t* u_qs, const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets,
                                    uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    if (int rc = check_gemm(x, g_qs, h_packed, total_rows, H, E_ffn, 128)) return rc;
    if (int rc = check_gather(sorted_idx, n_tokens, H)) return rc;
    MX_REQUIRE_PTR(g_d); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_d); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && qs_stride % 16 == 0 && d_stride % 2 == 0);
    MX_REQUIRE_ALIGN(u_qs, 16); MX_REQUIRE_ALIGN(g_d, 4); MX_REQUIRE_ALIGN(u_d, 4);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(x); g.Y = reinterpret_cast<half_t*>(h_packed); g.expert_offsets = expert_offsets;
    g.a_row_index = sorted_idx;
    g.M = total_rows; g.K = H; g.N = E_ffn; g.E = E;
    GemmQ8Soa::Bank bg{g_qs, g_d, qs_stride, d_stride, H}, bu{u_qs, u_d, qs_stride, d_stride, H};
    return launch_gemm<GemmQ8Soa, GEMM_MOE_GATE_UP_SILU>(s, bg, bu, g, total_rows);
}
int mx_moe_gemm_gate_up_silu_q8(mx_stream_t s, const uint16_t* x_packed, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                                const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets, uint16_t* h_packed,
                                uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    return moe_gemm_gate_up_silu_q8(s, x_packed, nullptr, 0, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, expert_offsets, h_packed, E, H, E_ffn, total_rows);
}
int mx_moe_gemm_gate_up_silu_q8_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens, const int8_t* g_qs,
                                       const uint16_t* g_d, const int8_t* u_qs, const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride,
                                       const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows) {
    MX_REQUIRE_PTR(sorted_idx);
    return moe_gemm_gate_up_silu_q8(s, x, sorted_idx, n_tokens, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, expert_offsets, h_packed, E, H, E_ffn, total_rows);
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

// soa != 0: every expert region holds its blocks as per-field streams (include/ie/quant_soa.hpp:33-51)
int mx_moe_gemm_gate_up_silu_q4k(mx_stream_t s, const uint16_t* x_packed, const void* gate_W, const void* up_W, const uint32_t* expert_offsets,
                                 uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    if (soa)
        return moe_gemm_aos<GemmQ4KStr, GEMM_MOE_GATE_UP_SILU>(s, x_packed, gate_W, up_W, expert_stride_bytes, expert_offsets, nullptr, h_packed, E, H, E_ffn,
                                                               total_rows, kQ4KBytes, 16);
    return moe_gemm_aos<GemmQ4K, GEMM_MOE_GATE_UP_SILU>(s, x_packed, gate_W, up_W, expert_stride_bytes, expert_offsets, nullptr, h_packed, E, H, E_ffn,
                                                        total_rows, kQ4KBytes, 16);
}

int mx_moe_gemm_gate_up_silu_q4k_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens, const void* gate_W, const void* up_W,
                                        const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                                        uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    MX_REQUIRE_PTR(sorted_idx);
    if (int rc = check_gather(sorted_idx, n_tokens, H)) return rc;
    if (soa)
        return moe_gemm_aos<GemmQ4KStr, GEMM_MOE_GATE_UP_SILU>(s, x, gate_W, up_W, expert_stride_bytes, expert_offsets, nullptr, h_packed, E, H, E_ffn,
                                                               total_rows, kQ4KBytes, 16, nullptr, nullptr, sorted_idx);
    return moe_gemm_aos<GemmQ4K, GEMM_MOE_GATE_UP_SILU>(s, x, gate_W, up_W, expert_stride_bytes, expert_offsets, nullptr, h_packed, E, H, E_ffn,
                                                        total_rows, kQ4KBytes, 16, nullptr, nullptr, sorted_idx);
}

int mx_moe_gemm_down_q4k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets, const uint16_t* sorted_w,
                         uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    if (soa)
        return moe_gemm_aos<GemmQ4KStr, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_w, out_packed, E, E_ffn, H,
                                                       total_rows, kQ4KBytes, 16);
    return moe_gemm_aos<GemmQ4K, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_w, out_packed, E, E_ffn, H,
                                                total_rows, kQ4KBytes, 16);
}

int mx_moe_gemm_down_q6k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets, const uint16_t* sorted_w,
                         uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows) {
    if (soa)
        return moe_gemm_aos<GemmQ6KStr, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_w, out_packed, E, E_ffn, H,
                                                       total_rows, kQ6KBytes, 2);
    return moe_gemm_aos<GemmQ6K, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_w, out_packed, E, E_ffn, H,
                                                total_rows, kQ6KBytes, 2);
}

// ---- MXFP4 planes and Q5_K blocks through the fused kernel (the reference dequantizes both to a [K, N] fp16 matrix and
// runs a plain GEMM: src/ops/gemv_mxfp4.cpp:316-341, src/model/gptoss.cpp:389-392, include/ie/dequant.hpp:81-86)
int mx_gemm_q5_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    return gemm_dense_aos<GemmQ5K>(s, A, W, y, M, K, N, 256, 16, K / 256 * 176u, nullptr);
}
int mx_gemm_mxfp4_soa(mx_stream_t s, const uint16_t* A, const uint8_t* qs_W, const uint8_t* e_W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N) {
    if (int rc = check_gemm(A, qs_W, y, M, K, N, 64)) return rc;
    MX_REQUIRE_PTR(e_W);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(A); g.Y = reinterpret_cast<half_t*>(y); g.M = M; g.K = K; g.N = N; g.E = 1;
    GemmMxfp4Soa::Bank b{qs_W, e_W, 0, 0, K};
    return launch_gemm<GemmMxfp4Soa, GEMM_DENSE>(s, b, b, g, M, nullptr);
}
static int moe_gemm_gate_up_oai_mxfp4(mx_stream_t s, const uint16_t* x_packed, const int32_t* sorted_idx, uint32_t n_tokens, const uint8_t* g_qs,
                                      const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride,
                                      const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E,
                                      uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha, float limit);
int mx_moe_gemm_gate_up_oai_mxfp4(mx_stream_t s, const uint16_t* x_packed, const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e,
                                  uint64_t qs_stride, uint64_t e_stride, const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets,
                                  uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha, float limit) {
    return moe_gemm_gate_up_oai_mxfp4(s, x_packed, nullptr, 0, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, expert_offsets, h_packed, E, H,
                                      E_ffn, total_rows, alpha, limit);
}
int mx_moe_gemm_gate_up_oai_mxfp4_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens, const uint8_t* g_qs,
                                         const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride,
                                         const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E,
                                         uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha, float limit) {
    MX_REQUIRE_PTR(sorted_idx);
    return moe_gemm_gate_up_oai_mxfp4(s, x, sorted_idx, n_tokens, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, expert_offsets, h_packed, E, H,
                                      E_ffn, total_rows, alpha, limit);
}
static int moe_gemm_gate_up_oai_mxfp4(mx_stream_t s, const uint16_t* x_packed, const int32_t* sorted_idx, uint32_t n_tokens, const uint8_t* g_qs,
                                      const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride,
                                      const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E,
                                      uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha, float limit) {
    if (int rc = check_gemm(x_packed, g_qs, h_packed, total_rows, H, E_ffn, 64)) return rc;
    if (int rc = check_gather(sorted_idx, n_tokens, H)) return rc;
    MX_REQUIRE_PTR(g_e); MX_REQUIRE_PTR(u_qs); MX_REQUIRE_PTR(u_e); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && qs_stride % 16 == 0);
    MX_REQUIRE_ALIGN(u_qs, 16);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(x_packed); g.Y = reinterpret_cast<half_t*>(h_packed); g.expert_offsets = expert_offsets;
    g.a_row_index = sorted_idx;
    g.M = total_rows; g.K = H; g.N = E_ffn; g.E = E; g.bias0 = gate_bias; g.bias1 = up_bias; g.alpha = alpha; g.limit = limit;
    GemmMxfp4Soa::Bank bg{g_qs, g_e, qs_stride, e_stride, H}, bu{u_qs, u_e, qs_stride, e_stride, H};
    return launch_gemm<GemmMxfp4Soa, GEMM_MOE_GATE_UP_OAI>(s, bg, bu, g, total_rows);
}
int mx_moe_gemm_down_mxfp4(mx_stream_t s, const uint16_t* h_packed, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride, uint64_t e_stride,
                           const float* down_bias, const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                           uint32_t total_rows) {
    if (int rc = check_gemm(h_packed, d_qs, out_packed, total_rows, E_ffn, H, 64)) return rc;
    MX_REQUIRE_PTR(d_e); MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && qs_stride % 16 == 0);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(h_packed); g.Y = reinterpret_cast<half_t*>(out_packed); g.expert_offsets = expert_offsets;
    g.M = total_rows; g.K = E_ffn; g.N = H; g.E = E; g.bias0 = down_bias;
    GemmMxfp4Soa::Bank b{d_qs, d_e, qs_stride, e_stride, E_ffn};
    return launch_gemm<GemmMxfp4Soa, GEMM_MOE_DOWN>(s, b, b, g, total_rows);
}

// moe_prefill_proj_q4_0_xmx (include/ie/ops.hpp:192-204): plain projection of expert-sorted fp16 rows through Q4_0 experts.
int mx_moe_prefill_proj_q4_0_xmx(mx_stream_t s, const uint16_t* x_fp16, const void* W_q4_0, const uint32_t* expert_offsets, uint16_t* out_packed,
                                 uint32_t E, uint32_t K, uint32_t N, uint64_t expert_stride_bytes, uint32_t total_rows) {
    if (int rc = check_gemm(x_fp16, W_q4_0, out_packed, total_rows, K, N, 128, 2)) return rc;
    MX_REQUIRE_PTR(expert_offsets);
    MX_REQUIRE_SHAPE(E > 0 && expert_stride_bytes % 2 == 0);
    GemmArgs g{};
    g.A = reinterpret_cast<const half_t*>(x_fp16); g.Y = reinterpret_cast<half_t*>(out_packed); g.expert_offsets = expert_offsets;
    g.M = total_rows; g.K = K; g.N = N; g.E = E;
    GemmQ40::Bank b{static_cast<const uint8_t*>(W_q4_0), expert_stride_bytes, K / 32 * 18u};
    return launch_gemm<GemmQ40, GEMM_MOE_DOWN>(s, b, b, g, total_rows);
}

// Accumulate form of the down projection (moe_prefill_down_q4k / _q6k, include/ie/ops.hpp:930-954):
// y_fp32[sorted_token_idx[row], n] += sorted_token_w[row] * (down_e . h_row)[n], fp32 atomics.
int mx_moe_prefill_down_q4k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets, const int32_t* sorted_token_idx,
                            const uint16_t* sorted_token_w, float* y_fp32, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes,
                            uint32_t total_rows) {
    MX_REQUIRE_PTR(sorted_token_idx); MX_REQUIRE_PTR(sorted_token_w); MX_REQUIRE_PTR(y_fp32);
    return moe_gemm_aos<GemmQ4K, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_token_w, nullptr, E, E_ffn, H,
                                                total_rows, kQ4KBytes, 16, sorted_token_idx, y_fp32);
}
int mx_moe_prefill_down_q6k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets, const int32_t* sorted_token_idx,
                            const uint16_t* sorted_token_w, float* y_fp32, uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes,
                            uint32_t total_rows) {
    MX_REQUIRE_PTR(sorted_token_idx); MX_REQUIRE_PTR(sorted_token_w); MX_REQUIRE_PTR(y_fp32);
    return moe_gemm_aos<GemmQ6K, GEMM_MOE_DOWN>(s, h_packed, down_W, down_W, expert_stride_bytes, expert_offsets, sorted_token_w, nullptr, E, E_ffn, H,
                                                total_rows, kQ6KBytes, 2, sorted_token_idx, y_fp32);
}

}  // extern "C"
