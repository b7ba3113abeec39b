// mxq_device.h — device-side helpers shared by every kernel: block layouts,
// bit casts, wave64 reductions, int8 dot, and the per-format weight-unit
// decoders.  gfx950 (CDNA4, wave64) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxq {

// On-disk GGUF block sizes (bytes) and elements per block.  The kernels address
// blocks by byte offset; nothing depends on struct padding.
// Layouts follow the reference's include/ie/quant_blocks.hpp:26-30 (Q8_0),
// :55-60 (MXFP4), :67-73 (Q4_K), :92-98 (Q6_K), :158-163 (q8_1x), :174-181 (q8_1s).
constexpr int kQ8_0Bytes = 34, kQ4KBytes = 144, kQ6KBytes = 210, kMxfp4Bytes = 17;
constexpr int kQ81xBytes = 40, kQ81sBytes = 48;

typedef _Float16 half_t;

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// E8M0 half-scaled exponent -> fp32 = 2^(e-128); e in {0,1} give fp32 denormals
// (include/ie/quant_blocks.hpp:46-54).
__device__ __forceinline__ float e8m0_half(uint32_t e) {
    return u2f(e < 2u ? (0x00200000u << e) : ((e - 1u) << 23));
}

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);  // v_dot4_i32_i8
}

// fp32 -> fp16, one RNE rounding of exactly this fp32 value.  Written as the
// bare conversion instruction so the compiler cannot fold a preceding multiply
// into v_fma_mixlo_f16 (a*b+0), which would turn -0.0 products into +0.0.
__device__ __forceinline__ half_t f32_to_f16_rne(float v) {
    uint32_t r;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(r) : "v"(v));
    return __builtin_bit_cast(half_t, (uint16_t)r);
}

template <class T>
__device__ __forceinline__ void store_out(T* p, float v);
template <>
__device__ __forceinline__ void store_out<half_t>(half_t* p, float v) { *p = (half_t)v; }
template <>
__device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float load_act(const half_t* p) { return (float)*p; }
__device__ __forceinline__ float load_act(const float* p) { return *p; }

// ---------------------------------------------------------------- wave64 reductions
// Sum over the G lanes of each aligned lane group (G = 8, 16, 32, 64).  DPP
// inside a 16-lane row (quad_perm, row_half_mirror, row_mirror), row broadcasts
// across rows.  After the call every lane of the group holds... only the LAST
// lane of each group is guaranteed to hold the group sum for G > 16; for
// G <= 16 every lane does.  Use group_sum_lane<G>() for the lane to read.
template <int CTRL, int ROW_MASK = 0xF, bool BOUND = true>
__device__ __forceinline__ float dpp_f(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), CTRL, ROW_MASK, 0xF, BOUND));
}
template <int G>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_f<0xB1>(v);                       // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);                       // quad_perm [2,3,0,1]
    if (G >= 8) v += dpp_f<0x141>(v);          // row_half_mirror: 8-lane sums
    if (G >= 16) v += dpp_f<0x140>(v);         // row_mirror: 16-lane sums (all lanes)
    if (G >= 32) v += dpp_f<0x142, 0xA, false>(v);  // row_bcast15 into rows 1,3
    if (G >= 64) v += dpp_f<0x143, 0xC, false>(v);  // row_bcast31 into rows 2,3
    return v;
}
// lane (within the wave) that holds group g's sum after group_sum<G>
template <int G>
__device__ __forceinline__ int group_sum_lane(int lane) {
    return (G <= 16) ? (lane & ~(G - 1)) : (lane | (G - 1));
}
__device__ __forceinline__ float group_max8(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    return v;
}
__device__ __forceinline__ int group_sum8_i(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
    return v;
}

// ---------------------------------------------------------------- block_q8_1x emission
// 8 lanes per 32-element block, 4 consecutive elements per lane (v), l8 = lane % 8.  All 8
// lanes of a group must call.  d = amax/127, inv = 127/amax (0 for a zero block),
// q = round-half-away(v*inv), s = d*float(sum q)  (src/ops/gemv_q8dot.cpp:94-124).
__device__ __forceinline__ void emit_q8_1x(const float (&v)[4], uint32_t l8, bool live, uint8_t* blk) {
    const float amax = group_max8(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    const float d = amax / 127.0f, inv = amax > 0.f ? 127.0f / amax : 0.f;
    int q[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = (int)roundf(v[i] * inv);
        sum += q[i];
    }
    const uint32_t packed = (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) | ((uint32_t)(q[2] & 0xFF) << 16) | ((uint32_t)(q[3] & 0xFF) << 24);
    const int tot = group_sum8_i(sum);
    if (!live) return;
    reinterpret_cast<uint32_t*>(blk + 8)[l8] = packed;
    if (l8 == 0) *reinterpret_cast<float2*>(blk) = make_float2(d, d * (float)tot);
}

// ---------------------------------------------------------------- scales
// The 8 six-bit (scale, min) pairs of a Q4_K block live in 12 bytes
// (include/ie/dequant_ref.hpp:20-29).  For the 64-element group g the two
// sub-blocks are j = 2g and 2g+1; both pairs come out of three 16-bit fields.
// Returns sc as (sc_j | sc_{j+1} << 8) and mn likewise.
__device__ __forceinline__ void q4k_scale_pair(uint32_t s0, uint32_t s1, uint32_t s2, int g, uint32_t& sc, uint32_t& mn) {
    const int sh = (g & 1) * 16;
    const uint32_t lo = (s0 >> sh) & 0xFFFFu, mid = (s1 >> sh) & 0xFFFFu, hi = (s2 >> sh) & 0xFFFFu;
    if (g < 2) {
        sc = lo & 0x3F3Fu;
        mn = mid & 0x3F3Fu;
    } else {
        sc = (hi & 0x0F0Fu) | ((lo >> 2) & 0x3030u);
        mn = ((hi >> 4) & 0x0F0Fu) | ((mid >> 2) & 0x3030u);
    }
}

// MXFP4 codes -> doubled E2M1 values as int8, four at a time.  `sel` holds the 3 magnitude bits of
// four codes (one per byte); `pick` byte i is i for a positive code and 4 + i for a negative one.
// LUT {0,1,2,3,4,6,8,12} / {0,-1,...,-12} by two byte permutes, then a third permute takes byte i from
// the positive or the negative result (include/ie/quant_blocks.hpp:46-54).
__device__ __forceinline__ uint32_t mxfp4_lut4(uint32_t sel, uint32_t pick) {
    const uint32_t pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
    const uint32_t neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
    return __builtin_amdgcn_perm(neg, pos, pick);
}
// One qs dword (bytes j..j+3 of a block) -> codes of elements j..j+3 (lo) and 16+j..16+j+3 (hi).
// The sign bit of a code (bit 3 / bit 7 of its byte) lands on bit 2 of the pick byte.
__device__ __forceinline__ void mxfp4_decode_word(uint32_t w, uint32_t& lo, uint32_t& hi) {
    lo = mxfp4_lut4(w & 0x07070707u, ((w >> 1) & 0x04040404u) | 0x03020100u);
    hi = mxfp4_lut4((w >> 4) & 0x07070707u, ((w >> 5) & 0x04040404u) | 0x03020100u);
}

}  // namespace mxq
