// host_repack.cpp — load-time host repackers (pure byte moves, host pointers).
#include <string.h>

#include "../../include/mxq.h"

extern "C" {

// block_mxfp4 {u8 e; u8 qs[16]} -> qs_plane[16*i + j], e_plane[i]
// (reference: src/model/gptoss.cpp:180-208).
int mx_repack_mxfp4_to_soa(const void* blocks, uint64_t n_blocks, uint8_t* qs_plane, uint8_t* e_plane) {
    if (!blocks || !qs_plane || !e_plane) return MX_ERR_NULL;
    const uint8_t* b = static_cast<const uint8_t*>(blocks);
    for (uint64_t i = 0; i < n_blocks; ++i, b += 17) {
        e_plane[i] = b[0];
        memcpy(qs_plane + 16 * i, b + 1, 16);
    }
    return MX_OK;
}

// block_q8_0 {fp16 d; i8 qs[32]} -> qs_plane[32*i + j], d_plane[i]
// (reference: src/model/qwen35moe_split.cpp:134-144).
int mx_repack_q8_0_to_soa(const void* blocks, uint64_t n_blocks, int8_t* qs_plane, uint16_t* d_plane) {
    if (!blocks || !qs_plane || !d_plane) return MX_ERR_NULL;
    const uint8_t* b = static_cast<const uint8_t*>(blocks);
    for (uint64_t i = 0; i < n_blocks; ++i, b += 34) {
        memcpy(d_plane + i, b, 2);
        memcpy(qs_plane + 32 * i, b + 2, 32);
    }
    return MX_OK;
}

// block_q4_0 {fp16 d; u8 qs[16]} -> qs_plane[16*i + j], d_plane[i]   (reference: src/ops/gemv_q4_0.cpp:179-192)
int mx_repack_q4_0_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q4_qs, uint16_t* q4_d) {
    if (!W_blocks || !q4_qs || !q4_d) return MX_ERR_NULL;
    if (K == 0 || K % 32) return MX_ERR_SHAPE;
    const uint8_t* b = static_cast<const uint8_t*>(W_blocks);
    const uint64_t nb = (uint64_t)N * (K / 32);
    for (uint64_t i = 0; i < nb; ++i, b += 18) {
        memcpy(q4_d + i, b, 2);
        memcpy(q4_qs + 16 * i, b + 2, 16);
    }
    return MX_OK;
}

// block_q4_K {fp16 d; fp16 dmin; u8 scales[12]; u8 qs[128]} x nb  ->  qs x nb | scales x nb | {d,dmin} x nb
// over all nb = N*K/256 blocks of a matrix (reference: src/ops/gemv_q8dot.cpp:134-147).
int mx_repack_q4_K_to_reorder(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* out) {
    if (!W_blocks || !out) return MX_ERR_NULL;
    if (K == 0 || K % 256) return MX_ERR_SHAPE;
    return mx_repack_moe_q4k_soa_host(W_blocks, out, 1, (uint64_t)N * (K / 256));
}

// The same split applied inside each expert region of an expert-major bank; region stride unchanged
// (reference: include/ie/quant_soa.hpp:127-141).
int mx_repack_moe_q4k_soa_host(const void* src, void* dst, uint32_t n_experts, uint64_t nblocks_per_expert) {
    if (!src || !dst) return MX_ERR_NULL;
    if (src == dst) return MX_ERR_SHAPE;
    const uint64_t nb = nblocks_per_expert;
    for (uint32_t e = 0; e < n_experts; ++e) {
        const uint8_t* b = static_cast<const uint8_t*>(src) + e * nb * 144;
        uint8_t* o = static_cast<uint8_t*>(dst) + e * nb * 144;
        for (uint64_t i = 0; i < nb; ++i, b += 144) {
            memcpy(o + i * 128, b + 16, 128);
            memcpy(o + nb * 128 + i * 12, b + 4, 12);
            memcpy(o + nb * 140 + i * 4, b, 4);
        }
    }
    return MX_OK;
}

// block_q6_K {u8 ql[128]; u8 qh[64]; i8 scales[16]; fp16 d} x nb  ->  ql x nb | qh x nb | scales x nb | d x nb
// per expert region (reference: include/ie/quant_soa.hpp:143-157).
int mx_repack_moe_q6k_soa_host(const void* src, void* dst, uint32_t n_experts, uint64_t nblocks_per_expert) {
    if (!src || !dst) return MX_ERR_NULL;
    if (src == dst) return MX_ERR_SHAPE;
    const uint64_t nb = nblocks_per_expert;
    for (uint32_t e = 0; e < n_experts; ++e) {
        const uint8_t* b = static_cast<const uint8_t*>(src) + e * nb * 210;
        uint8_t* o = static_cast<uint8_t*>(dst) + e * nb * 210;
        for (uint64_t i = 0; i < nb; ++i, b += 210) {
            memcpy(o + i * 128, b, 128);
            memcpy(o + nb * 128 + i * 64, b + 128, 64);
            memcpy(o + nb * 192 + i * 16, b + 192, 16);
            memcpy(o + nb * 208 + i * 2, b + 208, 2);
        }
    }
    return MX_OK;
}

// The 6-bit (scale, min) of sub-block j of a Q4_K block (reference: include/ie/dequant_ref.hpp:20-29).
static void q4k_scale_min(const uint8_t* sc, int j, uint8_t* s, uint8_t* m) {
    if (j < 4) {
        *s = sc[j] & 63;
        *m = sc[j + 4] & 63;
    } else {
        *s = (uint8_t)((sc[j + 4] & 15) | ((sc[j - 4] >> 6) << 4));
        *m = (uint8_t)((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4));
    }
}

// Q4_K rows -> natural element order: nibble of element k at q[k/2] bits 4*(k&1); unpacked per-32
// scale / min; per-256 d / dmin (reference: src/ops/gemv_q4_soa.cpp:115-151).  Element e of a block
// is qs[32*(e/64) + e%32], low nibble when (e%64) < 32 (include/ie/dequant_ref.hpp:38-53).
int mx_repack_q4_K_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q4_q, int8_t* q4_sc, int8_t* q4_mn, uint16_t* q4_d,
                          uint16_t* q4_dmin) {
    if (!W_blocks || !q4_q || !q4_sc || !q4_mn || !q4_d || !q4_dmin) return MX_ERR_NULL;
    if (K == 0 || K % 256) return MX_ERR_SHAPE;
    const uint64_t nb = (uint64_t)N * (K / 256);
    const uint8_t* b = static_cast<const uint8_t*>(W_blocks);
    for (uint64_t i = 0; i < nb; ++i, b += 144) {
        memcpy(q4_d + i, b, 2);
        memcpy(q4_dmin + i, b + 2, 2);
        for (int j = 0; j < 8; ++j) {
            uint8_t sv, mv;
            q4k_scale_min(b + 4, j, &sv, &mv);
            q4_sc[i * 8 + j] = (int8_t)sv;
            q4_mn[i * 8 + j] = (int8_t)mv;
        }
        const uint8_t* qs = b + 16;
        uint8_t* o = q4_q + i * 128;
        for (int e = 0; e < 256; e += 2) {
            uint8_t nib[2];
            for (int t = 0; t < 2; ++t) {
                const int el = e + t, byte = qs[32 * (el >> 6) + (el & 31)];
                nib[t] = (uint8_t)(((el & 63) < 32) ? (byte & 15) : (byte >> 4));
            }
            o[e >> 1] = (uint8_t)(nib[0] | (nib[1] << 4));
        }
    }
    return MX_OK;
}

// Q6_K rows -> natural element order bit planes: low nibble of element k at lo[k/2] bits 4*(k&1), high
// two bits at hi[k/4] bits 2*(k&3); per-16 int8 scales; per-256 d (reference: src/ops/gemv_q6_soa.cpp:
// 71-126).  Element e = 128h + 32s + l of a block has low nibble ql[64h + 32(s&1) + l] (high half when
// s >= 2) and high bits (qh[32h + l] >> 2s) & 3 (include/ie/dequant_ref.hpp:78-96).  Every output byte is
// written whole, so the planes need no clearing beforehand.
int mx_repack_q6_K_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q6_lo, uint8_t* q6_hi, int8_t* q6_sc, uint16_t* q6_d) {
    if (!W_blocks || !q6_lo || !q6_hi || !q6_sc || !q6_d) return MX_ERR_NULL;
    if (K == 0 || K % 256) return MX_ERR_SHAPE;
    const uint64_t nb = (uint64_t)N * (K / 256);
    const uint8_t* b = static_cast<const uint8_t*>(W_blocks);
    for (uint64_t i = 0; i < nb; ++i, b += 210) {
        memcpy(q6_d + i, b + 208, 2);
        memcpy(q6_sc + i * 16, b + 192, 16);
        uint8_t q6[256];
        for (int e = 0; e < 256; ++e) {
            const int h = e >> 7, sub = (e >> 5) & 3, l = e & 31;
            const int lb = b[64 * h + 32 * (sub & 1) + l];
            q6[e] = (uint8_t)(((sub & 2) ? lb >> 4 : lb & 15) | (((b[128 + 32 * h + l] >> (2 * sub)) & 3) << 4));
        }
        for (int e = 0; e < 256; e += 2) q6_lo[i * 128 + (e >> 1)] = (uint8_t)((q6[e] & 15) | ((q6[e + 1] & 15) << 4));
        for (int e = 0; e < 256; e += 4)
            q6_hi[i * 64 + (e >> 2)] = (uint8_t)((q6[e] >> 4) | ((q6[e + 1] >> 4) << 2) | ((q6[e + 2] >> 4) << 4) | ((q6[e + 3] >> 4) << 6));
    }
    return MX_OK;
}

}  // extern "C"
