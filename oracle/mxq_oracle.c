/*
 * mxq_oracle.c — CPU restatement of the Mach X quantized-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP kernels: it
 * is linked by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
 * of bench.py, and by nothing that ships.  The product library never calls it.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * the reference tree).  Parity status of each function (what pins it):
 *
 *   orc_fp16_to_fp32 / orc_fp32_to_fp16     pinned: exhaustive 2^16 sweep vs numpy
 *                                            float16 + vs oracle/_ref
 *   orc_get_scale_min_k4                     pinned: oracle/_ref + golden fixture
 *   orc_dequant (Q8_0, Q4_K, Q5_K, Q6_K)     pinned: oracle/_ref (ie::ref::dequant_*),
 *                                            golden fixtures, closed forms
 *   orc_dequant (MXFP4)                      pinned: closed forms (e=127 -> E2M1 table,
 *                                            e in {0,1} denormals, 2^(e-128)), the
 *                                            reference test's exponent list; no host
 *                                            header in the reference compiles it
 *   orc_dequant (Q4_0)                       pinned: closed forms (d = 1 -> y = nibble - 8, element j in the low
 *                                            and j+16 in the high nibble of qs[j]); the reference holds no host
 *                                            routine for it (device code src/ops/gemv_q4_0.cpp:3-8,455-477)
 *   orc_quantize_row_q4_0                    NOT IN REFERENCE (fixture generator only; ggml's published
 *                                            quantize_row_q4_0_ref recipe); pinned by round trip: error <= |d|/2
 *                                            except the clamped extreme
 *   orc_quantize_row_q4_K / _q6_K            pinned: oracle/_ref (bit-identical blocks),
 *                                            golden fixtures, reference error bounds
 *   orc_quantize_row_q8_0                    pinned: invariants + round trip
 *                                            (recipe tools/q8_0_repack_bench.cpp:62-74)
 *   orc_quantize_row_mxfp4                   NOT IN REFERENCE (fixture generator only);
 *                                            pinned by round trip through orc_dequant
 *   orc_quantize_q8_1 / _q8_1s               pinned: invariants (|q|<=127, s==d*sum,
 *                                            s0+s1==s, half-away rounding), brute force
 *   orc_gemv_* / orc_gemm_*                  pinned: brute-force int64 dots on tiny
 *                                            shapes, linearity, identity weights
 *   orc_gemv_q8schain                        pinned: equals orc_gemv_q8chain on rows whose stored sums are d * sum(q);
 *                                            closed forms with doctored sums (scale 0 / min 1 -> -(s0 + s1) per
 *                                            sub-block; Q6_K d = sc = 1, zero quants -> -32 * s_half per group)
 *   orc_route_from_logits                    pinned: textbook softmax/top-k brute force
 *   orc_build_moe_packing                    pinned: oracle/_ref (ie::build_moe_packing)
 *                                            + permutation invariants
 *   orc_repack_*                             pinned: view-equivalence / reconstruction
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fopenmp).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { ORC_Q8_0 = 0, ORC_Q4_K = 1, ORC_Q6_K = 2, ORC_MXFP4 = 3, ORC_Q5_K = 4 /* no encoder */, ORC_Q4_0 = 5 };

/* ---------------------------------------------------------------- layouts
 * include/ie/quant_blocks.hpp:26-30 (Q8_0), :55-60 (MXFP4), :67-73 (Q4_K),
 * :92-98 (Q6_K), :158-163 (q8_1x), :174-181 (q8_1s).  Byte offsets only; the
 * oracle never relies on struct padding. */
#define Q8_0_BYTES 34
#define Q4_K_BYTES 144
#define Q6_K_BYTES 210
#define Q5_K_BYTES 176
#define MXFP4_BYTES 17
#define Q4_0_BYTES 18
#define Q8_1X_BYTES 40
#define Q8_1S_BYTES 48

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ---------------------------------------------------------------- fp16
 * include/ie/quant_blocks.hpp:104-146.  Own formulation: subnormals are the
 * exact product mant * 2^-24; RNE is done on the 13 dropped bits. */
ORC_API float orc_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t ex = (h >> 10) & 31u, man = h & 1023u;
    if (ex == 31u) return u2f(sign | 0x7f800000u | (man << 13));
    if (ex == 0u) {
        const float v = (float)man * 5.9604644775390625e-8f; /* 2^-24, exact */
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((ex + 112u) << 23) | (man << 13));
}

ORC_API uint16_t orc_fp32_to_fp16(float f) {
    const uint32_t x = f2u(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0u));
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);       /* rounds to inf */
    if (ax < 0x33000001u) return sign;                             /* <= 2^-25: to zero (tie at 2^-25 -> even = 0) */
    int e = (int)(ax >> 23) - 127;                                 /* unbiased */
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;                     /* 24-bit significand */
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;                 /* bits to drop */
    uint32_t keep = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) keep++;
    if (e < -14) return (uint16_t)(sign | keep);                   /* subnormal (may carry into normal: correct) */
    /* keep includes the implicit bit at position 10; adding carries into exponent naturally */
    return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (keep - 0x400u)));
}

ORC_API void orc_fp16_to_fp32_n(const uint16_t* h, float* f, size_t n) {
    for (size_t i = 0; i < n; ++i) f[i] = orc_fp16_to_fp32(h[i]);
}
ORC_API void orc_fp32_to_fp16_n(const float* f, uint16_t* h, size_t n) {
    for (size_t i = 0; i < n; ++i) h[i] = orc_fp32_to_fp16(f[i]);
}
/* round an fp32 array through fp16 in place (value stays fp32) */
ORC_API void orc_round_fp16_n(float* f, size_t n) {
    for (size_t i = 0; i < n; ++i) f[i] = orc_fp16_to_fp32(orc_fp32_to_fp16(f[i]));
}

/* ---------------------------------------------------------------- RNG
 * Counter-based: value i of stream `seed` depends on (seed, i) only, so any
 * slice can be regenerated.  splitmix64 finaliser + Box-Muller in double. */
static inline uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline uint64_t rng_u64(uint64_t seed, uint64_t i) { return mix64(mix64(seed) ^ (i * 0xD1342543DE82EF95ull)); }
static inline double rng_unit(uint64_t seed, uint64_t i) { return ((double)(rng_u64(seed, i) >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

ORC_API void orc_rng_u64(uint64_t seed, uint64_t offset, size_t n, uint64_t* out) {
    for (size_t i = 0; i < n; ++i) out[i] = rng_u64(seed, offset + i);
}
ORC_API void orc_rng_bytes(uint64_t seed, uint64_t offset, size_t n, uint8_t* out) {
    for (size_t i = 0; i < n; ++i) out[i] = (uint8_t)(rng_u64(seed, offset + i) >> 32);
}
ORC_API void orc_rng_uniform(uint64_t seed, uint64_t offset, size_t n, float lo, float hi, float* out) {
    for (size_t i = 0; i < n; ++i) out[i] = (float)(lo + (hi - lo) * rng_unit(seed, offset + i));
}
ORC_API void orc_rng_normal(uint64_t seed, uint64_t offset, size_t n, float mean, float std, float* out) {
#pragma omp parallel for schedule(static) if (n > (1u << 16))
    for (size_t i = 0; i < n; ++i) {
        const uint64_t c = offset + i;
        const double u1 = rng_unit(seed, 2 * c), u2 = rng_unit(seed, 2 * c + 1);
        const double r = sqrt(-2.0 * log(u1));
        out[i] = (float)(mean + std * r * cos(6.283185307179586476925 * u2));
    }
}

/* ---------------------------------------------------------------- dequant
 * include/ie/dequant_ref.hpp:20-29 */
ORC_API void orc_get_scale_min_k4(int j, const uint8_t* q, uint8_t* sc, uint8_t* mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 15) | ((q[j - 4] >> 6) << 4));
        *mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* include/ie/dequant_ref.hpp:32-35 */
static void deq_q8_0(const uint8_t* b, float* y) {
    const float d = orc_fp16_to_fp32(rd16(b));
    const int8_t* qs = (const int8_t*)(b + 2);
    for (int i = 0; i < 32; ++i) y[i] = d * (float)qs[i];
}

/* include/ie/dequant_ref.hpp:38-53.  Element e = 64g + 32hi + l lives in byte
 * qs[32g + l], nibble hi; sub-block 2g+hi.  Operation order is the contract:
 * (d*sc)*q - (dmin*m), no FMA contraction (-ffp-contract=off). */
static void deq_q4_K(const uint8_t* b, float* y) {
    const float d = orc_fp16_to_fp32(rd16(b)), dmin = orc_fp16_to_fp32(rd16(b + 2));
    const uint8_t* scales = b + 4;
    const uint8_t* qs = b + 16;
    for (int e = 0; e < 256; ++e) {
        const int g = e >> 6, hi = (e >> 5) & 1, l = e & 31;
        uint8_t sc, mn;
        orc_get_scale_min_k4(2 * g + hi, scales, &sc, &mn);
        const float d1 = d * (float)sc, m1 = dmin * (float)mn;
        const uint8_t byte = qs[32 * g + l];
        const int q = hi ? (byte >> 4) : (byte & 15);
        y[e] = d1 * (float)q - m1;
    }
}

/* include/ie/dequant_ref.hpp:56-75, layout include/ie/quant_blocks.hpp:79-85 {d, dmin, scales[12],
 * qh[32], qs[128]}.  As Q4_K with a fifth bit: element e = 64g + 32hi + l takes bit (2g + hi) of
 * qh[l]; (d*sc)*q - (dmin*m) with q in 0..31. */
static void deq_q5_K(const uint8_t* b, float* y) {
    const float d = orc_fp16_to_fp32(rd16(b)), dmin = orc_fp16_to_fp32(rd16(b + 2));
    const uint8_t* scales = b + 4;
    const uint8_t* qh = b + 16;
    const uint8_t* qs = b + 48;
    for (int e = 0; e < 256; ++e) {
        const int g = e >> 6, hi = (e >> 5) & 1, l = e & 31;
        uint8_t sc, mn;
        orc_get_scale_min_k4(2 * g + hi, scales, &sc, &mn);
        const float d1 = d * (float)sc, m1 = dmin * (float)mn;
        const uint8_t byte = qs[32 * g + l];
        const int q = (hi ? (byte >> 4) : (byte & 15)) + (((qh[l] >> (2 * g + hi)) & 1) ? 16 : 0);
        y[e] = d1 * (float)q - m1;
    }
}

/* include/ie/dequant_ref.hpp:78-96.  Element e = 128h + 32sub + l. */
static void deq_q6_K(const uint8_t* b, float* y) {
    const uint8_t* ql = b;
    const uint8_t* qh = b + 128;
    const int8_t* sc = (const int8_t*)(b + 192);
    const float d = orc_fp16_to_fp32(rd16(b + 208));
    for (int e = 0; e < 256; ++e) {
        const int h = e >> 7, sub = (e >> 5) & 3, l = e & 31;
        const uint8_t lb = ql[64 * h + 32 * (sub & 1) + l];
        const int nib = (sub & 2) ? (lb >> 4) : (lb & 15);
        const int hi2 = (qh[32 * h + l] >> (2 * sub)) & 3;
        const int8_t q = (int8_t)((int8_t)(nib | (hi2 << 4)) - 32);
        const int8_t s = sc[8 * h + 2 * sub + (l >> 4)];
        y[e] = d * (float)s * (float)q; /* left to right: (d*s)*q */
    }
}

/* src/ops/dequant_kernels.cpp:325-359, tests/mxfp4_dequant_test.cpp:37-64,
 * include/ie/quant_blocks.hpp:46-54 */
static const int8_t kMxfp4Lut[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
ORC_API float orc_e8m0_half(uint8_t e) {
    return u2f(e < 2u ? (0x00200000u << e) : ((uint32_t)(e - 1u) << 23));
}
static void deq_mxfp4(const uint8_t* b, float* y) {
    const float d = orc_e8m0_half(b[0]);
    for (int j = 0; j < 16; ++j) {
        y[j] = (float)kMxfp4Lut[b[1 + j] & 15] * d;
        y[j + 16] = (float)kMxfp4Lut[b[1 + j] >> 4] * d;
    }
}

/* Q4_0: {fp16 d; u8 qs[16]}, w[j] = d * ((qs[j] & 15) - 8), w[j+16] = d * ((qs[j] >> 4) - 8)
 * (include/ie/quant_blocks.hpp:32-43, src/ops/gemv_q4_0.cpp:3-8) */
static void deq_q4_0(const uint8_t* b, float* y) {
    const float d = orc_fp16_to_fp32(rd16(b));
    for (int j = 0; j < 16; ++j) {
        y[j] = d * (float)((int)(b[2 + j] & 15) - 8);
        y[j + 16] = d * (float)((int)(b[2 + j] >> 4) - 8);
    }
}

ORC_API int orc_block_elems(int fmt) { return (fmt == ORC_Q8_0 || fmt == ORC_MXFP4 || fmt == ORC_Q4_0) ? 32 : 256; }
ORC_API int orc_block_bytes(int fmt) {
    switch (fmt) {
        case ORC_Q8_0: return Q8_0_BYTES;
        case ORC_Q4_K: return Q4_K_BYTES;
        case ORC_Q6_K: return Q6_K_BYTES;
        case ORC_MXFP4: return MXFP4_BYTES;
        case ORC_Q5_K: return Q5_K_BYTES;
        case ORC_Q4_0: return Q4_0_BYTES;
    }
    return 0;
}
static void deq_block(int fmt, const uint8_t* b, float* y) {
    switch (fmt) {
        case ORC_Q8_0: deq_q8_0(b, y); break;
        case ORC_Q4_K: deq_q4_K(b, y); break;
        case ORC_Q6_K: deq_q6_K(b, y); break;
        case ORC_MXFP4: deq_mxfp4(b, y); break;
        case ORC_Q5_K: deq_q5_K(b, y); break;
        case ORC_Q4_0: deq_q4_0(b, y); break;
    }
}

/* dequant_*_buffer, include/ie/dequant_ref.hpp:98-115 */
ORC_API void orc_dequant(int fmt, const void* packed, size_t n_elems, float* out) {
    const int be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
    const size_t nb = n_elems / (size_t)be;
#pragma omp parallel for schedule(static) if (nb > 4096)
    for (size_t i = 0; i < nb; ++i) deq_block(fmt, (const uint8_t*)packed + i * bb, out + i * be);
}

/* Bt[k*N + n] = half(W[n][k])   (src/ops/dequant_kernels.cpp:282-320) as fp16 bits */
ORC_API void orc_dequant_to_Bt(int fmt, const void* packed, uint32_t K, uint32_t N, uint16_t* Bt) {
    const int be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
    const size_t bpr = K / (size_t)be;
#pragma omp parallel for schedule(static)
    for (uint32_t n = 0; n < N; ++n) {
        float tmp[256];
        for (size_t b = 0; b < bpr; ++b) {
            deq_block(fmt, (const uint8_t*)packed + ((size_t)n * bpr + b) * bb, tmp);
            for (int i = 0; i < be; ++i) Bt[((size_t)b * be + i) * N + n] = orc_fp32_to_fp16(tmp[i]);
        }
    }
}

/* ---------------------------------------------------------------- encoders */
/* ggml's magic-number round-to-nearest-even (src/loaders/quantize_q4k.cpp:11-16) */
static inline int nearest_int(float v) {
    const float t = v + 12582912.f;
    int i;
    memcpy(&i, &t, 4);
    return (i & 0x007fffff) - 0x00400000;
}
static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* make_qkx2_quants, src/loaders/quantize_q4k.cpp:22-76 (ggml-quants.c).  The
 * arithmetic (float sums in this order) is the bit-compat contract. */
static float qkx2(int n, int nmax, const float* x, const float* w, uint8_t* L, float* the_min, uint8_t* Laux,
                  float rmin, float rdelta, int nstep) {
    float mn = x[0], mx = x[0], sum_w = w[0], sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (mn > 0) mn = 0;
    if (mx == mn) {
        memset(L, 0, (size_t)n);
        *the_min = -mn;
        return 0.f;
    }
    float iscale = nmax / (mx - mn), scale = 1.f / iscale, best = 0;
    for (int i = 0; i < n; ++i) {
        L[i] = (uint8_t)clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
        const float diff = scale * L[i] + mn - x[i];
        best += w[i] * diff * diff;
    }
    if (nstep < 1) {
        *the_min = -mn;
        return scale;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (mx - mn);
        float sl = 0, sl2 = 0, sxl = 0;
        for (int i = 0; i < n; ++i) {
            const int l = clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
            Laux[i] = (uint8_t)l;
            sl += w[i] * l;
            sl2 += w[i] * l * l;
            sxl += w[i] * l * x[i];
        }
        const float D = sum_w * sl2 - sl * sl;
        if (D > 0) {
            float ts = (sum_w * sxl - sum_x * sl) / D, tm = (sl2 * sum_x - sl * sxl) / D;
            if (tm > 0) {
                tm = 0;
                ts = sxl / sl2;
            }
            float err = 0;
            for (int i = 0; i < n; ++i) {
                const float diff = ts * Laux[i] + tm - x[i];
                err += w[i] * diff * diff;
            }
            if (err < best) {
                memcpy(L, Laux, (size_t)n);
                best = err;
                scale = ts;
                mn = tm;
            }
        }
    }
    *the_min = -mn;
    return scale;
}

/* quantize_row_q4_K, src/loaders/quantize_q4k.cpp:87-144 */
ORC_API void orc_quantize_row_q4_K(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t i = 0; i < k / 256; ++i, x += 256, y += Q4_K_BYTES) {
        uint8_t L[256], Laux[32], *scales = y + 4;
        float wts[32], mins[8], scs[8], max_scale = 0, max_min = 0;
        memset(y, 0, Q4_K_BYTES);
        for (int j = 0; j < 8; ++j) {
            float s2 = 0;
            for (int l = 0; l < 32; ++l) s2 += x[32 * j + l] * x[32 * j + l];
            const float av = sqrtf(s2 / 32);
            for (int l = 0; l < 32; ++l) wts[l] = av + fabsf(x[32 * j + l]);
            scs[j] = qkx2(32, 15, x + 32 * j, wts, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
            max_scale = max_scale > scs[j] ? max_scale : scs[j]; /* this form keeps -0.0 from an all-zero */
            max_min = max_min > mins[j] ? max_min : mins[j];       /* sub-block, as the reference does    */
        }
        const float inv_s = max_scale > 0 ? 63.f / max_scale : 0.f, inv_m = max_min > 0 ? 63.f / max_min : 0.f;
        for (int j = 0; j < 8; ++j) {
            int ls = nearest_int(inv_s * scs[j]), lm = nearest_int(inv_m * mins[j]);
            if (ls > 63) ls = 63;
            if (lm > 63) lm = 63;
            if (j < 4) {
                scales[j] = (uint8_t)ls;
                scales[j + 4] = (uint8_t)lm;
            } else {
                scales[j + 4] = (uint8_t)((ls & 15) | ((lm & 15) << 4));
                scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        const uint16_t hd = orc_fp32_to_fp16(max_scale / 63.f), hm = orc_fp32_to_fp16(max_min / 63.f);
        y[0] = (uint8_t)hd; y[1] = (uint8_t)(hd >> 8); y[2] = (uint8_t)hm; y[3] = (uint8_t)(hm >> 8);
        for (int j = 0; j < 8; ++j) {
            uint8_t sc, m;
            orc_get_scale_min_k4(j, scales, &sc, &m);
            const float d = orc_fp16_to_fp32(hd) * sc;
            if (!d) continue;
            const float dm = orc_fp16_to_fp32(hm) * m;
            for (int ii = 0; ii < 32; ++ii) L[32 * j + ii] = (uint8_t)clampi(nearest_int((x[32 * j + ii] + dm) / d), 0, 15);
        }
        uint8_t* q = y + 16;
        for (int j = 0; j < 256; j += 64, q += 32)
            for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
    }
}

/* make_qx_quants(rmse_type=1), src/loaders/quantize_q6k.cpp:27-67 */
static float qx_quants(int n, int nmax, const float* x, int8_t* L) {
    float mx = 0, amax = 0;
    for (int i = 0; i < n; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            mx = x[i];
        }
    }
    if (amax < 1e-15f) {
        memset(L, 0, (size_t)n);
        return 0.f;
    }
    float iscale = -(float)nmax / mx, slx = 0, sl2 = 0;
    for (int i = 0; i < n; ++i) {
        const int l = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        slx += w * x[i] * l;
        sl2 += w * l * l;
    }
    float scale = sl2 ? slx / sl2 : 0.f, best = scale * slx;
    for (int is = -9; is <= 9; ++is) {
        if (!is) continue;
        iscale = -(nmax + 0.1f * is) / mx;
        slx = sl2 = 0;
        for (int i = 0; i < n; ++i) {
            const int l = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
            const float w = x[i] * x[i];
            slx += w * x[i] * l;
            sl2 += w * l * l;
        }
        if (sl2 > 0 && slx * slx > best * sl2) {
            for (int i = 0; i < n; ++i) L[i] = (int8_t)(nmax + clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1));
            scale = slx / sl2;
            best = scale * slx;
        }
    }
    return scale;
}

/* quantize_row_q6_K, src/loaders/quantize_q6k.cpp:71-127 */
ORC_API void orc_quantize_row_q6_K(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t i = 0; i < k / 256; ++i, x += 256, y += Q6_K_BYTES) {
        int8_t L[256];
        float scs[16], max_scale = 0, max_abs = 0;
        for (int ib = 0; ib < 16; ++ib) {
            scs[ib] = qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
            const float a = fabsf(scs[ib]);
            if (a > max_abs) {
                max_abs = a;
                max_scale = scs[ib];
            }
        }
        memset(y, 0, Q6_K_BYTES);
        if (max_abs < 1e-15f) continue; /* all-zero block, d = +0 */
        const float iscale = -128.f / max_scale;
        const uint16_t hd = orc_fp32_to_fp16(1.f / iscale);
        y[208] = (uint8_t)hd; y[209] = (uint8_t)(hd >> 8);
        int8_t* sc = (int8_t*)(y + 192);
        for (int ib = 0; ib < 16; ++ib) {
            const int v = nearest_int(iscale * scs[ib]);
            sc[ib] = (int8_t)(v > 127 ? 127 : v);
        }
        for (int j = 0; j < 16; ++j) {
            const float d = orc_fp16_to_fp32(hd) * sc[j];
            if (!d) continue;
            for (int ii = 0; ii < 16; ++ii) L[16 * j + ii] = (int8_t)(clampi(nearest_int(x[16 * j + ii] / d), -32, 31) + 32);
        }
        uint8_t *ql = y, *qh = y + 128;
        for (int j = 0; j < 256; j += 128, ql += 64, qh += 32)
            for (int l = 0; l < 32; ++l) {
                const uint8_t a = (uint8_t)L[j + l], b = (uint8_t)L[j + l + 32], c = (uint8_t)L[j + l + 64], e = (uint8_t)L[j + l + 96];
                ql[l] = (uint8_t)((a & 15) | ((c & 15) << 4));
                ql[l + 32] = (uint8_t)((b & 15) | ((e & 15) << 4));
                qh[l] = (uint8_t)((a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6));
            }
    }
}

/* Q8_0 encode recipe of tools/q8_0_repack_bench.cpp:62-74: d = fp16(amax/127),
 * q = lround(x * 127/amax) (zero block -> d=0,q=0). */
ORC_API void orc_quantize_row_q8_0(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t i = 0; i < k / 32; ++i, x += 32, y += Q8_0_BYTES) {
        float amax = 0;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
        const uint16_t hd = orc_fp32_to_fp16(amax / 127.f);
        const float inv = amax > 0 ? 127.f / amax : 0.f;
        y[0] = (uint8_t)hd; y[1] = (uint8_t)(hd >> 8);
        for (int j = 0; j < 32; ++j) ((int8_t*)y)[2 + j] = (int8_t)clampi((int)lroundf(x[j] * inv), -127, 127);
    }
}

/* MXFP4 encoder.  NOT in the reference (gpt-oss GGUFs ship MXFP4 and are never
 * re-quantized, quant_blocks.hpp:54).  Fixture generator only: pick the smallest
 * e with amax <= 12 * 2^(e-128), then the nearest code (ties to the smaller
 * magnitude).  Pinned by decode(encode(x)) error <= half a code step. */
ORC_API void orc_quantize_row_mxfp4(const float* x, void* out, int64_t k) {
    static const float mag[8] = {0, 1, 2, 3, 4, 6, 8, 12};
    uint8_t* y = (uint8_t*)out;
    for (int64_t i = 0; i < k / 32; ++i, x += 32, y += MXFP4_BYTES) {
        float amax = 0;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
        int e = 0;
        if (amax > 0) {
            int ex;
            frexpf(amax / 12.f, &ex); /* amax/12 = f * 2^ex, f in [0.5,1) */
            /* smallest e with 2^(e-128) >= amax/12 */
            e = ex + 128;
            if (ldexpf(1.f, ex - 1) >= amax / 12.f) e -= 1;
            e = clampi(e, 0, 254);
        }
        const float d = orc_e8m0_half((uint8_t)e), inv = d > 0 ? 1.f / d : 0.f;
        uint8_t code[32];
        for (int j = 0; j < 32; ++j) {
            const float a = fabsf(x[j]) * inv;
            int best = 0;
            for (int c = 1; c < 8; ++c)
                if (fabsf(a - mag[c]) < fabsf(a - mag[best])) best = c;
            code[j] = (uint8_t)(best | ((x[j] < 0 && best) ? 8 : 0));
        }
        y[0] = (uint8_t)e;
        for (int j = 0; j < 16; ++j) y[1 + j] = (uint8_t)(code[j] | (code[j + 16] << 4));
    }
}

/* Q4_0 encoder.  NOT in the reference (Gemma-4 QAT GGUFs ship Q4_0).  Fixture generator only, after ggml's
 * published quantize_row_q4_0_ref: d = (value of largest magnitude) / -8, q = min(15, trunc(x/d + 8.5)). */
ORC_API void orc_quantize_row_q4_0(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t i = 0; i < k / 32; ++i, x += 32, y += Q4_0_BYTES) {
        float amax = 0, mx = 0;
        for (int j = 0; j < 32; ++j)
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
        const float d = mx / -8.f, id = d != 0.f ? 1.f / d : 0.f;
        const uint16_t hd = orc_fp32_to_fp16(d);
        y[0] = (uint8_t)hd; y[1] = (uint8_t)(hd >> 8);
        for (int j = 0; j < 16; ++j) {
            const int q0 = clampi((int)(x[j] * id + 8.5f), 0, 15), q1 = clampi((int)(x[j + 16] * id + 8.5f), 0, 15);
            y[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

ORC_API void orc_quantize_rows(int fmt, const float* x, void* out, int64_t n_rows, int64_t k) {
    const int64_t rb = k / orc_block_elems(fmt) * orc_block_bytes(fmt);
#pragma omp parallel for schedule(dynamic, 8)
    for (int64_t r = 0; r < n_rows; ++r) {
        uint8_t* o = (uint8_t*)out + r * rb;
        const float* xr = x + r * k;
        switch (fmt) {
            case ORC_Q8_0: orc_quantize_row_q8_0(xr, o, k); break;
            case ORC_Q4_K: orc_quantize_row_q4_K(xr, o, k); break;
            case ORC_Q6_K: orc_quantize_row_q6_K(xr, o, k); break;
            case ORC_MXFP4: orc_quantize_row_mxfp4(xr, o, k); break;
            case ORC_Q4_0: orc_quantize_row_q4_0(xr, o, k); break;
        }
    }
}

/* ---------------------------------------------------------------- activation quantizers
 * quantize_q8_1, src/ops/gemv_q8dot.cpp:94-124: d = amax/127, inv = 127/amax
 * (0 when amax==0), q = round-half-away(v*inv), s = d * float(sum q).  The
 * input is the fp32 value of the (fp16) activation. */
ORC_API void orc_quantize_q8_1(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t b = 0; b < k / 32; ++b, x += 32, y += Q8_1X_BYTES) {
        float amax = 0;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
        const float d = amax / 127.0f, inv = amax > 0.f ? 127.0f / amax : 0.f;
        int32_t sum = 0;
        for (int j = 0; j < 32; ++j) {
            const int32_t q = (int32_t)roundf(x[j] * inv);
            ((int8_t*)y)[8 + j] = (int8_t)q;
            sum += q;
        }
        const float s = d * (float)sum;
        memcpy(y, &d, 4);
        memcpy(y + 4, &s, 4);
    }
}
/* quantize_q8_1s, src/ops/gemv_q8dot.cpp:57-91 */
ORC_API void orc_quantize_q8_1s(const float* x, void* out, int64_t k) {
    uint8_t* y = (uint8_t*)out;
    for (int64_t b = 0; b < k / 32; ++b, x += 32, y += Q8_1S_BYTES) {
        float amax = 0;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
        const float d = amax / 127.0f, inv = amax > 0.f ? 127.0f / amax : 0.f;
        int32_t lo = 0, hi = 0;
        for (int j = 0; j < 32; ++j) {
            const int32_t q = (int32_t)roundf(x[j] * inv);
            ((int8_t*)y)[16 + j] = (int8_t)q;
            if (j < 16) lo += q; else hi += q;
        }
        const float hdr[4] = {d, d * (float)lo, d * (float)hi, 0.f};
        memcpy(y, hdr, 16);
    }
}

/* ---------------------------------------------------------------- reference matmuls */
/* Float-activation chain = the reference's CPU path: dequant the row to fp32,
 * then a sequential fp32 dot (tests/unit/gemv_q4k_test.cpp:78-83,152-159).
 * W is [N][K/blk] blocks; x fp32 [T][K]; y fp32 [T][N]. */
ORC_API void orc_gemv_f32chain(int fmt, const void* W, const float* x, float* y, uint32_t K, uint32_t N, uint32_t T) {
    const size_t rb = (size_t)K / orc_block_elems(fmt) * orc_block_bytes(fmt);
#pragma omp parallel
    {
        float* w = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            orc_dequant(fmt, (const uint8_t*)W + n * rb, K, w);
            for (uint32_t t = 0; t < T; ++t) {
                float acc = 0.f;
                const float* xt = x + (size_t)t * K;
                for (uint32_t k = 0; k < K; ++k) acc += xt[k] * w[k];
                y[(size_t)t * N + n] = acc;
            }
        }
        free(w);
    }
}
/* Same products accumulated in double: the tight target for fp32 kernels. */
ORC_API void orc_gemv_f64(int fmt, const void* W, const float* x, double* y, uint32_t K, uint32_t N, uint32_t T, int round_w_fp16) {
    const size_t rb = (size_t)K / orc_block_elems(fmt) * orc_block_bytes(fmt);
#pragma omp parallel
    {
        float* w = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            orc_dequant(fmt, (const uint8_t*)W + n * rb, K, w);
            if (round_w_fp16) orc_round_fp16_n(w, K); /* XMX/`Bt` routes round weights to fp16: gemm_q4k_xmx.cpp:107-108 */
            for (uint32_t t = 0; t < T; ++t) {
                double acc = 0.0;
                const float* xt = x + (size_t)t * K;
                for (uint32_t k = 0; k < K; ++k) acc += (double)xt[k] * (double)w[k];
                y[(size_t)t * N + n] = acc;
            }
        }
        free(w);
    }
}
/* q8-chain: dequantized fp32 weight times (d8 * q8) in double
 * (tests/gemv_q6k_ktiled_test.cpp:89-103, tests/unit/q8dot_test.cpp:79-94).
 * xq8 = T rows of K/32 block_q8_1x. */
ORC_API void orc_gemv_q8chain(int fmt, const void* W, const void* xq8, double* y, uint32_t K, uint32_t N, uint32_t T) {
    const size_t rb = (size_t)K / orc_block_elems(fmt) * orc_block_bytes(fmt);
#pragma omp parallel
    {
        float* w = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            orc_dequant(fmt, (const uint8_t*)W + n * rb, K, w);
            for (uint32_t t = 0; t < T; ++t) {
                const uint8_t* xb = (const uint8_t*)xq8 + (size_t)t * (K / 32) * Q8_1X_BYTES;
                double acc = 0.0;
                for (uint32_t b = 0; b < K / 32; ++b, xb += Q8_1X_BYTES) {
                    float d8;
                    memcpy(&d8, xb, 4);
                    const int8_t* q = (const int8_t*)(xb + 8);
                    for (int i = 0; i < 32; ++i) acc += (double)w[b * 32 + i] * (double)d8 * (double)q[i];
                }
                y[(size_t)t * N + n] = acc;
            }
        }
        free(w);
    }
}
/* q8_1s-chain: the int-dot fold with the STORED half sums of block_q8_1s rows {d, s0, s1, pad, qs[32]}, the form the
 * reference's expert-grouped K-quant kernels evaluate:
 *   Q4_K  y += (d*sc)*(d8*idot) - (dmin*m)*(s0 + s1)   per 32-element sub-block (src/ops/moe_fused.cpp:672-687;
 *         batched dense form with one half sum per lane, src/ops/gemv_q8dot.cpp:552-567)
 *   Q6_K  y += (d*sc16)*(d8*idot_u - 32*s_half)        per 16-element group, idot_u over the unsigned 6-bit codes
 *         (src/ops/moe_fused.cpp:1882-1891)
 * Formats without a min term never read the sums: d_w * d8 * idot per block.  Accumulated in double.
 * xq8s = T rows of K/32 block_q8_1s. */
ORC_API void orc_int_codes(int fmt, const void* row, uint32_t K, int8_t* codes);
ORC_API void orc_gemv_q8schain(int fmt, const void* W, const void* xq8s, double* y, uint32_t K, uint32_t N, uint32_t T) {
    const size_t rb = (size_t)K / orc_block_elems(fmt) * orc_block_bytes(fmt);
#pragma omp parallel
    {
        int8_t* codes = (int8_t*)malloc((size_t)K);
        float* w = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            const uint8_t* row = (const uint8_t*)W + n * rb;
            orc_int_codes(fmt, row, K, codes);
            if (fmt != ORC_Q4_K && fmt != ORC_Q6_K) orc_dequant(fmt, row, K, w);
            for (uint32_t t = 0; t < T; ++t) {
                const uint8_t* xb = (const uint8_t*)xq8s + (size_t)t * (K / 32) * Q8_1S_BYTES;
                double acc = 0.0;
                for (uint32_t b = 0; b < K / 32; ++b, xb += Q8_1S_BYTES) {
                    float hdr[4];
                    memcpy(hdr, xb, 16);
                    const int8_t* q = (const int8_t*)(xb + 16);
                    const double d8 = hdr[0];
                    if (fmt == ORC_Q4_K) {
                        const uint8_t* blk = row + (size_t)(b / 8) * Q4_K_BYTES;
                        uint8_t sc, mn;
                        orc_get_scale_min_k4((int)(b % 8), blk + 4, &sc, &mn);
                        const float d1 = orc_fp16_to_fp32(rd16(blk)) * (float)sc, m1 = orc_fp16_to_fp32(rd16(blk + 2)) * (float)mn;
                        long idot = 0;
                        for (int i = 0; i < 32; ++i) idot += (long)codes[b * 32 + i] * q[i];
                        acc += (double)d1 * (d8 * (double)idot) - (double)m1 * ((double)hdr[1] + (double)hdr[2]);
                    } else if (fmt == ORC_Q6_K) {
                        const uint8_t* blk = row + (size_t)(b / 8) * Q6_K_BYTES;
                        const float d = orc_fp16_to_fp32(rd16(blk + 208));
                        for (int hf = 0; hf < 2; ++hf) {
                            const float c = d * (float)(int8_t)blk[192 + (b % 8) * 2 + hf];
                            long idot_u = 0;
                            for (int i = 0; i < 16; ++i) idot_u += (long)(codes[b * 32 + hf * 16 + i] + 32) * q[hf * 16 + i];
                            acc += (double)c * (d8 * (double)idot_u - 32.0 * (double)hdr[1 + hf]);
                        }
                    } else {
                        for (int i = 0; i < 32; ++i) acc += (double)w[b * 32 + i] * d8 * (double)q[i];
                    }
                }
                y[(size_t)t * N + n] = acc;
            }
        }
        free(codes);
        free(w);
    }
}
/* Exact integer dot of one weight row against one q8 row, per 32-element
 * block, for brute-force checks of the int-dot kernels' integer part.
 * qw = the format's integer code (Q8_0: qs; Q4_K: nibble 0..15; Q6_K: q-32;
 * MXFP4: doubled E2M1 value; Q4_0: nibble - 8; Q5_K: 5-bit code 0..31). */
ORC_API void orc_int_codes(int fmt, const void* row, uint32_t K, int8_t* codes) {
    const int be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
    for (uint32_t b = 0; b < K / be; ++b) {
        const uint8_t* p = (const uint8_t*)row + (size_t)b * bb;
        int8_t* c = codes + (size_t)b * be;
        if (fmt == ORC_Q8_0) memcpy(c, p + 2, 32);
        else if (fmt == ORC_MXFP4)
            for (int j = 0; j < 16; ++j) { c[j] = kMxfp4Lut[p[1 + j] & 15]; c[j + 16] = kMxfp4Lut[p[1 + j] >> 4]; }
        else if (fmt == ORC_Q4_0)
            for (int j = 0; j < 16; ++j) { c[j] = (int8_t)((p[2 + j] & 15) - 8); c[j + 16] = (int8_t)((p[2 + j] >> 4) - 8); }
        else if (fmt == ORC_Q5_K)
            for (int e = 0; e < 256; ++e) {
                const uint8_t by = p[48 + 32 * (e >> 6) + (e & 31)];
                c[e] = (int8_t)((((e >> 5) & 1) ? by >> 4 : by & 15) | (((p[16 + (e & 31)] >> (e >> 5)) & 1) << 4));
            }
        else if (fmt == ORC_Q4_K)
            for (int e = 0; e < 256; ++e) { const uint8_t by = p[16 + 32 * (e >> 6) + (e & 31)]; c[e] = (int8_t)(((e >> 5) & 1) ? by >> 4 : by & 15); }
        else
            for (int e = 0; e < 256; ++e) {
                const int h = e >> 7, sub = (e >> 5) & 3, l = e & 31;
                const uint8_t lb = p[64 * h + 32 * (sub & 1) + l];
                c[e] = (int8_t)((((sub & 2) ? lb >> 4 : lb & 15) | (((p[128 + 32 * h + l] >> (2 * sub)) & 3) << 4)) - 32);
            }
    }
}

/* ---------------------------------------------------------------- epilogues
 * swiglu: src/ops/elementwise.cpp:449-466; swiglu_oai: :468-492 (alpha 1.702,
 * limit 7).  exp in double here; the device uses an approximate exp. */
ORC_API float orc_swiglu(float g, float u) { return (float)(g / (1.0 + exp(-(double)g))) * u; }
ORC_API float orc_swiglu_oai(float g, float u, float alpha, float limit) {
    const float x = fminf(g, limit), z = fmaxf(fminf(u, limit), -limit);
    return (float)(x / (1.0 + exp((double)alpha * -(double)x))) * (z + 1.f);
}

/* ---------------------------------------------------------------- MoE routing / packing
 * route_from_logits, src/model/gptoss.cpp:29-47: softmax over all E, top-k by
 * probability, renormalise over the k picks, sort ascending by expert id.
 * Ties are broken towards the lower expert id (deterministic restatement). */
ORC_API void orc_route_from_logits(const float* logit, uint32_t E, uint32_t k, int32_t* ids, float* wts) {
    float m = logit[0];
    for (uint32_t e = 1; e < E; ++e) m = fmaxf(m, logit[e]);
    double sum = 0.0;
    float* p = (float*)malloc(E * sizeof(float));
    uint8_t* used = (uint8_t*)calloc(E, 1);
    for (uint32_t e = 0; e < E; ++e) { p[e] = expf(logit[e] - m); sum += p[e]; }
    for (uint32_t e = 0; e < E; ++e) p[e] = (float)(p[e] / sum);
    float wsum = 0.f;
    for (uint32_t j = 0; j < k; ++j) {
        int best = -1;
        for (uint32_t e = 0; e < E; ++e)
            if (!used[e] && (best < 0 || p[e] > p[best])) best = (int)e;
        used[best] = 1;
        wsum += p[best];
    }
    uint32_t o = 0;
    for (uint32_t e = 0; e < E; ++e)
        if (used[e]) { ids[o] = (int32_t)e; wts[o] = p[e] / wsum; ++o; }
    free(p);
    free(used);
}

/* build_moe_packing, src/model/qwen3moe_pack.cpp:5-31: stable counting sort of
 * the T*K (token, slot) pairs by expert id.  topk_ids[T*K] per token ascending. */
ORC_API void orc_build_moe_packing(const int32_t* topk_ids, const float* topk_w, uint32_t T, uint32_t K, uint32_t E,
                                   uint32_t* expert_offsets, int32_t* sorted_idx, float* weights_packed, int32_t* tk_to_packed) {
    uint32_t* cur = (uint32_t*)calloc(E + 1, sizeof(uint32_t));
    memset(expert_offsets, 0, (E + 1) * sizeof(uint32_t));
    for (uint32_t i = 0; i < T * K; ++i) expert_offsets[topk_ids[i] + 1]++;
    for (uint32_t e = 0; e < E; ++e) expert_offsets[e + 1] += expert_offsets[e];
    memcpy(cur, expert_offsets, E * sizeof(uint32_t));
    for (uint32_t t = 0; t < T; ++t)
        for (uint32_t s = 0; s < K; ++s) {
            const uint32_t pos = cur[topk_ids[t * K + s]]++;
            sorted_idx[pos] = (int32_t)t;
            weights_packed[pos] = topk_w[t * K + s];
            tk_to_packed[t * K + s] = (int32_t)pos;
        }
    free(cur);
}

/* ---------------------------------------------------------------- repacks
 * MXFP4 AoS -> SoA planes, src/model/gptoss.cpp:180-208 / gemv_mxfp4.cpp:13-16:
 * qs_plane[i*16 + j] = block(i).qs[j];  e_plane[i] = block(i).e */
ORC_API void orc_repack_mxfp4_to_soa(const void* blocks, size_t n_blocks, uint8_t* qs_plane, uint8_t* e_plane) {
    const uint8_t* b = (const uint8_t*)blocks;
    for (size_t i = 0; i < n_blocks; ++i) {
        e_plane[i] = b[i * MXFP4_BYTES];
        memcpy(qs_plane + i * 16, b + i * MXFP4_BYTES + 1, 16);
    }
}
/* Q8_0 AoS -> SoA, src/model/qwen35moe_split.cpp:134-144 / gemv_q8dot.cpp:601-607:
 * qs_W[i*32 + j] = block(i).qs[j];  d_W[i] = block(i).d */
ORC_API void orc_repack_q8_0_to_soa(const void* blocks, size_t n_blocks, int8_t* qs_plane, uint16_t* d_plane) {
    const uint8_t* b = (const uint8_t*)blocks;
    for (size_t i = 0; i < n_blocks; ++i) {
        d_plane[i] = rd16(b + i * Q8_0_BYTES);
        memcpy(qs_plane + i * 32, b + i * Q8_0_BYTES + 2, 32);
    }
}
