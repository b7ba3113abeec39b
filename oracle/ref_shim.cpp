// ref_shim.cpp — C-ABI window onto the reference's own SYCL-free host code.
//
// TEST INFRASTRUCTURE ONLY.  Compiled (by oracle/Makefile, only where the
// reference tree is mounted) together with the reference sources *where they
// lie*; nothing from the reference is copied into this repository.  The
// resulting oracle/_ref/libmxref.so is used to pin oracle/mxq_oracle.c and to
// write the fixtures under tests/golden/.
//
// Reference units compiled in: include/ie/{quant_blocks,dequant_ref,quantize,
// qwen3moe_pack,dp4a,quant_soa}.hpp, src/loaders/quantize_q4k.cpp,
// src/loaders/quantize_q6k.cpp, src/model/qwen3moe_pack.cpp.
#include "ie/dequant_ref.hpp"
#include "ie/dp4a.hpp"
#include "ie/quant_blocks.hpp"
#include "ie/quant_soa.hpp"
#include "ie/quantize.hpp"
#include "ie/qwen3moe_pack.hpp"

#include <cstring>
#include <utility>
#include <vector>

extern "C" {

float ref_fp16_to_fp32(uint16_t h) { return ie::fp16_to_fp32(h); }
uint16_t ref_fp32_to_fp16(float f) { return ie::fp32_to_fp16(f); }

void ref_get_scale_min_k4(int j, const uint8_t* q, uint8_t* sc, uint8_t* m) {
    ie::ref::get_scale_min_k4(j, q, *sc, *m);
}

// fmt: 0 Q8_0, 1 Q4_K, 2 Q6_K, 4 Q5_K  (MXFP4 has no host routine in the reference headers)
int ref_dequant(int fmt, const void* packed, size_t n, float* out) {
    switch (fmt) {
        case 0: ie::ref::dequant_q8_0_buffer(packed, n, out); return 0;
        case 1: ie::ref::dequant_q4_K_buffer(packed, n, out); return 0;
        case 2: ie::ref::dequant_q6_K_buffer(packed, n, out); return 0;
        case 4: ie::ref::dequant_q5_K_buffer(packed, n, out); return 0;
    }
    return 1;
}

void ref_quantize_row_q4_K(const float* x, void* out, int64_t k) {
    ie::quantize_row_q4_K(x, static_cast<ie::block_q4_K*>(out), k);
}
void ref_quantize_row_q6_K(const float* x, void* out, int64_t k) {
    ie::quantize_row_q6_K(x, static_cast<ie::block_q6_K*>(out), k);
}

int32_t ref_dp4a_us(uint32_t a, int32_t b, int32_t c) { return ie::dp4a_us(a, b, c); }
int32_t ref_dp4a_ss(int32_t a, int32_t b, int32_t c) { return ie::dp4a_ss(a, b, c); }

// topk_ids / topk_w: [T*K], per token ascending by expert id.
void ref_build_moe_packing(const int32_t* topk_ids, const float* topk_w, uint32_t T, uint32_t K, uint32_t E,
                           uint32_t* expert_offsets, int32_t* sorted_idx, float* weights_packed,
                           int32_t* tk_to_packed) {
    std::vector<std::vector<std::pair<uint32_t, float>>> routes(T);
    for (uint32_t t = 0; t < T; ++t)
        for (uint32_t s = 0; s < K; ++s) routes[t].emplace_back(uint32_t(topk_ids[t * K + s]), topk_w[t * K + s]);
    ie::MoePacking pk;
    ie::build_moe_packing(routes, E, K, pk);
    std::memcpy(expert_offsets, pk.expert_offsets.data(), (E + 1) * sizeof(uint32_t));
    std::memcpy(sorted_idx, pk.sorted_idx.data(), size_t(T) * K * sizeof(int32_t));
    std::memcpy(weights_packed, pk.weights_packed.data(), size_t(T) * K * sizeof(float));
    std::memcpy(tk_to_packed, pk.tk_to_packed.data(), size_t(T) * K * sizeof(int32_t));
}

void ref_repack_moe_q4k_soa(const uint8_t* src, uint8_t* dst, uint32_t E, uint64_t nb) {
    ie::repack_moe_q4k_soa_host(src, dst, E, nb);
}
void ref_repack_moe_q6k_soa(const uint8_t* src, uint8_t* dst, uint32_t E, uint64_t nb) {
    ie::repack_moe_q6k_soa_host(src, dst, E, nb);
}

// The reference's CPU GEMV path as its tests run it: whole-row dequant to fp32
// via ie::ref::dequant_*_buffer, then a sequential fp32 dot.  One thread.
int ref_gemv_cpu(int fmt, const void* W, const float* x, float* y, uint32_t K, uint32_t N) {
    const size_t rb = fmt == 0 ? size_t(K) / 32 * 34 : fmt == 1 ? size_t(K) / 256 * 144 : size_t(K) / 256 * 210;
    std::vector<float> w(K);
    for (uint32_t n = 0; n < N; ++n) {
        if (ref_dequant(fmt, static_cast<const uint8_t*>(W) + n * rb, K, w.data())) return 1;
        float acc = 0.f;
        for (uint32_t k = 0; k < K; ++k) acc += x[k] * w[k];
        y[n] = acc;
    }
    return 0;
}

}  // extern "C"
