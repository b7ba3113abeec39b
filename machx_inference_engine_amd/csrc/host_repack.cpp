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

}  // extern "C"
