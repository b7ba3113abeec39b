/*
 * mxq.h — C ABI of the MI355X (gfx950) quantized-weight matmul path.
 *
 * Drop-in replacement boundary for the `src/ops` quantized matmul family of the
 * Mach X inference engine.  Every entry point mirrors one reference free
 * function `sycl::event ie::f(sycl::queue&, <device pointers>, <dims>, deps)`
 * (include/ie/ops.hpp:3-7) with these mechanical changes:
 *   - `sycl::queue&`  -> `mx_stream_t` (a hipStream_t passed as void*; NULL = the
 *                        default stream); ordering is stream order, so there is
 *                        no `deps` argument and no returned event;
 *   - `sycl::half*`   -> `uint16_t*` (IEEE binary16 bit patterns);
 *   - the return value is an `int` status (MX_OK = 0).  Where the reference
 *     silently returns an empty event on an unsupported shape
 *     (src/ops/gemm_q4k_xmx.cpp:120-121) this ABI returns MX_ERR_SHAPE and
 *     launches nothing.  Argument checks run before any HIP call.
 * All pointers are caller-owned device memory unless a comment says "host".
 * Weight layouts are the unchanged GGUF block layouts
 * (include/ie/quant_blocks.hpp) in "W[K,N] column-packed" order: output row n
 * owns K/blk consecutive blocks (src/ops/gemv_q4k.cpp:3-11).
 * Argument order is (K, N) for GEMV and (M, K, N) for GEMM, as in the reference.
 */
#ifndef MXQ_H
#define MXQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mx_stream_t;

enum {
    MX_OK = 0,
    MX_ERR_NULL = 1,        /* a required pointer is NULL */
    MX_ERR_SHAPE = 2,       /* a dimension violates the documented precondition */
    MX_ERR_ALIGN = 3,       /* a pointer violates the documented alignment */
    MX_ERR_LAUNCH = 4,      /* the HIP runtime reported an error (see mx_last_hip_error) */
    MX_ERR_UNSUPPORTED = 5, /* valid arguments, combination not built */
    MX_ERR_IO = 6,          /* a file could not be opened or mapped (see mx_gguf_last_error) */
    MX_ERR_FORMAT = 7,      /* a file is not what its format prescribes (see mx_gguf_last_error) */
    MX_ERR_NOT_FOUND = 8,   /* no tensor / key of that name */
    MX_ERR_WORKSPACE = 9    /* the workspace passed to a *_ws entry point is smaller than the launch needs */
};

const char* mx_status_string(int status);
int mx_last_hip_error(void);  /* hipError_t of the last MX_ERR_LAUNCH on this thread */
int mx_version(void);
/* Optional set-up for the current device: resolves the addresses of the library's per-device scratch arrays (see the
 * batched GEMVs and mx_gemm_* below) so that the first split-K launch does it no more.  Callers that record HIP
 * graphs call it once per device before capturing; everyone else may leave it to the first launch.  */
int mx_init(void);

/* Measurement aid, no counterpart in the reference: reads n_bytes (a multiple of 16, 16-byte aligned) once with the
 * launch geometry of the decode GEMV and no arithmetic, so that a GEMV launch can be priced against a pure read of
 * the same bytes on the same device.  `sink` may be NULL (a word that is practically never written).  */
int mx_probe_stream_read(mx_stream_t s, const void* src, uint64_t n_bytes, uint32_t* sink);
/* Measurement aids, no counterpart in the reference.  mx_probe_read_variant reads n_bytes (a multiple of 1024, 16-byte
 * aligned) once with `workgroups` workgroups of 256 threads that stride over the buffer: `in_flight` 16-byte loads per
 * thread (2, 4, 8, 16) with mode 0 (plain) or 1 (nontemporal), or mode 2: `in_flight` (4, 8, 16) loads of 1 KB per wave
 * straight into LDS.  mx_probe_lane_pattern reads a region (region_bytes incl. 16 spare bytes at its end, rows of
 * `pitch` bytes, pitch % 128 == 0) `iters` times with 16-byte loads whose lanes cover 16 (pattern 0), 32 (1), 64 (2) or
 * 128 (3) contiguous bytes per row, or 128 bytes displaced by 2, 4, 8 bytes (4, 5, 6); each workgroup moves
 * 4 * 64 * pitch * iters bytes.  Both are timed by the caller with events on `s`.  */
int mx_probe_read_variant(mx_stream_t s, const void* src, uint64_t n_bytes, int in_flight, int mode, uint32_t workgroups, uint32_t* sink);
int mx_probe_lane_pattern(mx_stream_t s, const void* region, uint64_t region_bytes, uint32_t pitch, int pattern, uint32_t iters,
                          uint32_t workgroups, uint32_t* sink);

/* ---------------------------------------------------------------- activation quantizers
 * quantize_q8_1   include/ie/ops.hpp:301-304, src/ops/gemv_q8dot.cpp:94-124
 * quantize_q8_1s  include/ie/ops.hpp:307-310, src/ops/gemv_q8dot.cpp:57-91
 * x: n elements (n % 32 == 0; several rows are simply contiguous) -> n/32
 * block_q8_1x (40 B) / block_q8_1s (48 B).  d = amax/127, q = round-half-away,
 * s = d * sum(q).  `_f32` variants take fp32 activations (same math).  */
int mx_quantize_q8_1(mx_stream_t s, const uint16_t* x_f16, void* out_q8, uint64_t n);
int mx_quantize_q8_1_f32(mx_stream_t s, const float* x, void* out_q8, uint64_t n);
int mx_quantize_q8_1s(mx_stream_t s, const uint16_t* x_f16, void* out_q8s, uint64_t n);
int mx_quantize_q8_1s_f32(mx_stream_t s, const float* x, void* out_q8s, uint64_t n);

/* ---------------------------------------------------------------- block dequant
 * dequant_q8_0/q4_K/q5_K/q6_K  include/ie/dequant.hpp, src/ops/dequant_kernels.cpp:55-269
 * dequant_mxfp4           src/ops/dequant_kernels.cpp:325-359
 * Bit-exact with ie::ref::dequant_* (include/ie/dequant_ref.hpp:32-96); fp16
 * output is the single RNE rounding of that fp32 value.  n_elements must be a
 * whole number of blocks.  `_f32` variants write the unrounded fp32 value.  */
int mx_dequant_q8_0(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_q4_K(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_q5_K(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_q6_K(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_mxfp4(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_q8_0_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
int mx_dequant_q4_K_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
int mx_dequant_q5_K_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
int mx_dequant_q6_K_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
int mx_dequant_mxfp4_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
/* dequant_*_to_Bt  src/ops/dequant_kernels.cpp:282-320,392-431,567-609,611-632,364-390:
 * whole matrix -> fp16 Bt[k*N + n].  */
int mx_dequant_q8_0_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q4_K_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q5_K_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q6_K_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_mxfp4_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
/* Q4_0 (Gemma-4 QAT; 18-byte blocks {fp16 d; u8 qs[16]}, w = d * (q - 8), element j in the low and j + 16
 * in the high nibble of qs[j]; include/ie/quant_blocks.hpp:32-43):
 *   dequant_q4_0_to_Bt / dequant_q4_0_soa_to_Bt   include/ie/ops.hpp:550-567, src/ops/gemv_q4_0.cpp:455-477
 * (the flat forms have no counterpart in the reference and exist for symmetry with the other formats)  */
int mx_dequant_q4_0(mx_stream_t s, const void* packed, uint16_t* out_f16, uint64_t n_elements);
int mx_dequant_q4_0_f32(mx_stream_t s, const void* packed, float* out, uint64_t n_elements);
int mx_dequant_q4_0_to_Bt(mx_stream_t s, const void* W, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q4_0_soa_to_Bt(mx_stream_t s, const uint8_t* soa_qs, const uint16_t* soa_d, uint16_t* Bt, uint32_t K, uint32_t N);
/* Transposed dequant of the repacked layouts; bit-identical to the AoS form of the same weights:
 *   dequant_q4_moe_soa_to_Bt   include/ie/dequant.hpp:72-80   one expert region as streams qs | scales | {d,dmin}
 *   dequant_q6_K_soa_to_Bt     include/ie/dequant.hpp:64-71   one expert region as streams ql | qh | scales | d
 *   dequant_q4_soa_to_Bt       include/ie/ops.hpp:453-458, src/ops/gemv_q4_soa.cpp:319-348   natural-order planes
 *   dequant_q6_soa_to_Bt       include/ie/ops.hpp:421-426, src/ops/gemv_q6_soa.cpp:415-444   natural-order planes
 *   dequant_mxfp4_soa_to_Bt    include/ie/dequant.hpp:60-63, src/ops/gemv_mxfp4.cpp:316-341  qs / e planes
 * Any N (the reference's N % 64 == 0 is not required).  */
int mx_dequant_q4_moe_soa_to_Bt(mx_stream_t s, const void* soa_region, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q6_K_soa_to_Bt(mx_stream_t s, const void* soa_region, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q4_soa_to_Bt(mx_stream_t s, const uint8_t* q4_q, const int8_t* q4_sc, const int8_t* q4_mn, const uint16_t* q4_d,
                            const uint16_t* q4_dmin, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_q6_soa_to_Bt(mx_stream_t s, const uint8_t* q6_lo, const uint8_t* q6_hi, const int8_t* q6_sc,
                            const uint16_t* q6_d, uint16_t* Bt, uint32_t K, uint32_t N);
int mx_dequant_mxfp4_soa_to_Bt(mx_stream_t s, const uint8_t* qs_plane, const uint8_t* e_plane, uint16_t* Bt, uint32_t K,
                               uint32_t N);

/* ---------------------------------------------------------------- decode GEMV, int-dot on q8 activations
 * y[n] = sum_k deq(W)[n,k] * (d8 * q8)[k], fp32 accumulate, fp16 out.
 * x_q8: block_q8_1x stream from mx_quantize_q8_1 (8-byte aligned).
 * K % 256 == 0 for K-quants, K % 32 == 0 for Q8_0 / MXFP4.  W 16-byte aligned
 * (Q4_K, SoA planes) or 2-byte aligned (Q6_K, AoS Q8_0).
 *
 * gemv_q4_K_q8          include/ie/ops.hpp:312-316, src/ops/gemv_q8dot.cpp:261-357
 * gemv_q6_K_q8(_ktiled) include/ie/ops.hpp:375-391, src/ops/gemv_q6k.cpp:335-589
 * gemv_q8_0_soa_q8(_g)  include/ie/ops.hpp:351-364, src/ops/gemv_q8dot.cpp:609-707
 * gemv_mxfp4_soa_q8     include/ie/ops.hpp:498-502, src/ops/gemv_mxfp4.cpp:80-154
 * mx_gemv_q8_0_q8 takes the AoS GGUF block_q8_0 array (no reference counterpart:
 * the reference only has the SoA kernel).  */
int mx_gemv_q4_K_q8(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q6_K_q8(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0_q8(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0_soa_q8(mx_stream_t s, const void* x_q8, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y,
                        uint32_t K, uint32_t N);
int mx_gemv_mxfp4_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* qs_plane, const uint8_t* e_plane,
                         uint16_t* y, uint32_t K, uint32_t N);
/* gemv_mxfp4_soa_q8_x2  include/ie/ops.hpp:507-513, src/ops/gemv_mxfp4.cpp:165-250:
 * gate and up share x; per-row fp32 bias (may be NULL) added after the reduce.  */
int mx_gemv_mxfp4_soa_q8_x2(mx_stream_t s, const void* x_q8, const uint8_t* gate_qs, const uint8_t* gate_e,
                            const uint8_t* up_qs, const uint8_t* up_e, const float* gate_bias,
                            const float* up_bias, uint16_t* gate_y, uint16_t* up_y, uint32_t K, uint32_t N);

/* Batched-T variants: weights read once, dotted against T activation rows.
 * x_q8 = T contiguous block_q8_1x rows (row t at block t*(K/32)); y[t*N + n].
 * 1 <= T <= 16 (T > 8 runs as two passes).
 * gemv_q4_K_q8_batched   include/ie/ops.hpp:332-336, src/ops/gemv_q8dot.cpp:375-470
 * gemv_q6_soa_q8_batched include/ie/ops.hpp:420-426 (the reference batches Q6_K only
 *                        in its SoA form; here the GGUF AoS blocks are batched directly)
 * Q8_0 / MXFP4 batched have no reference counterpart (T >= 2 falls to dequant +
 * GEMM there, src/model/qwen35_dense.cpp:811-831).
 *
 * Library-owned scratch (no counterpart in the reference's signatures; it is what lets callers that cannot
 * allocate -- code under HIP graph capture, serving loops, harnesses that forbid hipMalloc -- use these entry
 * points as they are): batched launches with T >= 2 and K >= 8192 whose row groups alone would leave CUs idle
 * split K over workgroups and keep slices x T x N fp32 partial sums in a 2 MB file-scope device array (one copy
 * per device, resolved with hipGetSymbolAddress on first use or by mx_init, never allocated or freed).  Limit:
 * slices * min(T, 8) * N <= 524288 floats (e.g. T = 8, N = 16384); a launch beyond it runs unsplit.  Every call
 * on a device shares that device's array: two such calls that overlap on one device (different streams, graph
 * branches) race on it, exactly as calls sharing the reference's static per-device scratch buffers would
 * (src/model/dense_dispatch.hpp:547-560).  Callers that overlap launches use the *_ws forms below.  */
int mx_gemv_q4_K_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
/* gemv_q4_K_q8s_batched  include/ie/ops.hpp (gemv_q4_K_q8s_batched), src/ops/gemv_q8dot.cpp:483-597: the
 * activation rows are block_q8_1s (48 B, stored half sums s0/s1; 16-byte aligned) from
 * mx_quantize_q8_1s.  Q4_K folds the min term with s0 + s1 (one more fp32 rounding than the
 * block_q8_1x form's d*float(sum32)).  The Q6_K form has no counterpart in the reference: its
 * per-16 sums are exactly s0 / s1, so it is bit-identical to mx_gemv_q6_K_q8_batched.  */
int mx_gemv_q4_K_q8s_batched(mx_stream_t s, const void* x_q8s, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q6_K_q8s_batched(mx_stream_t s, const void* x_q8s, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q6_K_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q8_0_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q8_0_soa_q8_batched(mx_stream_t s, const void* x_q8, const int8_t* qs_W, const uint16_t* d_W,
                                uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
/* Caller-workspace forms of the batched GEMVs (no counterpart in the reference): identical results, but the split-K
 * partial sums go to `ws` (16-byte aligned device memory of at least mx_gemv_batched_ws_bytes(K, N, T) bytes, which
 * is 0 for shapes that never split), so launches on different streams can overlap.  A workspace that is too small
 * is MX_ERR_WORKSPACE; nothing is launched.  */
int mx_gemv_batched_ws_bytes(uint32_t K, uint32_t N, uint32_t T, uint64_t* bytes);
int mx_gemv_q4_K_q8_batched_ws(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T,
                               void* ws, uint64_t ws_bytes);
int mx_gemv_q6_K_q8_batched_ws(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T,
                               void* ws, uint64_t ws_bytes);
int mx_gemv_q8_0_q8_batched_ws(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T,
                               void* ws, uint64_t ws_bytes);
int mx_gemv_q8_0_soa_q8_batched_ws(mx_stream_t s, const void* x_q8, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y,
                                   uint32_t K, uint32_t N, uint32_t T, void* ws, uint64_t ws_bytes);
/* Fused gate + up for the other int-dot formats: y_a = W_a . x, y_b = W_b . x in one launch, both matrices [N, K].
 * No counterpart of these names in the reference, which fuses gate/up this way for MXFP4 (gemv_mxfp4_soa_q8_x2,
 * include/ie/ops.hpp:503-513) and for Q4_K with fp16 activations (gemv_q4_K_dual_ffn, src/ops/gemv_q4k.cpp:603-612).
 * Each output is bit-identical to the single-matrix entry point's.  */
int mx_gemv_q8_0_soa_q8_x2(mx_stream_t s, const void* x_q8, const int8_t* a_qs, const uint16_t* a_d, const int8_t* b_qs,
                           const uint16_t* b_d, uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N);
int mx_gemv_q4_K_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b,
                       uint32_t K, uint32_t N);
int mx_gemv_q6_K_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b,
                       uint32_t K, uint32_t N);
int mx_gemv_q8_0_q8_x2(mx_stream_t s, const void* x_q8, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b,
                       uint32_t K, uint32_t N);

/* Decode FFN forms (T = 1), no counterpart in the reference, which launches gemv, gemv, swiglu and quantize_q8_1
 * separately (src/model/dense_dispatch.hpp:562-754, src/ops/elementwise.cpp:449-466).
 * *_x2_silu: h[n] = half(silu(half(g[n])) * half(u[n])) with g, u the two GEMVs on the same activation row, the
 *   bits of mx_gemv_*_q8_x2 followed by the fp16 output of mx_swiglu_q8.  x is the q8 row (block_q8_1x,
 *   x_is_f16 = 0) or the fp16 row (x_is_f16 = 1: quantized while it is staged, the values of mx_quantize_q8_1,
 *   16-byte aligned).
 * *_f16q8: y = W . q8(x) on an fp16 activation row quantized while it is staged: the bits of mx_quantize_q8_1
 *   followed by mx_gemv_*_q8.  K up to one LDS tile (32,768 elements for Q6_K, more for the other formats).  */
int mx_gemv_q8_0_soa_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const int8_t* g_qs, const uint16_t* g_d,
                             const int8_t* u_qs, const uint16_t* u_d, uint16_t* h, uint32_t K, uint32_t N);
int mx_gemv_q4_K_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h,
                         uint32_t K, uint32_t N);
int mx_gemv_q6_K_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h,
                         uint32_t K, uint32_t N);
int mx_gemv_q8_0_x2_silu(mx_stream_t s, const void* x, int x_is_f16, const void* gate_W, const void* up_W, uint16_t* h,
                         uint32_t K, uint32_t N);
int mx_gemv_q8_0_soa_f16q8(mx_stream_t s, const uint16_t* x_f16, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y,
                           uint32_t K, uint32_t N);
int mx_gemv_q4_K_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q6_K_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0_f16q8(mx_stream_t s, const uint16_t* x_f16, const void* W, uint16_t* y, uint32_t K, uint32_t N);
/* Sibling formats on the same kernels.
 * Q4_0:
 *   gemv_q4_0                 include/ie/ops.hpp:525-529, src/ops/gemv_q4_0.cpp:54-120   fp16 activations, GGUF blocks
 *   gemv_q4_0_soa_q8          include/ie/ops.hpp:573-576, src/ops/gemv_q4_0.cpp:194-270  planes q4_qs[n*(K/2)+16b+j], q4_d[n*(K/32)+b]
 *   gemv_q4_0_soa_q8_batched  include/ie/ops.hpp:597-601  (T <= 16 here; the reference stops at 8)
 *   gemv_q4_0_soa_q8_multi    include/ie/ops.hpp:577-592: up to 3 banks of different N sharing x_q8, one launch;
 *                             qs / d / y / N are HOST arrays of n_banks entries (device pointers, row counts)
 *   mx_gemv_q4_0_q8_batched   int-dot over the GGUF blocks themselves (no counterpart: the reference repacks first)
 *   fold: acc += d * (d8 * idot - 8 * s), K % 32 == 0.
 * Q5_K (no GEMV in the reference, which dequantizes Q5_K tensors and runs the dense GEMM; include/ie/dequant.hpp:81-86):
 *   the Q4_K kernels with the fifth bit from qh; K % 256 == 0, W 16-byte aligned.  */
int mx_gemv_q4_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q4_0_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q4_0_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q4_qs, const uint16_t* q4_d, uint16_t* y, uint32_t K,
                        uint32_t N);
int mx_gemv_q4_0_soa_q8_batched(mx_stream_t s, const void* x_q8, const uint8_t* q4_qs, const uint16_t* q4_d, uint16_t* y,
                                uint32_t K, uint32_t N, uint32_t T);
int mx_gemv_q4_0_soa_q8_multi(mx_stream_t s, const void* x_q8, const uint8_t* const* qs, const uint16_t* const* d,
                              uint16_t* const* y, const uint32_t* N, int n_banks, uint32_t K);
int mx_gemv_q5_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q5_K_q8(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q5_K_q8_batched(mx_stream_t s, const void* x_q8, const void* W, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
/* Int-dot GEMV over the repacked K-quant layouts (written by the mx_repack_* host functions below):
 *   gemv_q4_K_reorder_q8     include/ie/ops.hpp:322-326, src/ops/gemv_q8dot.cpp:152-256   three-region streams
 *   gemv_q4_soa_q8           include/ie/ops.hpp:444-451, src/ops/gemv_q4_soa.cpp:160-312  natural-order planes
 *   gemv_q6_soa_q8(_batched) include/ie/ops.hpp:402-419, src/ops/gemv_q6_soa.cpp:137-407  natural-order bit planes
 * Same products and fold as the AoS kernels; planes 16-byte aligned.  */
int mx_gemv_q4_K_reorder_q8(mx_stream_t s, const void* x_q8, const void* W_reorder, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q4_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q4_q, const int8_t* q4_sc, const int8_t* q4_mn,
                      const uint16_t* q4_d, const uint16_t* q4_dmin, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q6_soa_q8(mx_stream_t s, const void* x_q8, const uint8_t* q6_lo, const uint8_t* q6_hi, const int8_t* q6_sc,
                      const uint16_t* q6_d, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q6_soa_q8_batched(mx_stream_t s, const void* x_q8, const uint8_t* q6_lo, const uint8_t* q6_hi,
                              const int8_t* q6_sc, const uint16_t* q6_d, uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
/* Two plane sets (gate and up of one FFN) against one q8 row in one launch; no counterpart in the reference (the fused
 * gate + up form of mx_gemv_q6_K_q8_x2 for the planes of repack_q6_K_to_soa).  */
int mx_gemv_q6_soa_q8_x2(mx_stream_t s, const void* x_q8, const uint8_t* a_lo, const uint8_t* a_hi, const int8_t* a_sc,
                         const uint16_t* a_d, const uint8_t* b_lo, const uint8_t* b_hi, const int8_t* b_sc, const uint16_t* b_d,
                         uint16_t* y_a, uint16_t* y_b, uint32_t K, uint32_t N);
int mx_gemv_mxfp4_soa_q8_batched(mx_stream_t s, const void* x_q8, const uint8_t* qs_plane, const uint8_t* e_plane,
                                 uint16_t* y, uint32_t K, uint32_t N, uint32_t T);
/* fp32-output twins of the T = 1 int-dot kernels (no reference counterpart; for
 * callers that keep fp32 activations end to end).  */
int mx_gemv_q4_K_q8_f32(mx_stream_t s, const void* x_q8, const void* W, float* y, uint32_t K, uint32_t N);
int mx_gemv_q6_K_q8_f32(mx_stream_t s, const void* x_q8, const void* W, float* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0_q8_f32(mx_stream_t s, const void* x_q8, const void* W, float* y, uint32_t K, uint32_t N);

/* ---------------------------------------------------------------- decode GEMV, float activations
 * gemv_q4_K           include/ie/ops.hpp:468-472, src/ops/gemv_q4k.cpp:55-149
 * gemv_q6_K           include/ie/ops.hpp (gemv_q6_K), src/ops/gemv_q6k.cpp:591-633
 * gemv_mxfp4_soa_f16  include/ie/ops.hpp:493-497, src/ops/gemv_mxfp4.cpp:257-305
 * A fp16 [K], y fp16 [N]; `_f32`: fp32 A, fp32 y (the shape of BASELINE config 1).  */
int mx_gemv_q4_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q6_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t K, uint32_t N);
int mx_gemv_mxfp4_soa_f16(mx_stream_t s, const uint16_t* A, const uint8_t* qs_plane, const uint8_t* e_plane,
                          uint16_t* y, uint32_t K, uint32_t N);
/* Launch-count fusions of the W4A16 GEMV (same inner loop):
 *   gemv_q4_K_dual (_dual_ssm, _dual_ffn)  src/ops/gemv_q4k.cpp:170-275,594-612: two matrices of the same
 *     shape against one activation vector, y_a = W_a . A, y_b = W_b . A
 *   gemv_q4_K_down_accum                    include/ie/ops.hpp:827-831, src/ops/gemv_q4k.cpp:398-472:
 *     y[n] = half(float(y[n]) + float(sh_g[0]) * (W . A)[n])  */
int mx_gemv_q4_K_dual(mx_stream_t s, const uint16_t* A, const void* W_a, const void* W_b, uint16_t* y_a, uint16_t* y_b,
                      uint32_t K, uint32_t N);
int mx_gemv_q4_K_down_accum(mx_stream_t s, const uint16_t* A, const void* W, const uint16_t* sh_g, uint16_t* y, uint32_t K,
                            uint32_t N);
/*   gemv_q4_K_shexp_gate_up                 include/ie/ops.hpp:807-813, src/ops/gemv_q4k.cpp:288-395:
 *     y_h[n] = half(silu(W_gate . A)[n] * (W_up . A)[n]) and, from one extra workgroup,
 *     sh_g_out[0] = half(sigmoid(sum_k A[k] * W_shg[k]))
 *   gemv_q4_K_dual_ssm_gbeta                include/ie/ops.hpp:819-826, src/ops/gemv_q4k.cpp:480-590:
 *     a = float(half(W_alpha . A)), b = float(half(W_beta . A));
 *     g_out[n] = A_log[n] * softplus(a[n] + dt_bias[n]), beta_out[n] = sigmoid(b[n])   (any N)  */
int mx_gemv_q4_K_shexp_gate_up(mx_stream_t s, const uint16_t* A, const void* W_gate, const void* W_up, const float* W_shg,
                               uint16_t* y_h, uint16_t* sh_g_out, uint32_t K, uint32_t N);
int mx_gemv_q4_K_dual_ssm_gbeta(mx_stream_t s, const uint16_t* A, const void* W_alpha, const void* W_beta, const float* A_log,
                                const float* dt_bias, float* g_out, float* beta_out, uint32_t K, uint32_t N);
int mx_gemv_q4_K_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N);
int mx_gemv_q6_K_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N);
int mx_gemv_q8_0_f32(mx_stream_t s, const float* A, const void* W, float* y, uint32_t K, uint32_t N);

/* ---------------------------------------------------------------- prefill quant-GEMM (matrix cores)
 * y[M,N] = A[M,K] . half(deq(W))[N,K]^T, fp16 x fp16 MFMA, fp32 accumulate, fp16 out; any M.
 * Replaces the 16-row XMX launches and the dequant + dense-GEMM route:
 *   gemm_q4_K_xmx / gemm_q4_K_esimd / gemm_q4_K  include/ie/ops.hpp:607-611, src/ops/gemm_q4k_xmx.cpp:115-234
 *   dequant_q4_K_to_Bt + gemm_fp16(_onednn)      src/model/dense_dispatch.hpp:658-693
 * K % 256 == 0 (Q4_K), K % 128 == 0 (Q8_0 planes); A and W 16-byte aligned.
 * mx_gemm_q8_0_soa takes the SoA planes of gemv_q8_0_soa_q8 (the reference runs Q8_0 prefill
 * as dequant_q8_0_soa_to_Bt + gemm_fp16, src/model/qwen35_dense.cpp:811-831).
 * A launch whose 128-token tiles would cover at most half of the CUs (a short batch against a narrow
 * matrix) and whose K is at least 2048 is cut into 2..8 K slices; their fp32 partial sums go through a
 * 32 MB per-device scratch array owned by the library (a file-scope device array resolved with hipGetSymbolAddress,
 * never allocated; slices * M * N <= 8 Mi floats, fewer slices beyond that) and are added in slice
 * order by a second small launch: two such calls that overlap on one device race on it, as the
 * reference's static per-device scratch buffers would (src/model/dense_dispatch.hpp:547-560).  The *_ws forms
 * below keep the partial sums in the caller's workspace instead.  */
int mx_gemm_q4_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
int mx_gemm_q8_0_soa(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M,
                     uint32_t K, uint32_t N);
/* Q6_K and AoS Q8_0 weights through the same kernel:
 *   gemm_q6_K_xmx / gemm_q6_K   include/ie/ops.hpp (gemm_q6_K_xmx), src/ops/gemm_q4k_xmx.cpp:284-387, src/ops/gemv_q6k.cpp:655-748
 *   dequant_q6_K_to_Bt / dequant_q8_0_to_Bt + gemm_fp16   src/ops/dequant_kernels.cpp:392-431,611-632
 * K % 256 == 0 (Q6_K), K % 128 == 0 (Q8_0); W is the GGUF block stream, 2-byte aligned.  */
int mx_gemm_q6_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
int mx_gemm_q8_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
/* Caller-workspace forms (no counterpart in the reference): same results; K-sliced launches keep their partial sums
 * in `ws` (16-byte aligned device memory), so launches on different streams can overlap.  mx_gemm_ws_bytes gives the
 * size that allows every slice the launch would like (0: the shape is never sliced); a smaller workspace, NULL / 0
 * included, is legal and means fewer slices or none.  */
int mx_gemm_ws_bytes(uint32_t M, uint32_t K, uint32_t N, uint64_t* bytes);
int mx_gemm_q4_K_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws,
                    uint64_t ws_bytes);
int mx_gemm_q6_K_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws,
                    uint64_t ws_bytes);
int mx_gemm_q8_0_ws(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N, void* ws,
                    uint64_t ws_bytes);
int mx_gemm_q8_0_soa_ws(mx_stream_t s, const uint16_t* A, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M,
                        uint32_t K, uint32_t N, void* ws, uint64_t ws_bytes);
/* Q4_0 weights through the same kernel: gemm_q4_0 / gemm_q4_0_xmx  include/ie/ops.hpp:530-534, src/ops/gemv_q4_0.cpp,
 * src/ops/gemm_q4k_xmx.cpp:418-522; K % 128 == 0, W 2-byte aligned.  */
int mx_gemm_q4_0(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
/* Plain dense GEMM for the dequant-to-Bt route (formats without a fused quant-GEMM: Q5_K, MXFP4):
 *   gemm_fp16          include/ie/ops.hpp:275-286, src/ops/gemm_fp16.cpp:46-178    C fp32 [M,N]
 *   gemm_fp16_onednn   include/ie/ops.hpp:460-465, src/ops/gemm_onednn.cpp:75-111  y fp16 [M,N]
 * A fp16 [M,K] row-major, B fp16 [K,N] row-major (the Bt the mx_dequant_*_to_Bt functions write),
 * fp32 accumulation.  Argument order (M, N, K) as in the reference.  mx_gemm_fp16 is a hand-tiled matrix-core kernel
 * (both tiles through LDS, B transposed on the way; ragged M, N, K into an exactly sized C); mx_gemm_fp16_onednn runs the
 * vendor library (rocBLAS' gemm_ex, as the reference runs oneDNN), loaded on first use: MX_ERR_UNSUPPORTED where it is
 * not installed.  */
int mx_gemm_fp16(mx_stream_t s, const uint16_t* A, const uint16_t* B, float* C, uint32_t M, uint32_t N, uint32_t K);
int mx_gemm_fp16_onednn(mx_stream_t s, const uint16_t* A, const uint16_t* B, uint16_t* y, uint32_t M, uint32_t N, uint32_t K);
/* Expert-grouped GEMM over expert-sorted fp16 rows (Q8_0 SoA expert banks): the matrix-core
 * form of moe_prefill_gate_up_silu_q8 / moe_prefill_down_q8 (include/ie/moe_q8.hpp:51-72) for
 * fp16 activations — same arguments except that the activation rows are fp16 instead of
 * block_q8_1x and the host passes total_rows = expert_offsets[E] (known from the packing).
 *   h_packed[row, n]   = half(silu(gate_e . x_row) * (up_e . x_row))
 *   out_packed[row, n] = half(sorted_w[row] * (down_e . h_row))
 * H % 128 == 0 and E_ffn % 128 == 0.  */
int mx_moe_gemm_gate_up_silu_q8(mx_stream_t s, const uint16_t* x_packed, const int8_t* g_qs, const uint16_t* g_d,
                                const int8_t* u_qs, const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride,
                                const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                                uint32_t total_rows);
int mx_moe_gemm_down_q8(mx_stream_t s, const uint16_t* h_packed, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                        uint64_t d_stride, const uint32_t* expert_offsets, const uint16_t* sorted_w, uint16_t* out_packed,
                        uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows);
/* Gather forms of the grouped gate/up GEMMs: moe_gather_rows (include/ie/ops.hpp, src/ops/moe.cpp:423-446) folded into the
 * load of the activation rows.  x is the unsorted [n_tokens, H] fp16 matrix and sorted_idx[r] (device, total_rows
 * entries, each in [0, n_tokens)) the source row of sorted row r, as build_moe_packing returns it; no gathered copy
 * is written or read.  Same results as mx_moe_gather_rows followed by the entry of the same name, bit for bit.
 * n_tokens * H * 2 < 2^32.  */
int mx_moe_gemm_gate_up_silu_q8_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens,
                                       const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs, const uint16_t* u_d,
                                       uint64_t qs_stride, uint64_t d_stride, const uint32_t* expert_offsets, uint16_t* h_packed,
                                       uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows);
int mx_moe_gemm_gate_up_silu_q4k_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens,
                                        const void* gate_W, const void* up_W, const uint32_t* expert_offsets, uint16_t* h_packed,
                                        uint32_t E, uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, int soa,
                                        uint32_t total_rows);
int mx_moe_gemm_gate_up_oai_mxfp4_gather(mx_stream_t s, const uint16_t* x, const int32_t* sorted_idx, uint32_t n_tokens,
                                         const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs, const uint8_t* u_e,
                                         uint64_t qs_stride, uint64_t e_stride, const float* gate_bias, const float* up_bias,
                                         const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H,
                                         uint32_t E_ffn, uint32_t total_rows, float alpha, float limit);
/* The same for AoS K-quant expert banks (expert e at W + e*expert_stride_bytes, include/ie/ops.hpp:1027-1029):
 *   moe_prefill_gate_up_silu_q4k (fp16 x_packed) / _q4k_xmx   include/ie/ops.hpp:922-929, src/ops/moe_fused.cpp:727-901,
 *                                                             src/ops/gemm_q4k_xmx.cpp:662-847
 *   moe_prefill_down_packed_q4k / _q6k (and _v2)              include/ie/ops.hpp:968-983, src/ops/moe_fused.cpp:1090-1572
 * sorted_w may be NULL: the rows are then written unweighted, as the reference's packed down
 * kernels do (the weights are applied by moe_prefill_reduce); with sorted_w the product
 * half(sorted_w[row] * acc) is folded into the store.  H % 256 == 0 and E_ffn % 256 == 0.
 * soa != 0 as in the reference (include/ie/ops.hpp:918,927,997,1005): every expert region holds its blocks as
 * per-field streams (mx_repack_moe_q4k_soa / _q6k_soa, include/ie/quant_soa.hpp:33-51); total_rows follows it.  */
int mx_moe_gemm_gate_up_silu_q4k(mx_stream_t s, const uint16_t* x_packed, const void* gate_W, const void* up_W,
                                 const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                                 uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
int mx_moe_gemm_down_q4k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets,
                         const uint16_t* sorted_w, uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                         uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
int mx_moe_gemm_down_q6k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets,
                         const uint16_t* sorted_w, uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn,
                         uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
/* MXFP4 planes and Q5_K blocks through the fused matrix-core kernel.  The reference has no fused form for them: it
 * dequantizes to a [K, N] fp16 matrix and runs a plain GEMM (dequant_mxfp4_soa_to_Bt + gemm_fp16, src/ops/gemv_mxfp4.cpp:
 * 316-341, src/model/gptoss.cpp:389-392; dequant_q5_K_to_Bt, include/ie/dequant.hpp:81-86); these compute the same
 * y = A . half(deq(W))^T without writing that matrix.  mx_gemm_mxfp4_soa takes the planes of gemv_mxfp4_soa_q8
 * (include/ie/ops.hpp, gemv_mxfp4.cpp:120-141), K % 64 == 0 (gpt-oss: K = 2880); mx_gemm_q5_K the GGUF block stream
 * (176-byte blocks, 16-byte aligned), K % 256 == 0.  The grouped forms are the fp16-row counterparts of
 * mx_moe_grouped_gate_up_oai_mxfp4 / mx_moe_grouped_down_mxfp4 (same arithmetic after the matrix product:
 * half(swiglu_oai(half(g + bias), half(u + bias))) and half(half(acc) + bias); biases may be NULL).  */
int mx_gemm_q5_K(mx_stream_t s, const uint16_t* A, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
int mx_gemm_mxfp4_soa(mx_stream_t s, const uint16_t* A, const uint8_t* qs_W, const uint8_t* e_W, uint16_t* y, uint32_t M,
                      uint32_t K, uint32_t N);
int mx_moe_gemm_gate_up_oai_mxfp4(mx_stream_t s, const uint16_t* x_packed, const uint8_t* g_qs, const uint8_t* g_e,
                                  const uint8_t* u_qs, const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride,
                                  const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets,
                                  uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha,
                                  float limit);
int mx_moe_gemm_down_mxfp4(mx_stream_t s, const uint16_t* h_packed, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                           uint64_t e_stride, const float* down_bias, const uint32_t* expert_offsets, uint16_t* out_packed,
                           uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows);
/* Q4_0 expert banks (Gemma-4 MoE) and the dense W4A8 GEMM; plain projections, no epilogue:
 *   moe_prefill_proj_q4_0_q8      include/ie/ops.hpp:166-177   block_q8_1s rows, GGUF blocks, expert e at W + e*expert_stride_bytes
 *   moe_prefill_proj_q4_0_soa_q8  include/ie/ops.hpp:179-190   block_q8_1s rows, planes: qs_bank + e*qs_stride bytes, d_bank + e*d_stride entries
 *   moe_prefill_proj_q4_0_xmx     include/ie/ops.hpp:192-204   fp16 rows, matrix cores (K % 128 == 0 here; the reference needs K % 256, N % 64)
 *   gemm_q4_0_q8                  include/ie/ops.hpp:538-548   y[M,N] = q8(x)[M,K] . W, any M and any K % 32 == 0, int-dot
 * out_packed[row, n] = half(acc); rows of expert e are [expert_offsets[e], expert_offsets[e+1]); total_rows = expert_offsets[E].  */
int mx_moe_prefill_proj_q4_0_q8(mx_stream_t s, const void* xq8s_packed, const void* W_q4_0, const uint32_t* expert_offsets,
                                uint16_t* out_packed, uint32_t E, uint32_t K, uint32_t N, uint64_t expert_stride_bytes,
                                uint32_t total_rows);
int mx_moe_prefill_proj_q4_0_soa_q8(mx_stream_t s, const void* xq8s_packed, const uint8_t* qs_bank, const uint16_t* d_bank,
                                    const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E, uint32_t K, uint32_t N,
                                    uint64_t qs_stride, uint64_t d_stride, uint32_t total_rows);
int mx_moe_prefill_proj_q4_0_xmx(mx_stream_t s, const uint16_t* x_fp16, const void* W_q4_0, const uint32_t* expert_offsets,
                                 uint16_t* out_packed, uint32_t E, uint32_t K, uint32_t N, uint64_t expert_stride_bytes,
                                 uint32_t total_rows);
int mx_gemm_q4_0_q8(mx_stream_t s, const void* xq8s_packed, const void* W_q4_0, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
/* The dense int-dot GEMM for the other formats (no counterpart in the reference, whose gemm_q4_0_q8 exists for Q4_0
 * only): y[M,N] = q8(x)[M,K] . W[N,K]^T over block_q8_1s rows [M, K/32] (mx_quantize_q8_1s), any M; int8 matrix cores,
 * one instruction per 32-element block, fp32 fold per block (the q8 chain of mx_gemv_*_q8, row for row).  */
int mx_gemm_q4_K_q8(mx_stream_t s, const void* xq8s_packed, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
int mx_gemm_q6_K_q8(mx_stream_t s, const void* xq8s_packed, const void* W, uint16_t* y, uint32_t M, uint32_t K, uint32_t N);
int mx_gemm_q8_0_soa_q8(mx_stream_t s, const void* xq8s_packed, const int8_t* qs_W, const uint16_t* d_W, uint16_t* y, uint32_t M,
                        uint32_t K, uint32_t N);
/* Accumulate form of the down projection (the reference's first prefill path), same matrix-core kernel
 * with an atomic fp32 epilogue:
 *   moe_prefill_down_q4k / _q6k       include/ie/ops.hpp:930-954, src/ops/moe_fused.cpp:937-1085
 *     y_fp32[sorted_token_idx[row], n] += float(sorted_token_w[row]) * (down_e . h_row)[n]; the caller zeroes
 *     y_fp32; the order of the additions (and so the last bits) is not fixed, as in the reference
 *   moe_prefill_merge_fp32_to_fp16    include/ie/ops.hpp:956-962, src/ops/moe_fused.cpp:1956-1972
 *     y_fp16[i] = half(float(y_fp16[i]) + y_fp32[i])  */
int mx_moe_prefill_down_q4k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets,
                            const int32_t* sorted_token_idx, const uint16_t* sorted_token_w, float* y_fp32, uint32_t E,
                            uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, uint32_t total_rows);
int mx_moe_prefill_down_q6k(mx_stream_t s, const uint16_t* h_packed, const void* down_W, const uint32_t* expert_offsets,
                            const int32_t* sorted_token_idx, const uint16_t* sorted_token_w, float* y_fp32, uint32_t E,
                            uint32_t H, uint32_t E_ffn, uint64_t expert_stride_bytes, uint32_t total_rows);
int mx_moe_prefill_merge_fp32_to_fp16(mx_stream_t s, const float* y_fp32, uint16_t* y_fp16, uint64_t n);

/* ---------------------------------------------------------------- MoE, expert-indexed GEMV
 * Q8_0-expert decode kernels (device-resident routing: the expert of token slot
 * tk = t*K + k is read from topk_idx[tk]; no host round trip):
 *   moe_gate_up_silu_q8  include/ie/moe_q8.hpp:17-23, src/ops/moe_q8.cpp:45-100
 *     h_out[tk, n] = half(silu(gate_e . x_t) * (up_e . x_t)); x_q8 = T rows of H/32 blocks
 *   moe_down_q8          include/ie/moe_q8.hpp:25-31, src/ops/moe_q8.cpp:102-147
 *     y_packed[tk, n] = half(topk_w[tk] * (down_e . h_tk)); h_q8 = T*K rows of E_ffn/32 blocks
 *   moe_reduce_q8        include/ie/moe_q8.hpp:33-35, src/ops/moe_q8.cpp:149-158
 * Expert e of a SoA bank: qs + e*qs_stride (bytes), d + e*d_stride (fp16 entries).  */
int mx_moe_gate_up_silu_q8(mx_stream_t s, const void* x_q8, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                           const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const int32_t* topk_idx,
                           uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H, uint32_t E_ffn);
int mx_moe_down_q8(mx_stream_t s, const void* h_q8, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                   uint64_t d_stride, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T,
                   uint32_t K, uint32_t E_ffn, uint32_t H);
int mx_moe_reduce_q8(mx_stream_t s, const uint16_t* y_packed, uint16_t* y, uint32_t T, uint32_t K, uint32_t H);
/* The same two launches with the number of experts in the bank as a last argument (no counterpart in the reference,
 * whose signatures carry no expert count): a slot whose id lies outside [0, n_experts) is skipped, its output row is
 * left as it was.  Through the reference signatures above only negative ids can be recognised; a positive id past
 * the bank would read past it.  */
int mx_moe_gate_up_silu_q8_n(mx_stream_t s, const void* x_q8, const int8_t* g_qs, const uint16_t* g_d, const int8_t* u_qs,
                             const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride, const int32_t* topk_idx,
                             uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H, uint32_t E_ffn, uint32_t n_experts);
int mx_moe_down_q8_n(mx_stream_t s, const void* h_q8, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                     uint64_t d_stride, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T,
                     uint32_t K, uint32_t E_ffn, uint32_t H, uint32_t n_experts);
/* K-quant expert-major expert banks with fp16 activations, decode — the reference's fused
 * Q4_K / Q6_K expert kernels; fp32 fold acc += (d*sc)*sum(a*q) - (dmin*m)*sum(a):
 *   moe_decode_gate_up_silu_q4k  include/ie/ops.hpp:1034-1041, src/ops/moe_fused.cpp:82-211
 *     h_out[t*K_top + k, n] = half(silu(gate_e . x_t) * (up_e . x_t)),  e = topk_idx[t*K_top + k]
 *   moe_decode_down_q4k / _q6k   include/ie/ops.hpp:1078-1095, src/ops/moe_fused.cpp:224-330,352-522
 *     y_out[t, n] = half(sum_k topk_w[t*K_top + k] * (down_e . h[t*K_top + k])); written, not accumulated
 * The reference signatures are single-token; T (last argument) generalises them to T tokens per
 * launch, T = 1 being the reference call.  H % 256 == 0, E_ffn % 256 == 0.  soa = 0: every expert
 * region is an array of GGUF blocks; soa != 0: every region holds the same blocks as per-field
 * streams (q4k_wview / q6k_wview<true>, include/ie/quant_soa.hpp:33-125), written by
 * mx_repack_moe_q4k_soa_host / mx_repack_moe_q6k_soa_host.  */
int mx_moe_decode_gate_up_silu_q4k(mx_stream_t s, const uint16_t* x, const void* gate_W, const void* up_W,
                                   const int32_t* topk_idx, uint16_t* h_out, uint32_t H, uint32_t E_ffn, uint32_t K_top,
                                   uint64_t expert_stride_bytes, int soa, uint32_t T);
int mx_moe_decode_down_q4k(mx_stream_t s, const uint16_t* h, const void* down_W, const int32_t* topk_idx,
                           const uint16_t* topk_w, uint16_t* y_out, uint32_t H, uint32_t E_ffn, uint32_t K_top,
                           uint64_t expert_stride_bytes, int soa, uint32_t T);
int mx_moe_decode_down_q6k(mx_stream_t s, const uint16_t* h, const void* down_W, const int32_t* topk_idx,
                           const uint16_t* topk_w, uint16_t* y_out, uint32_t H, uint32_t E_ffn, uint32_t K_top,
                           uint64_t expert_stride_bytes, int soa, uint32_t T);
/* Int-dot grouped kernels for K-quant expert banks (soa as above), expert-sorted rows partitioned by
 * expert_offsets[E+1] (total_rows = expert_offsets[E], known to the host from the packing):
 * Every entry of the family takes block_q8_1s rows (48 B {d, s0, s1, pad, qs[32]} from mx_quantize_q8_1s, 16-byte
 * aligned): the reference kernels read the header as one float4 and fold the min term on s0 + s1
 * (src/ops/moe_fused.cpp:559-566,672-687; the "block_q8_1x" of the comment above that kernel is stale).
 *   moe_prefill_gate_up_silu_q4k_q8       include/ie/ops.hpp:912-919, src/ops/moe_fused.cpp:546-725
 *   moe_prefill_gate_up_silu_q6k_q8       src/ops/moe_qwen3.cpp:330-551 (include/ie/moe_qwen3.hpp)
 *   moe_prefill_down_packed_q4k_q8/_q6k_q8, moe_prefill_down_q{4,6}k_q8_gen
 *                                         include/ie/ops.hpp:993-1006, src/ops/moe_fused.cpp:1603-1924
 *     out_packed[row, n] = half(down_e . h_row), unweighted (moe_prefill_reduce applies the weights);
 *     any E_ffn % 256 == 0 (the reference's register-resident variant needs E_ffn == 512).
 * total_rows is the one argument the reference signatures do not have.  It only picks the launch shape (rows staged
 * per workgroup and row blocks per workgroup are sized for total_rows / E rows per expert) and never changes a
 * result: the rows that are computed are those expert_offsets names.  0xFFFFFFFF means "not known" and is always
 * legal (the launch is then sized for large, uneven experts); a wrapper with the reference's exact argument list
 * passes that value.  The same holds for every other total_rows argument of this header.  */
int mx_moe_prefill_gate_up_silu_q4k_q8(mx_stream_t s, const void* xq8s_packed, const void* gate_W, const void* up_W,
                                       const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H,
                                       uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
int mx_moe_prefill_gate_up_silu_q6k_q8(mx_stream_t s, const void* xq8s_packed, const void* gate_W, const void* up_W,
                                       const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H,
                                       uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
int mx_moe_prefill_down_packed_q4k_q8(mx_stream_t s, const void* hq8s_packed, const void* down_W,
                                      const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E, uint32_t H,
                                      uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
int mx_moe_prefill_down_packed_q6k_q8(mx_stream_t s, const void* hq8s_packed, const void* down_W,
                                      const uint32_t* expert_offsets, uint16_t* out_packed, uint32_t E, uint32_t H,
                                      uint32_t E_ffn, uint64_t expert_stride_bytes, int soa, uint32_t total_rows);
/* Expert-grouped form: activation rows are expert-sorted and partitioned by
 * expert_offsets[E+1]; each expert's weights are streamed once per tile of rows;
 * experts without rows cost nothing (src/ops/moe_q8.cpp:211).
 *   moe_prefill_gate_up_silu_q8  include/ie/moe_q8.hpp:51-58, src/ops/moe_q8.cpp:185-275
 *   moe_prefill_down_q8          include/ie/moe_q8.hpp:65-72, src/ops/moe_q8.cpp:277-366
 *     out_packed[row, n] = half(sorted_w[row] * acc)
 *   moe_prefill_reduce_sum       include/ie/moe_q8.hpp:77-80, src/ops/moe_q8.cpp:368-384
 *   moe_prefill_reduce           include/ie/ops.hpp:1008-1017, src/ops/moe_fused.cpp:1927-1954
 *     y[t] += sum_k w[row] * out_packed[row], row = tk_to_packed[t*K+k]  (accumulates: caller zeroes y)
 *   moe_gather_rows              src/ops/moe.cpp:262-282  */
int mx_moe_prefill_gate_up_silu_q8(mx_stream_t s, const void* xq8_packed, const int8_t* g_qs, const uint16_t* g_d,
                                   const int8_t* u_qs, const uint16_t* u_d, uint64_t qs_stride, uint64_t d_stride,
                                   const uint32_t* expert_offsets, uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn);
int mx_moe_prefill_down_q8(mx_stream_t s, const void* hq8_packed, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                           uint64_t d_stride, const uint32_t* expert_offsets, const uint16_t* sorted_w, uint16_t* out_packed,
                           uint32_t E, uint32_t H, uint32_t E_ffn);
int mx_moe_prefill_reduce_sum(mx_stream_t s, const uint16_t* out_packed, const uint32_t* tk_to_packed, uint16_t* y, uint32_t T,
                              uint32_t K, uint32_t H);
int mx_moe_prefill_reduce(mx_stream_t s, const uint16_t* out_packed, const uint32_t* tk_to_packed, const uint16_t* weights_packed,
                          uint16_t* y, uint32_t T, uint32_t K_top, uint32_t H);
int mx_moe_gather_rows(mx_stream_t s, const uint16_t* x, const int32_t* indices, uint16_t* y_packed, uint32_t n_rows,
                       uint32_t hidden);
/* moe_scatter_add  include/ie/ops.hpp:1053-1064, src/ops/moe.cpp:284-313
 *   y[indices[i], :] = half(float(y[indices[i], :]) + float(x_packed[i, :]) * float(weights[i]));
 *   plain read-modify-write as in the reference, so the rows one call names must be distinct. */
int mx_moe_scatter_add(mx_stream_t s, const uint16_t* x_packed, const int32_t* indices, const uint16_t* weights, uint16_t* y,
                       uint32_t n_tok, uint32_t hidden);
/* MXFP4-expert (gpt-oss) kernels.  The reference runs this layer as a host loop
 * over experts of gemv_mxfp4_soa_q8 / add_bias / swiglu_oai launches
 * (src/model/gptoss.cpp:366-420); these entry points are that loop moved onto the
 * device, with the same rounding points: h = half(swiglu_oai(half(gate.x + bg),
 * half(up.x + bu))), out = half(half(down.h) + bd).  Biases fp32 [E][N], may be NULL.
 * Decode form reads topk_idx; grouped form takes expert-sorted rows +
 * expert_offsets (total_rows = expert_offsets[E], known to the host from the packing).
 * Exponent bytes: the grouped entry points with H (gate/up) or E_ffn (down) of 256 and more hand the stored E8M0 byte
 * to the scaled matrix instruction, whose block sum is formed in fp32 before the activation scale is applied.  They
 * agree with the decode kernels and with e8m0_half (include/ie/quant_blocks.hpp:46-54) for exponent bytes 2 .. 240
 * (2^-126 .. 2^112 of the doubled E2M1 value; trained tensors sit near 2^-10); byte 255 is NaN to the instruction (as
 * in the OCP MX definition) where e8m0_half returns 2^127, and beyond 240 a block sum can overflow fp32 before the
 * activation scale brings it back.  */
int mx_moe_gate_up_oai_mxfp4(mx_stream_t s, const void* x_q8, const uint8_t* g_qs, const uint8_t* g_e, const uint8_t* u_qs,
                             const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride, const float* gate_bias,
                             const float* up_bias, const int32_t* topk_idx, uint16_t* h_out, uint32_t T, uint32_t K, uint32_t H,
                             uint32_t E_ffn, uint32_t n_experts, float alpha, float limit);
int mx_moe_down_mxfp4(mx_stream_t s, const void* h_q8, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                      uint64_t e_stride, const float* down_bias, const int32_t* topk_idx, uint16_t* out_packed, uint32_t T,
                      uint32_t K, uint32_t E_ffn, uint32_t H, uint32_t n_experts);
int mx_moe_grouped_gate_up_oai_mxfp4(mx_stream_t s, const void* xq8_packed, const uint8_t* g_qs, const uint8_t* g_e,
                                     const uint8_t* u_qs, const uint8_t* u_e, uint64_t qs_stride, uint64_t e_stride,
                                     const float* gate_bias, const float* up_bias, const uint32_t* expert_offsets,
                                     uint16_t* h_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows, float alpha,
                                     float limit);
int mx_moe_grouped_down_mxfp4(mx_stream_t s, const void* hq8_packed, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                              uint64_t e_stride, const float* down_bias, const uint32_t* expert_offsets, uint16_t* out_packed,
                              uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows);
/* Down projections that take h as fp16 rows and quantize it while staging it (the staged tile is bit-identical to
 * staging mx_quantize_q8_1(h)), so the quantize launch between the two expert stages disappears.  No counterpart in
 * the reference (it launches quantize_q8_1 between swiglu and the down GEMV, src/model/gptoss.cpp:400-412).
 * h rows 16-byte aligned; otherwise the arguments of mx_moe_down_mxfp4 / mx_moe_grouped_down_mxfp4 / mx_moe_down_q8.  */
int mx_moe_down_mxfp4_f16(mx_stream_t s, const uint16_t* h_f16, const uint8_t* d_qs, const uint8_t* d_e, uint64_t qs_stride,
                          uint64_t e_stride, const float* down_bias, const int32_t* topk_idx, uint16_t* out_packed, uint32_t T,
                          uint32_t K, uint32_t E_ffn, uint32_t H, uint32_t n_experts);
int mx_moe_grouped_down_mxfp4_f16(mx_stream_t s, const uint16_t* h_packed_f16, const uint8_t* d_qs, const uint8_t* d_e,
                                  uint64_t qs_stride, uint64_t e_stride, const float* down_bias, const uint32_t* expert_offsets,
                                  uint16_t* out_packed, uint32_t E, uint32_t H, uint32_t E_ffn, uint32_t total_rows);
int mx_moe_down_q8_f16(mx_stream_t s, const uint16_t* h_f16, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                       uint64_t d_stride, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T,
                       uint32_t K, uint32_t E_ffn, uint32_t H);
int mx_moe_down_q8_f16_n(mx_stream_t s, const uint16_t* h_f16, const int8_t* d_qs, const uint16_t* d_d, uint64_t qs_stride,
                         uint64_t d_stride, const int32_t* topk_idx, const uint16_t* topk_w, uint16_t* y_packed, uint32_t T,
                         uint32_t K, uint32_t E_ffn, uint32_t H, uint32_t n_experts);   /* ids outside [0, n_experts) skipped */
/* ---------------------------------------------------------------- MoE routing and packing on the device
 *   moe_router             include/ie/ops.hpp:780-786, src/ops/moe.cpp:22-216
 *     logits = W_gate[E,H] (fp32) . x_t, softmax, top-k, renormalise, ascending expert id; any
 *     E <= 1024, k <= 64 (the reference handles E = 256, k = 8 only).  logits_ws: caller-owned
 *     workspace of n_tokens*n_experts floats (the reference keeps a static per-device buffer).
 *   moe_topk_from_logits   include/ie/ops.hpp:790-793, src/ops/moe.cpp:366-412   (fp16 logits, n_tokens rows)
 *   moe_build_pack_decode  include/ie/ops.hpp:797-802, src/ops/moe.cpp:423-446   (one token)
 *   mx_moe_build_packing_device: the arrays of build_moe_packing (src/model/qwen3moe_pack.cpp:5-31)
 *     for T tokens without leaving the device: stable counting sort of the T*K slots by expert.
 * An exact probability tie goes to the higher expert id, as in the reference.  */
int mx_moe_router(mx_stream_t s, const uint16_t* x, const float* W_gate, int32_t* topk_idx, uint16_t* topk_w,
                  uint32_t n_tokens, uint32_t hidden, uint32_t n_experts, uint32_t k, float* logits_ws);
int mx_moe_topk_from_logits(mx_stream_t s, const uint16_t* logits, int32_t* topk_idx, uint16_t* topk_w, uint32_t E,
                            uint32_t K, uint32_t n_tokens);
int mx_moe_build_pack_decode(mx_stream_t s, const int32_t* topk_idx, const uint16_t* topk_w, uint32_t* expert_offsets,
                             int32_t* sorted_idx, int32_t* tk_to_packed, uint16_t* weights_packed, uint32_t E, uint32_t K);
int mx_moe_build_packing_device(mx_stream_t s, const int32_t* topk_idx, const uint16_t* topk_w, uint32_t T, uint32_t K,
                                uint32_t E, uint32_t* expert_offsets, int32_t* sorted_idx, uint16_t* weights_packed,
                                int32_t* tk_to_packed);

/* ---------------------------------------------------------------- producers of the q8 activation stream
 * Normalisation fused with block_q8_1x emission; the quantizer sees the rounded fp16 outputs, so
 * q8_out equals quantize_q8_1(y) bit for bit.  hidden % 32 == 0.
 *   rms_norm_f32w_q8   include/ie/ops.hpp:51-56, src/ops/elementwise.cpp:136-191
 *     y = half((x * rsqrt(mean(x^2) + eps)) * w), x fp16, w fp32
 *   gated_rms_norm_q8  include/ie/ops.hpp:367-372, src/ops/deltanet.cpp:73-130
 *     y = half((w * (x * r)) * silu(z)), x fp32, z and w fp16  */
int mx_rms_norm_f32w_q8(mx_stream_t s, const uint16_t* x, const float* w, uint16_t* y, void* q8_out, uint32_t n_rows,
                        uint32_t hidden, float eps);
int mx_gated_rms_norm_q8(mx_stream_t s, const float* x, const uint16_t* z, const uint16_t* weight, uint16_t* y,
                         void* q8_out, uint32_t n_rows, uint32_t hidden, float eps);
/* Gated activations with the same fused emitter (no counterpart in the reference, which runs swiglu /
 * swiglu_oai and then quantize_q8_1): y = half(silu(gate) * up) (swiglu, src/ops/elementwise.cpp:449-467)
 * or the clamped gpt-oss form (swiglu_oai, :469-492; alpha 1.702, limit 7.0 there), and q8_out = the
 * block_q8_1x stream of the rounded y, bit-identical to mx_quantize_q8_1(y).  y may be NULL when only
 * the stream is wanted; n % 32 == 0.  */
int mx_swiglu_q8(mx_stream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* y, void* q8_out, uint64_t n);
int mx_swiglu_oai_q8(mx_stream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* y, void* q8_out, uint64_t n, float alpha,
                     float limit);

/* build_moe_packing  src/model/qwen3moe_pack.cpp:5-31 (host pointers): stable counting sort by expert.  */
int mx_build_moe_packing(const int32_t* topk_ids, const float* topk_w, uint32_t T, uint32_t K, uint32_t E,
                         uint32_t* expert_offsets, int32_t* sorted_idx, float* weights_packed, int32_t* tk_to_packed);

/* ---------------------------------------------------------------- host repackers (host pointers)
 * MXFP4 AoS -> SoA planes  src/model/gptoss.cpp:180-208
 * Q8_0  AoS -> SoA planes  src/model/qwen35moe_split.cpp:134-144  */
int mx_repack_mxfp4_to_soa(const void* blocks, uint64_t n_blocks, uint8_t* qs_plane, uint8_t* e_plane);
int mx_repack_q8_0_to_soa(const void* blocks, uint64_t n_blocks, int8_t* qs_plane, uint16_t* d_plane);
/* K-quant repacks (pure bit moves; every weight keeps its value):
 *   repack_q4_K_to_reorder    include/ie/ops.hpp:316-321, src/ops/gemv_q8dot.cpp:134-147
 *     all nb = N*K/256 blocks of a matrix -> qs[128] x nb | scales[12] x nb | {d,dmin}[4] x nb (N*K/256*144 bytes)
 *   repack_moe_q4k_soa_host   include/ie/quant_soa.hpp:127-141   the same split inside each expert region
 *   repack_moe_q6k_soa_host   include/ie/quant_soa.hpp:143-157   ql[128] x nb | qh[64] x nb | scales[16] x nb | d[2] x nb
 *     (src and dst are whole banks of n_experts * nblocks_per_expert blocks and must not alias)
 *   repack_q4_K_to_soa        include/ie/ops.hpp:431-440, src/ops/gemv_q4_soa.cpp:115-151
 *     natural element order per row: q4_q N*K/2 bytes (element k = nibble k&1 of byte k/2), q4_sc / q4_mn N*K/32
 *     unpacked 6-bit scales / mins, q4_d / q4_dmin N*K/256 fp16 bits
 *   repack_q6_K_to_soa        include/ie/ops.hpp:393-399, src/ops/gemv_q6_soa.cpp:71-126
 *     q6_lo N*K/2 (low nibbles), q6_hi N*K/4 (element k = bits 2*(k&3) of byte k/4), q6_sc N*K/16 int8,
 *     q6_d N*K/256 fp16 bits; unlike the reference's, the planes need not be zeroed first  */
/* repack_q4_0_to_soa  include/ie/ops.hpp:571-572, src/ops/gemv_q4_0.cpp:179-192: q4_qs N*K/2 bytes, q4_d N*K/32 fp16 bits */
int mx_repack_q4_0_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q4_qs, uint16_t* q4_d);
int mx_repack_q4_K_to_reorder(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* out);
int mx_repack_moe_q4k_soa_host(const void* src, void* dst, uint32_t n_experts, uint64_t nblocks_per_expert);
int mx_repack_moe_q6k_soa_host(const void* src, void* dst, uint32_t n_experts, uint64_t nblocks_per_expert);
int mx_repack_q4_K_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q4_q, int8_t* q4_sc, int8_t* q4_mn,
                          uint16_t* q4_d, uint16_t* q4_dmin);
int mx_repack_q6_K_to_soa(const void* W_blocks, uint32_t K, uint32_t N, uint8_t* q6_lo, uint8_t* q6_hi, int8_t* q6_sc,
                          uint16_t* q6_d);

/* ---------------------------------------------------------------- GGUF reader (host)
 * Memory-mapped reader of GGUF v2 / v3 files, the on-disk form of every weight this library takes:
 * GgufReader  include/ie/gguf.hpp:72-117, src/loaders/gguf_reader.cpp.  Tensor data is not copied;
 * `data` points into the mapping (valid until mx_gguf_close) at the GGUF block layout, i.e. exactly
 * what the AoS kernels and the mx_repack_* functions read.  Split models: open the first shard
 * ("...-00001-of-0000N.gguf"); the other shards are mapped too and their tensors appended.
 * Strings are not NUL-terminated: use the length.  A kv payload points at the scalar, at a string's
 * u64 length followed by its bytes, or at an array's first element (strings in arrays likewise
 * length-prefixed).  ggml_type ids as in ggml (Q4_0 2, Q8_0 8, Q4_K 12, Q5_K 13, Q6_K 14, MXFP4 39...);
 * nbytes is 0 for a type this reader does not size.  */
typedef struct {
    const char* name;
    uint64_t name_len;
    uint32_t ggml_type;
    uint32_t n_dims;
    uint64_t shape[4];          /* shape[0] is the contiguous (K) dimension; unused dims are 1 */
    uint64_t offset_in_data;
    uint64_t nbytes;
    const void* data;
} mx_gguf_tensor_t;
typedef struct {
    const char* key;
    uint64_t key_len;
    uint32_t type;              /* 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array, 10 u64, 11 i64, 12 f64 */
    uint32_t inner_type;        /* arrays: element type */
    uint64_t n_array;           /* arrays: element count */
    const void* payload;
} mx_gguf_kv_t;
int mx_gguf_open(const char* path, void** handle);
int mx_gguf_close(void* handle);
int mx_gguf_info(const void* handle, uint32_t* version, uint64_t* n_tensors, uint64_t* n_kv, uint64_t* alignment,
                 uint64_t* tensor_data_offset);
int mx_gguf_tensor(const void* handle, uint64_t i, mx_gguf_tensor_t* out);
int mx_gguf_find_tensor(const void* handle, const char* name, uint64_t* index);
int mx_gguf_kv(const void* handle, uint64_t i, mx_gguf_kv_t* out);
int mx_gguf_find_kv(const void* handle, const char* key, uint64_t* index);
const char* mx_gguf_last_error(void);   /* text of the last MX_ERR_IO / MX_ERR_FORMAT on this thread */

#ifdef __cplusplus
}
#endif
#endif /* MXQ_H */
