"""Host-side mirror of the reference's `src/ops` quantized-matmul functions.

Same names, argument order and meaning as `namespace ie` (include/ie/ops.hpp,
include/ie/moe_q8.hpp); device pointers become torch tensors on a HIP device,
the queue becomes torch's current stream, and a violated precondition raises
MxError instead of silently doing nothing.  Outputs are allocated here when the
caller does not pass them (the reference's callers own all buffers).
"""
import numpy as np
import torch

from . import lib

Q81X_BYTES, Q81S_BYTES = 40, 48
BLOCK = {"q8_0": (32, 34), "q4_K": (256, 144), "q6_K": (256, 210), "mxfp4": (32, 17), "q5_K": (256, 176), "q4_0": (32, 18)}


class MxError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        msg = lib.mx_status_string(status).decode()
        if status == 4:
            msg += " (hipError %d)" % lib.mx_last_hip_error()
        super().__init__("%s: %s" % (fn, msg))


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("tensor must live on the HIP device")
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous")
    return t.data_ptr()


def _call(name, *args):
    rc = getattr(lib, name)(_stream(), *args)
    if rc != 0:
        raise MxError(name, rc)


def _f16(t):
    assert t.dtype == torch.float16, t.dtype
    return _ptr(t)


def _u8(t):
    assert t.dtype in (torch.uint8, torch.int8), t.dtype
    return _ptr(t)


def _out(y, shape, dtype, like):
    if y is None:
        y = torch.empty(shape, dtype=dtype, device=like.device)
    assert y.dtype == dtype and y.numel() == int(torch.Size(shape).numel())
    return y


# ---------------------------------------------------------------- quantizers
def quantize_q8_1(x, out_q8=None):
    """x fp16/fp32 [..., K] -> uint8 block_q8_1x stream (numel/32 * 40 bytes)."""
    n = x.numel()
    out_q8 = _out(out_q8, (n // 32 * Q81X_BYTES,), torch.uint8, x)
    _call("mx_quantize_q8_1" if x.dtype == torch.float16 else "mx_quantize_q8_1_f32", _ptr(x), _ptr(out_q8), n)
    return out_q8


def quantize_q8_1s(x, out_q8=None):
    n = x.numel()
    out_q8 = _out(out_q8, (n // 32 * Q81S_BYTES,), torch.uint8, x)
    _call("mx_quantize_q8_1s" if x.dtype == torch.float16 else "mx_quantize_q8_1s_f32", _ptr(x), _ptr(out_q8), n)
    return out_q8


def probe_stream_read(buf, n_bytes=None):
    """Pure read of `buf` (or its first n_bytes) with the decode GEMV's launch geometry: the bandwidth yardstick."""
    n = buf.numel() * buf.element_size() if n_bytes is None else n_bytes
    _call("mx_probe_stream_read", _ptr(buf), n, None)


def probe_read_variant(buf, in_flight, mode, workgroups, n_bytes=None):
    """One read of `buf` with a chosen launch shape (mode 0 plain / 1 nontemporal register loads, 2 loads into LDS)."""
    n = buf.numel() * buf.element_size() if n_bytes is None else n_bytes
    _call("mx_probe_read_variant", _ptr(buf), n, in_flight, mode, workgroups, None)


def probe_lane_pattern(region, pitch, pattern, iters, workgroups):
    """16-byte-per-lane loads over `region` (uint8, 16 spare bytes at its end) under lane -> address pattern 0..6."""
    _call("mx_probe_lane_pattern", _ptr(region), region.numel() * region.element_size(), pitch, pattern, iters, workgroups, None)


# ---------------------------------------------------------------- dequant
def dequant(fmt, packed, n_elements, out=None, dtype=torch.float16):
    out = _out(out, (n_elements,), dtype, packed)
    _call("mx_dequant_%s%s" % (fmt, "" if dtype == torch.float16 else "_f32"), _u8(packed), _ptr(out), n_elements)
    return out


def dequant_to_Bt(fmt, W, K, N, Bt=None):
    Bt = _out(Bt, (K, N), torch.float16, W)
    _call("mx_dequant_%s_to_Bt" % fmt, _u8(W), _ptr(Bt), K, N)
    return Bt


def gemm_fp16(A, B, M, N, K, out_dtype=torch.float32, C=None):
    """C[M,N] = A[M,K] . B[K,N] (fp16 operands, fp32 accumulate); fp32 out = gemm_fp16, fp16 out = gemm_fp16_onednn."""
    C = _out(C, (M, N), out_dtype, A)
    _call("mx_gemm_fp16" if out_dtype == torch.float32 else "mx_gemm_fp16_onednn", _f16(A), _f16(B), _ptr(C), M, N, K)
    return C


def dequant_soa_to_Bt(name, planes, K, N, Bt=None):
    """name in ('q4_moe_soa', 'q6_K_soa', 'q4_soa', 'q6_soa', 'mxfp4_soa'); planes = device tensors in C-ABI order."""
    Bt = _out(Bt, (K, N), torch.float16, planes[0])
    _call("mx_dequant_%s_to_Bt" % name, *[_ptr(t) for t in planes], _ptr(Bt), K, N)
    return Bt


# ---------------------------------------------------------------- int-dot GEMV
def _gemv_q8(name, x_q8, wargs, K, N, T, y, dtype=torch.float16):
    y = _out(y, (T, N) if T > 1 else (N,), dtype, x_q8)
    if T > 1 or name.endswith("_batched"):
        _call(name, _u8(x_q8), *wargs, _ptr(y), K, N, T)
    else:
        _call(name, _u8(x_q8), *wargs, _ptr(y), K, N)
    return y


def gemv_q4_K_q8(x_q8, W, K, N, y=None):
    return _gemv_q8("mx_gemv_q4_K_q8", x_q8, (_u8(W),), K, N, 1, y)


def gemv_q6_K_q8(x_q8, W, K, N, y=None):
    return _gemv_q8("mx_gemv_q6_K_q8", x_q8, (_u8(W),), K, N, 1, y)


def gemv_q8_0_q8(x_q8, W, K, N, y=None):
    return _gemv_q8("mx_gemv_q8_0_q8", x_q8, (_u8(W),), K, N, 1, y)


def gemv_q8_0_soa_q8(x_q8, qs_W, d_W, K, N, y=None):
    return _gemv_q8("mx_gemv_q8_0_soa_q8", x_q8, (_u8(qs_W), _ptr(d_W)), K, N, 1, y)


def gemv_mxfp4_soa_q8(x_q8, qs_plane, e_plane, K, N, y=None):
    return _gemv_q8("mx_gemv_mxfp4_soa_q8", x_q8, (_u8(qs_plane), _u8(e_plane)), K, N, 1, y)


def gemv_q4_K_q8_batched(x_q8, W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q4_K_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_kquant_q8s_batched(fmt, x_q8s, W, K, N, T, y=None):
    """fmt in ('q4_K', 'q6_K'); x_q8s: block_q8_1s rows from quantize_q8_1s."""
    return _gemv_q8("mx_gemv_%s_q8s_batched" % fmt, x_q8s, (_u8(W),), K, N, T, y)


def gemv_q6_K_q8_batched(x_q8, W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q6_K_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_q8_0_q8_batched(x_q8, W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q8_0_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_q8_0_soa_q8_batched(x_q8, qs_W, d_W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q8_0_soa_q8_batched", x_q8, (_u8(qs_W), _ptr(d_W)), K, N, T, y)


def init():
    """Resolve the library's per-device scratch addresses for the current device (optional; see mx_init)."""
    rc = lib.mx_init()
    if rc != 0:
        raise MxError("mx_init", rc)


def gemv_batched_ws_bytes(K, N, T):
    import ctypes
    n = ctypes.c_uint64(0)
    rc = lib.mx_gemv_batched_ws_bytes(K, N, T, ctypes.addressof(n))
    if rc != 0:
        raise MxError("mx_gemv_batched_ws_bytes", rc)
    return n.value


def gemm_ws_bytes(M, K, N):
    import ctypes
    n = ctypes.c_uint64(0)
    rc = lib.mx_gemm_ws_bytes(M, K, N, ctypes.addressof(n))
    if rc != 0:
        raise MxError("mx_gemm_ws_bytes", rc)
    return n.value


def gemv_q8_batched_ws(fmt, x_q8, wargs, K, N, T, ws, y=None):
    """Caller-workspace batched GEMV: fmt in ('q4_K', 'q6_K', 'q8_0', 'q8_0_soa'); wargs = weight tensors in C-ABI order;
    ws = a device tensor of at least gemv_batched_ws_bytes(K, N, T) bytes (or None when that is 0)."""
    y = _out(y, (T, N), torch.float16, x_q8)
    _call("mx_gemv_%s_q8_batched_ws" % fmt, _u8(x_q8), *[_ptr(w) for w in wargs], _ptr(y), K, N, T, _ptr(ws) if ws is not None else None,
          ws.numel() * ws.element_size() if ws is not None else 0)
    return y


def gemm_ws(fmt, A, wargs, M, K, N, ws, y=None):
    """Caller-workspace dense quant-GEMM: fmt in ('q4_K', 'q6_K', 'q8_0', 'q8_0_soa')."""
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_%s_ws" % fmt, _f16(A), *[_ptr(w) for w in wargs], _ptr(y), M, K, N, _ptr(ws) if ws is not None else None,
          ws.numel() * ws.element_size() if ws is not None else 0)
    return y


def gemv_mxfp4_soa_q8_batched(x_q8, qs_plane, e_plane, K, N, T, y=None):
    return _gemv_q8("mx_gemv_mxfp4_soa_q8_batched", x_q8, (_u8(qs_plane), _u8(e_plane)), K, N, T, y)


def gemv_q8_f32(fmt, x_q8, W, K, N, y=None):
    """fp32-output int-dot GEMV (fmt in q4_K, q6_K, q8_0)."""
    return _gemv_q8("mx_gemv_%s_q8_f32" % fmt, x_q8, (_u8(W),), K, N, 1, y, torch.float32)


def gemv_mxfp4_soa_q8_x2(x_q8, gate_qs, gate_e, up_qs, up_e, gate_bias, up_bias, K, N, gate_y=None, up_y=None):
    gate_y = _out(gate_y, (N,), torch.float16, x_q8)
    up_y = _out(up_y, (N,), torch.float16, x_q8)
    _call("mx_gemv_mxfp4_soa_q8_x2", _u8(x_q8), _u8(gate_qs), _u8(gate_e), _u8(up_qs), _u8(up_e), _ptr(gate_bias),
          _ptr(up_bias), _ptr(gate_y), _ptr(up_y), K, N)
    return gate_y, up_y


# ---------------------------------------------------------------- float-activation GEMV
def _gemv_f(fmt, A, W, K, N, y):
    if A.dtype == torch.float16:
        y = _out(y, (N,), torch.float16, A)
        _call("mx_gemv_%s" % fmt, _ptr(A), _u8(W), _ptr(y), K, N)
    else:
        assert A.dtype == torch.float32
        y = _out(y, (N,), torch.float32, A)
        _call("mx_gemv_%s_f32" % fmt, _ptr(A), _u8(W), _ptr(y), K, N)
    return y


def gemv_q4_K(A, W, K, N, y=None):
    return _gemv_f("q4_K", A, W, K, N, y)


def gemv_q6_K(A, W, K, N, y=None):
    return _gemv_f("q6_K", A, W, K, N, y)


def gemv_q8_0(A, W, K, N, y=None):
    return _gemv_f("q8_0", A, W, K, N, y)


def gemv_mxfp4_soa_f16(A, qs_plane, e_plane, K, N, y=None):
    y = _out(y, (N,), torch.float16, A)
    _call("mx_gemv_mxfp4_soa_f16", _f16(A), _u8(qs_plane), _u8(e_plane), _ptr(y), K, N)
    return y


# ---------------------------------------------------------------- MoE, expert-indexed GEMV
def moe_gate_up_silu_q8(x_q8, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, topk_idx, T, K, H, E_ffn, h_out=None, n_experts=None):
    """n_experts given: the *_n entry point, slots whose id lies outside [0, n_experts) are skipped."""
    h_out = _out(h_out, (T * K, E_ffn), torch.float16, x_q8)
    args = (_u8(x_q8), _u8(g_qs), _ptr(g_d), _u8(u_qs), _ptr(u_d), qs_stride, d_stride, _ptr(topk_idx), _ptr(h_out), T, K, H, E_ffn)
    if n_experts is None:
        _call("mx_moe_gate_up_silu_q8", *args)
    else:
        _call("mx_moe_gate_up_silu_q8_n", *args, n_experts)
    return h_out


def moe_down_q8(h_q8, d_qs, d_d, qs_stride, d_stride, topk_idx, topk_w, T, K, E_ffn, H, y_packed=None, n_experts=None):
    y_packed = _out(y_packed, (T * K, H), torch.float16, h_q8)
    args = (_u8(h_q8), _u8(d_qs), _ptr(d_d), qs_stride, d_stride, _ptr(topk_idx), _f16(topk_w), _ptr(y_packed), T, K, E_ffn, H)
    if n_experts is None:
        _call("mx_moe_down_q8", *args)
    else:
        _call("mx_moe_down_q8_n", *args, n_experts)
    return y_packed


def moe_down_q8_f16(h_f16, d_qs, d_d, qs_stride, d_stride, topk_idx, topk_w, T, K, E_ffn, H, y_packed=None, n_experts=None):
    """moe_down_q8 on fp16 h rows [T*K][E_ffn], quantized while they are staged (no quantize launch)."""
    y_packed = _out(y_packed, (T * K, H), torch.float16, h_f16)
    args = (_f16(h_f16), _u8(d_qs), _ptr(d_d), qs_stride, d_stride, _ptr(topk_idx), _f16(topk_w), _ptr(y_packed), T, K, E_ffn, H)
    if n_experts is None:
        _call("mx_moe_down_q8_f16", *args)
    else:
        _call("mx_moe_down_q8_f16_n", *args, n_experts)
    return y_packed


def moe_reduce_q8(y_packed, T, K, H, y=None):
    y = _out(y, (T, H), torch.float16, y_packed)
    _call("mx_moe_reduce_q8", _f16(y_packed), _ptr(y), T, K, H)
    return y


def moe_prefill_gate_up_silu_q8(xq8_packed, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, expert_offsets, TK, E, H, E_ffn, h_packed=None):
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, xq8_packed)
    _call("mx_moe_prefill_gate_up_silu_q8", _u8(xq8_packed), _u8(g_qs), _ptr(g_d), _u8(u_qs), _ptr(u_d), qs_stride, d_stride,
          _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn)
    return h_packed


def moe_prefill_down_q8(hq8_packed, d_qs, d_d, qs_stride, d_stride, expert_offsets, sorted_w, TK, E, H, E_ffn, out_packed=None):
    out_packed = _out(out_packed, (TK, H), torch.float16, hq8_packed)
    _call("mx_moe_prefill_down_q8", _u8(hq8_packed), _u8(d_qs), _ptr(d_d), qs_stride, d_stride, _ptr(expert_offsets), _f16(sorted_w),
          _ptr(out_packed), E, H, E_ffn)
    return out_packed


def moe_prefill_reduce_sum(out_packed, tk_to_packed, T, K, H, y=None):
    y = _out(y, (T, H), torch.float16, out_packed)
    _call("mx_moe_prefill_reduce_sum", _f16(out_packed), _ptr(tk_to_packed), _ptr(y), T, K, H)
    return y


def moe_prefill_reduce(out_packed, tk_to_packed, weights_packed, y, T, K_top, H):
    """y[t] += sum_k w[row] * out_packed[row]; accumulates into y (the caller zeroes it)."""
    _call("mx_moe_prefill_reduce", _f16(out_packed), _ptr(tk_to_packed), _f16(weights_packed), _f16(y), T, K_top, H)
    return y


def moe_decode_gate_up_silu_q4k(x, gate_W, up_W, topk_idx, H, E_ffn, K_top, expert_stride_bytes, T=1, h_out=None, soa=False):
    h_out = _out(h_out, (T * K_top, E_ffn), torch.float16, x)
    _call("mx_moe_decode_gate_up_silu_q4k", _f16(x), _u8(gate_W), _u8(up_W), _ptr(topk_idx), _ptr(h_out), H, E_ffn, K_top, expert_stride_bytes,
          int(soa), T)
    return h_out


def moe_decode_down_kquant(fmt, h, down_W, topk_idx, topk_w, H, E_ffn, K_top, expert_stride_bytes, T=1, y_out=None, soa=False):
    """fmt in ('q4k', 'q6k')."""
    y_out = _out(y_out, (T, H), torch.float16, h)
    _call("mx_moe_decode_down_%s" % fmt, _f16(h), _u8(down_W), _ptr(topk_idx), _f16(topk_w), _ptr(y_out), H, E_ffn, K_top, expert_stride_bytes,
          int(soa), T)
    return y_out


def moe_prefill_gate_up_silu_kquant_q8(fmt, xq8s_packed, gate_W, up_W, expert_offsets, TK, E, H, E_ffn, expert_stride_bytes, h_packed=None,
                                       soa=False):
    """fmt in ('q4k', 'q6k'); xq8s_packed: block_q8_1s rows (quantize_q8_1s), as the reference kernels read them."""
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, xq8s_packed)
    _call("mx_moe_prefill_gate_up_silu_%s_q8" % fmt, _ptr(xq8s_packed), _u8(gate_W), _u8(up_W), _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn,
          expert_stride_bytes, int(soa), TK)
    return h_packed


def moe_prefill_down_packed_kquant_q8(fmt, hq8s_packed, down_W, expert_offsets, TK, E, H, E_ffn, expert_stride_bytes, out_packed=None,
                                      soa=False):
    """fmt in ('q4k', 'q6k'); hq8s_packed: block_q8_1s rows."""
    out_packed = _out(out_packed, (TK, H), torch.float16, hq8s_packed)
    _call("mx_moe_prefill_down_packed_%s_q8" % fmt, _ptr(hq8s_packed), _u8(down_W), _ptr(expert_offsets), _ptr(out_packed), E, H, E_ffn,
          expert_stride_bytes, int(soa), TK)
    return out_packed


def moe_gather_rows(x, indices, n_rows, hidden, y_packed=None):
    y_packed = _out(y_packed, (n_rows, hidden), torch.float16, x)
    _call("mx_moe_gather_rows", _f16(x), _ptr(indices), _ptr(y_packed), n_rows, hidden)
    return y_packed


def moe_prefill_down_kquant_accum(fmt, h_packed, down_W, expert_offsets, sorted_token_idx, sorted_token_w, y_fp32, TK, E, H, E_ffn,
                                  expert_stride_bytes):
    """fmt in ('q4k', 'q6k'): y_fp32[token] += w * (down . h) with fp32 atomics (the caller zeroes y_fp32)."""
    assert y_fp32.dtype == torch.float32
    _call("mx_moe_prefill_down_%s" % fmt, _f16(h_packed), _u8(down_W), _ptr(expert_offsets), _ptr(sorted_token_idx), _f16(sorted_token_w),
          _ptr(y_fp32), E, H, E_ffn, expert_stride_bytes, TK)
    return y_fp32


def moe_prefill_merge_fp32_to_fp16(y_fp32, y_fp16):
    _call("mx_moe_prefill_merge_fp32_to_fp16", _ptr(y_fp32), _f16(y_fp16), y_fp16.numel())
    return y_fp16


def moe_scatter_add(x_packed, indices, weights, y, n_tok, hidden):
    """y[indices[i]] += weights[i] * x_packed[i] in place (rows named by one call must be distinct)."""
    _call("mx_moe_scatter_add", _f16(x_packed), _ptr(indices), _f16(weights), _f16(y), n_tok, hidden)
    return y


def moe_gate_up_oai_mxfp4(x_q8, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, topk_idx, T, K, H, E_ffn, n_experts,
                          alpha=1.702, limit=7.0, h_out=None):
    h_out = _out(h_out, (T * K, E_ffn), torch.float16, x_q8)
    _call("mx_moe_gate_up_oai_mxfp4", _u8(x_q8), _u8(g_qs), _u8(g_e), _u8(u_qs), _u8(u_e), qs_stride, e_stride, _ptr(gate_bias),
          _ptr(up_bias), _ptr(topk_idx), _ptr(h_out), T, K, H, E_ffn, n_experts, alpha, limit)
    return h_out


def moe_down_mxfp4(h_q8, d_qs, d_e, qs_stride, e_stride, down_bias, topk_idx, T, K, E_ffn, H, n_experts, out_packed=None):
    out_packed = _out(out_packed, (T * K, H), torch.float16, h_q8)
    _call("mx_moe_down_mxfp4", _u8(h_q8), _u8(d_qs), _u8(d_e), qs_stride, e_stride, _ptr(down_bias), _ptr(topk_idx), _ptr(out_packed),
          T, K, E_ffn, H, n_experts)
    return out_packed


def moe_down_mxfp4_f16(h_f16, d_qs, d_e, qs_stride, e_stride, down_bias, topk_idx, T, K, E_ffn, H, n_experts, out_packed=None):
    """moe_down_mxfp4 on fp16 h rows [T*K][E_ffn], quantized while they are staged (no quantize launch)."""
    out_packed = _out(out_packed, (T * K, H), torch.float16, h_f16)
    _call("mx_moe_down_mxfp4_f16", _f16(h_f16), _u8(d_qs), _u8(d_e), qs_stride, e_stride, _ptr(down_bias), _ptr(topk_idx),
          _ptr(out_packed), T, K, E_ffn, H, n_experts)
    return out_packed


def moe_grouped_gate_up_oai_mxfp4(xq8_packed, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, expert_offsets, TK, E, H,
                                  E_ffn, alpha=1.702, limit=7.0, h_packed=None):
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, xq8_packed)
    _call("mx_moe_grouped_gate_up_oai_mxfp4", _u8(xq8_packed), _u8(g_qs), _u8(g_e), _u8(u_qs), _u8(u_e), qs_stride, e_stride,
          _ptr(gate_bias), _ptr(up_bias), _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn, TK, alpha, limit)
    return h_packed


def moe_grouped_down_mxfp4(hq8_packed, d_qs, d_e, qs_stride, e_stride, down_bias, expert_offsets, TK, E, H, E_ffn, out_packed=None):
    out_packed = _out(out_packed, (TK, H), torch.float16, hq8_packed)
    _call("mx_moe_grouped_down_mxfp4", _u8(hq8_packed), _u8(d_qs), _u8(d_e), qs_stride, e_stride, _ptr(down_bias), _ptr(expert_offsets),
          _ptr(out_packed), E, H, E_ffn, TK)
    return out_packed


def moe_grouped_down_mxfp4_f16(h_packed_f16, d_qs, d_e, qs_stride, e_stride, down_bias, expert_offsets, TK, E, H, E_ffn, out_packed=None):
    """moe_grouped_down_mxfp4 on fp16 packed h rows [TK][E_ffn], quantized while they are staged."""
    out_packed = _out(out_packed, (TK, H), torch.float16, h_packed_f16)
    _call("mx_moe_grouped_down_mxfp4_f16", _f16(h_packed_f16), _u8(d_qs), _u8(d_e), qs_stride, e_stride, _ptr(down_bias),
          _ptr(expert_offsets), _ptr(out_packed), E, H, E_ffn, TK)
    return out_packed


def build_moe_packing(topk_ids, topk_w, E):
    """Host counting sort (numpy in, numpy out): expert_offsets[E+1], sorted_idx, weights_packed, tk_to_packed."""
    ids = np.ascontiguousarray(topk_ids, np.int32)
    w = np.ascontiguousarray(topk_w, np.float32)
    T, K = ids.shape
    off, si = np.empty(E + 1, np.uint32), np.empty(T * K, np.int32)
    wp, t2p = np.empty(T * K, np.float32), np.empty(T * K, np.int32)
    rc = lib.mx_build_moe_packing(ids.ctypes.data, w.ctypes.data, T, K, E, off.ctypes.data, si.ctypes.data, wp.ctypes.data, t2p.ctypes.data)
    if rc != 0:
        raise MxError("mx_build_moe_packing", rc)
    return off, si, wp, t2p


def gemv_q4_K_dual(A, W_a, W_b, K, N):
    ya = torch.empty(N, dtype=torch.float16, device=A.device)
    yb = torch.empty(N, dtype=torch.float16, device=A.device)
    _call("mx_gemv_q4_K_dual", _f16(A), _u8(W_a), _u8(W_b), _ptr(ya), _ptr(yb), K, N)
    return ya, yb


def gemv_q4_K_down_accum(A, W, sh_g, y, K, N):
    _call("mx_gemv_q4_K_down_accum", _f16(A), _u8(W), _f16(sh_g), _f16(y), K, N)
    return y


def gemv_q8_x2(fmt, x_q8, W_a, W_b, K, N, y_a=None, y_b=None):
    """Fused gate + up: fmt in ('q4_K', 'q6_K', 'q8_0') with W = GGUF blocks, 'q8_0_soa' with W = (qs, d), or 'q6_soa' with W = planes."""
    y_a, y_b = _out(y_a, (N,), torch.float16, x_q8), _out(y_b, (N,), torch.float16, x_q8)
    if fmt == "q8_0_soa":
        _call("mx_gemv_q8_0_soa_q8_x2", _u8(x_q8), _u8(W_a[0]), _ptr(W_a[1]), _u8(W_b[0]), _ptr(W_b[1]), _ptr(y_a), _ptr(y_b), K, N)
    elif fmt == "q6_soa":   # W = (q6_lo, q6_hi, q6_sc, q6_d) from repack_q6_K_to_soa
        _call("mx_gemv_q6_soa_q8_x2", _u8(x_q8), *[_ptr(t) for t in W_a], *[_ptr(t) for t in W_b], _ptr(y_a), _ptr(y_b), K, N)
    else:
        _call("mx_gemv_%s_q8_x2" % fmt, _u8(x_q8), _u8(W_a), _u8(W_b), _ptr(y_a), _ptr(y_b), K, N)
    return y_a, y_b


def gemv_x2_silu(fmt, x, W_gate, W_up, K, N, h=None):
    """h = silu(W_gate . x) * (W_up . x) in one launch (decode, T = 1); x = the q8 row (uint8 tensor) or the fp16 row.
    fmt as gemv_q8_x2.  Same bits as gemv_q8_x2 + swiglu (and quantize_q8_1 in front when x is fp16)."""
    x_is_f16 = 1 if x.dtype == torch.float16 else 0
    h = _out(h, (N,), torch.float16, x)
    if fmt == "q8_0_soa":
        _call("mx_gemv_q8_0_soa_x2_silu", _ptr(x), x_is_f16, _u8(W_gate[0]), _ptr(W_gate[1]), _u8(W_up[0]), _ptr(W_up[1]), _ptr(h), K, N)
    else:
        _call("mx_gemv_%s_x2_silu" % fmt, _ptr(x), x_is_f16, _u8(W_gate), _u8(W_up), _ptr(h), K, N)
    return h


def gemv_f16q8(fmt, x_f16, W, K, N, y=None):
    """y = W . q8(x) with the fp16 row x quantized while it is staged: quantize_q8_1 + gemv_*_q8 in one launch (T = 1)."""
    y = _out(y, (N,), torch.float16, x_f16)
    if fmt == "q8_0_soa":
        _call("mx_gemv_q8_0_soa_f16q8", _f16(x_f16), _u8(W[0]), _ptr(W[1]), _ptr(y), K, N)
    else:
        _call("mx_gemv_%s_f16q8" % fmt, _f16(x_f16), _u8(W), _ptr(y), K, N)
    return y


def gemv_q4_0(A, W, K, N, y=None):
    y = _out(y, (N,), torch.float16, A)
    _call("mx_gemv_q4_0", _f16(A), _u8(W), _ptr(y), K, N)
    return y


def gemv_q4_0_q8(x_q8, W, K, N, T=1, y=None):
    return _gemv_q8("mx_gemv_q4_0_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_q4_0_soa_q8(x_q8, q4_qs, q4_d, K, N, T=1, y=None):
    return _gemv_q8("mx_gemv_q4_0_soa_q8" + ("_batched" if T > 1 else ""), x_q8, (_u8(q4_qs), _ptr(q4_d)), K, N, T, y)


def gemv_q4_0_soa_q8_multi(x_q8, banks, K):
    """banks = [(q4_qs, q4_d, N), ...] (1 to 3) sharing x_q8 -> list of fp16 [N] outputs, one launch."""
    import ctypes as C
    n = len(banks)
    ys = [torch.empty(b[2], dtype=torch.float16, device=x_q8.device) for b in banks]
    qs = (C.c_void_p * n)(*[_u8(b[0]) for b in banks])
    d = (C.c_void_p * n)(*[_ptr(b[1]) for b in banks])
    yp = (C.c_void_p * n)(*[_ptr(t) for t in ys])
    Ns = (C.c_uint32 * n)(*[b[2] for b in banks])
    _call("mx_gemv_q4_0_soa_q8_multi", _u8(x_q8), C.cast(qs, C.c_void_p), C.cast(d, C.c_void_p), C.cast(yp, C.c_void_p), C.cast(Ns, C.c_void_p), n, K)
    return ys


def gemv_q5_K(A, W, K, N, y=None):
    y = _out(y, (N,), torch.float16, A)
    _call("mx_gemv_q5_K", _f16(A), _u8(W), _ptr(y), K, N)
    return y


def gemv_q5_K_q8(x_q8, W, K, N, T=1, y=None):
    return _gemv_q8("mx_gemv_q5_K_q8" + ("_batched" if T > 1 else ""), x_q8, (_u8(W),), K, N, T, y)


def gemm_q4_0(A, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q4_0", _f16(A), _u8(W), _ptr(y), M, K, N)
    return y


def moe_prefill_proj_q4_0(kind, rows, W, expert_offsets, TK, E, K, N, stride, out_packed=None):
    """kind 'q8' (rows = block_q8_1s stream, W = GGUF blocks, stride = expert_stride_bytes), 'soa_q8' (W = (qs_bank, d_bank),
    stride = (qs_stride, d_stride)) or 'xmx' (rows = fp16 [TK, K], W = GGUF blocks)."""
    out_packed = _out(out_packed, (TK, N), torch.float16, rows)
    if kind == "soa_q8":
        _call("mx_moe_prefill_proj_q4_0_soa_q8", _ptr(rows), _u8(W[0]), _ptr(W[1]), _ptr(expert_offsets), _ptr(out_packed), E, K, N, stride[0], stride[1], TK)
    else:
        _call("mx_moe_prefill_proj_q4_0_%s" % kind, _ptr(rows), _u8(W), _ptr(expert_offsets), _ptr(out_packed), E, K, N, stride, TK)
    return out_packed


def gemm_q4_0_q8(xq8s, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, xq8s)
    _call("mx_gemm_q4_0_q8", _ptr(xq8s), _u8(W), _ptr(y), M, K, N)
    return y


def repack_q4_0_to_soa(W, K, N):
    W = _np_u8(W)
    qs, d = np.empty(N * K // 2, np.uint8), np.empty(N * K // 32, np.uint16)
    _host("mx_repack_q4_0_to_soa", W.ctypes.data, K, N, qs.ctypes.data, d.ctypes.data)
    return qs, d


def gemv_q4_K_reorder_q8(x_q8, W_reorder, K, N, y=None):
    return _gemv_q8("mx_gemv_q4_K_reorder_q8", x_q8, (_u8(W_reorder),), K, N, 1, y)


def gemv_q4_soa_q8(x_q8, planes, K, N, y=None):
    """planes = (q4_q, q4_sc, q4_mn, q4_d, q4_dmin) from repack_q4_K_to_soa."""
    return _gemv_q8("mx_gemv_q4_soa_q8", x_q8, tuple(_ptr(t) for t in planes), K, N, 1, y)


def gemv_q6_soa_q8(x_q8, planes, K, N, T=1, y=None):
    """planes = (q6_lo, q6_hi, q6_sc, q6_d) from repack_q6_K_to_soa."""
    return _gemv_q8("mx_gemv_q6_soa_q8" + ("_batched" if T > 1 else ""), x_q8, tuple(_ptr(t) for t in planes), K, N, T, y)


# ---------------------------------------------------------------- host repackers (numpy in, numpy out)
def _np_u8(a):
    a = np.ascontiguousarray(a).view(np.uint8).ravel()
    return a


def repack_q4_K_to_reorder(W, K, N):
    W = _np_u8(W)
    out = np.empty(N * (K // 256) * 144, np.uint8)
    _host("mx_repack_q4_K_to_reorder", W.ctypes.data, K, N, out.ctypes.data)
    return out


def repack_moe_kquant_soa(fmt, bank, n_experts, nblocks_per_expert):
    """fmt in ('q4k', 'q6k'): AoS expert-major bank -> the same regions as per-field streams."""
    bank = _np_u8(bank)
    out = np.empty_like(bank)
    _host("mx_repack_moe_%s_soa_host" % fmt, bank.ctypes.data, out.ctypes.data, n_experts, nblocks_per_expert)
    return out


def repack_q4_K_to_soa(W, K, N):
    W = _np_u8(W)
    q = np.empty(N * K // 2, np.uint8)
    sc, mn = np.empty(N * K // 32, np.int8), np.empty(N * K // 32, np.int8)
    d, dmin = np.empty(N * K // 256, np.uint16), np.empty(N * K // 256, np.uint16)
    _host("mx_repack_q4_K_to_soa", W.ctypes.data, K, N, q.ctypes.data, sc.ctypes.data, mn.ctypes.data, d.ctypes.data, dmin.ctypes.data)
    return q, sc, mn, d, dmin


def repack_q6_K_to_soa(W, K, N):
    W = _np_u8(W)
    lo, hi = np.empty(N * K // 2, np.uint8), np.empty(N * K // 4, np.uint8)
    sc, d = np.empty(N * K // 16, np.int8), np.empty(N * K // 256, np.uint16)
    _host("mx_repack_q6_K_to_soa", W.ctypes.data, K, N, lo.ctypes.data, hi.ctypes.data, sc.ctypes.data, d.ctypes.data)
    return lo, hi, sc, d


def repack_block32_to_soa(fmt, blocks):
    """fmt 'q8_0' -> (qs int8, d uint16); 'mxfp4' -> (qs uint8, e uint8)."""
    blocks = _np_u8(blocks)
    if fmt == "q8_0":
        nb = blocks.size // 34
        qs, d = np.empty(nb * 32, np.int8), np.empty(nb, np.uint16)
        _host("mx_repack_q8_0_to_soa", blocks.ctypes.data, nb, qs.ctypes.data, d.ctypes.data)
        return qs, d
    nb = blocks.size // 17
    qs, e = np.empty(nb * 16, np.uint8), np.empty(nb, np.uint8)
    _host("mx_repack_mxfp4_to_soa", blocks.ctypes.data, nb, qs.ctypes.data, e.ctypes.data)
    return qs, e


def _host(name, *args):
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise MxError(name, rc)


def gemv_q4_K_shexp_gate_up(A, W_gate, W_up, W_shg, K, N):
    """-> (y_h fp16 [N] = silu(W_gate.A) * (W_up.A), sh_g fp16 [1] = sigmoid(W_shg . A))."""
    assert W_shg.dtype == torch.float32
    y_h = torch.empty(N, dtype=torch.float16, device=A.device)
    sh_g = torch.empty(1, dtype=torch.float16, device=A.device)
    _call("mx_gemv_q4_K_shexp_gate_up", _f16(A), _u8(W_gate), _u8(W_up), _ptr(W_shg), _ptr(y_h), _ptr(sh_g), K, N)
    return y_h, sh_g


def gemv_q4_K_dual_ssm_gbeta(A, W_alpha, W_beta, A_log, dt_bias, K, N):
    """-> (g fp32 [N] = A_log * softplus(half(W_alpha.A) + dt_bias), beta fp32 [N] = sigmoid(half(W_beta.A)))."""
    assert A_log.dtype == torch.float32 and dt_bias.dtype == torch.float32
    g = torch.empty(N, dtype=torch.float32, device=A.device)
    beta = torch.empty(N, dtype=torch.float32, device=A.device)
    _call("mx_gemv_q4_K_dual_ssm_gbeta", _f16(A), _u8(W_alpha), _u8(W_beta), _ptr(A_log), _ptr(dt_bias), _ptr(g), _ptr(beta), K, N)
    return g, beta


# ---------------------------------------------------------------- routing / packing on the device
def moe_router(x, W_gate, n_experts, k):
    """x fp16 [T, H], W_gate fp32 [E, H] -> (topk_idx int32 [T, k] ascending, topk_w fp16 [T, k])."""
    T, H = x.shape
    idx = torch.empty((T, k), dtype=torch.int32, device=x.device)
    w = torch.empty((T, k), dtype=torch.float16, device=x.device)
    ws = torch.empty((T, n_experts), dtype=torch.float32, device=x.device)
    assert W_gate.dtype == torch.float32
    _call("mx_moe_router", _f16(x), _ptr(W_gate), _ptr(idx), _ptr(w), T, H, n_experts, k, _ptr(ws))
    return idx, w


def moe_topk_from_logits(logits, k):
    T, E = logits.shape
    idx = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, k), dtype=torch.float16, device=logits.device)
    _call("mx_moe_topk_from_logits", _f16(logits), _ptr(idx), _ptr(w), E, k, T)
    return idx, w


def moe_build_packing_device(topk_idx, topk_w, E, decode=False):
    """Device arrays (expert_offsets uint32-as-int32 [E+1], sorted_idx, weights_packed fp16, tk_to_packed)."""
    T, K = topk_idx.shape
    dev = topk_idx.device
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    si = torch.empty(T * K, dtype=torch.int32, device=dev)
    wp = torch.empty(T * K, dtype=torch.float16, device=dev)
    t2p = torch.empty(T * K, dtype=torch.int32, device=dev)
    if decode:
        assert T == 1
        _call("mx_moe_build_pack_decode", _ptr(topk_idx), _f16(topk_w), _ptr(off), _ptr(si), _ptr(t2p), _ptr(wp), E, K)
    else:
        _call("mx_moe_build_packing_device", _ptr(topk_idx), _f16(topk_w), T, K, E, _ptr(off), _ptr(si), _ptr(wp), _ptr(t2p))
    return off, si, wp, t2p


# ---------------------------------------------------------------- fused norm -> q8 producers
def rms_norm_f32w_q8(x, w, eps):
    n_rows, hidden = x.shape
    y = torch.empty_like(x)
    q8 = torch.empty(n_rows * hidden // 32 * Q81X_BYTES, dtype=torch.uint8, device=x.device)
    assert w.dtype == torch.float32
    _call("mx_rms_norm_f32w_q8", _f16(x), _ptr(w), _ptr(y), _ptr(q8), n_rows, hidden, float(eps))
    return y, q8


def swiglu_q8(gate, up, oai=False, alpha=1.702, limit=7.0, want_y=True, out=None):
    """-> (y fp16 or None, block_q8_1x stream of y): silu(gate)*up, or the clamped gpt-oss form with oai=True.
    out = (y, q8) reuses caller buffers."""
    n = gate.numel()
    if out is not None:
        y, q8 = out
    else:
        y = torch.empty_like(gate) if want_y else None
        q8 = torch.empty(n // 32 * Q81X_BYTES, dtype=torch.uint8, device=gate.device)
    if oai:
        _call("mx_swiglu_oai_q8", _f16(gate), _f16(up), _ptr(y), _ptr(q8), n, alpha, limit)
    else:
        _call("mx_swiglu_q8", _f16(gate), _f16(up), _ptr(y), _ptr(q8), n)
    return y, q8


def gated_rms_norm_q8(x, z, weight, eps):
    n_rows, hidden = x.shape
    assert x.dtype == torch.float32
    y = torch.empty((n_rows, hidden), dtype=torch.float16, device=x.device)
    q8 = torch.empty(n_rows * hidden // 32 * Q81X_BYTES, dtype=torch.uint8, device=x.device)
    _call("mx_gated_rms_norm_q8", _ptr(x), _f16(z), _f16(weight), _ptr(y), _ptr(q8), n_rows, hidden, float(eps))
    return y, q8


# ---------------------------------------------------------------- prefill GEMM (MFMA)
def gemm_q4_K(A, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q4_K", _f16(A), _u8(W), _ptr(y), M, K, N)
    return y


def gemm_q6_K(A, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q6_K", _f16(A), _u8(W), _ptr(y), M, K, N)
    return y


def gemm_q8_0(A, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q8_0", _f16(A), _u8(W), _ptr(y), M, K, N)
    return y


def moe_gemm_gate_up_silu_q4k(x_packed, gate_W, up_W, expert_offsets, TK, E, H, E_ffn, expert_stride_bytes, h_packed=None, soa=False, sorted_idx=None):
    """soa: the expert regions hold per-field streams (repack_moe_kquant_soa) instead of GGUF blocks.
    sorted_idx (int32 [TK]): x_packed is the unsorted [T, H] matrix and the rows are gathered while they are loaded."""
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, x_packed)
    if sorted_idx is not None:
        _call("mx_moe_gemm_gate_up_silu_q4k_gather", _f16(x_packed), _ptr(sorted_idx), x_packed.numel() // H, _u8(gate_W), _u8(up_W), _ptr(expert_offsets),
              _ptr(h_packed), E, H, E_ffn, expert_stride_bytes, 1 if soa else 0, TK)
        return h_packed
    _call("mx_moe_gemm_gate_up_silu_q4k", _f16(x_packed), _u8(gate_W), _u8(up_W), _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn,
          expert_stride_bytes, 1 if soa else 0, TK)
    return h_packed


def moe_gemm_down_kquant(fmt, h_packed, down_W, expert_offsets, sorted_w, TK, E, H, E_ffn, expert_stride_bytes, out_packed=None, soa=False):
    """fmt in ('q4k', 'q6k'); sorted_w None -> unweighted packed rows."""
    out_packed = _out(out_packed, (TK, H), torch.float16, h_packed)
    _call("mx_moe_gemm_down_%s" % fmt, _f16(h_packed), _u8(down_W), _ptr(expert_offsets), _f16(sorted_w) if sorted_w is not None else None,
          _ptr(out_packed), E, H, E_ffn, expert_stride_bytes, 1 if soa else 0, TK)
    return out_packed


def gemm_q5_K(A, W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q5_K", _f16(A), _u8(W), _ptr(y), M, K, N)
    return y


def gemm_mxfp4_soa(A, qs_plane, e_plane, M, K, N, y=None):
    """y[M,N] = A . half(deq(W))^T for MXFP4 planes, K % 64 == 0 (fused: no [K,N] fp16 matrix is written)."""
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_mxfp4_soa", _f16(A), _u8(qs_plane), _u8(e_plane), _ptr(y), M, K, N)
    return y


def moe_gemm_gate_up_oai_mxfp4(x_packed, g_qs, g_e, u_qs, u_e, qs_stride, e_stride, gate_bias, up_bias, expert_offsets, TK, E, H, E_ffn,
                               alpha=1.702, limit=7.0, h_packed=None, sorted_idx=None):
    """sorted_idx (int32 [TK]): x_packed is the unsorted [T, H] matrix and the rows are gathered while they are loaded."""
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, x_packed)
    if sorted_idx is not None:
        _call("mx_moe_gemm_gate_up_oai_mxfp4_gather", _f16(x_packed), _ptr(sorted_idx), x_packed.numel() // H, _u8(g_qs), _u8(g_e), _u8(u_qs), _u8(u_e),
              qs_stride, e_stride, _ptr(gate_bias) if gate_bias is not None else None, _ptr(up_bias) if up_bias is not None else None,
              _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn, TK, float(alpha), float(limit))
        return h_packed
    _call("mx_moe_gemm_gate_up_oai_mxfp4", _f16(x_packed), _u8(g_qs), _u8(g_e), _u8(u_qs), _u8(u_e), qs_stride, e_stride,
          _ptr(gate_bias) if gate_bias is not None else None, _ptr(up_bias) if up_bias is not None else None, _ptr(expert_offsets), _ptr(h_packed),
          E, H, E_ffn, TK, float(alpha), float(limit))
    return h_packed


def moe_gemm_down_mxfp4(h_packed, d_qs, d_e, qs_stride, e_stride, down_bias, expert_offsets, TK, E, H, E_ffn, out_packed=None):
    out_packed = _out(out_packed, (TK, H), torch.float16, h_packed)
    _call("mx_moe_gemm_down_mxfp4", _f16(h_packed), _u8(d_qs), _u8(d_e), qs_stride, e_stride, _ptr(down_bias) if down_bias is not None else None,
          _ptr(expert_offsets), _ptr(out_packed), E, H, E_ffn, TK)
    return out_packed


def gemm_q8_0_soa(A, qs_W, d_W, M, K, N, y=None):
    y = _out(y, (M, N), torch.float16, A)
    _call("mx_gemm_q8_0_soa", _f16(A), _u8(qs_W), _ptr(d_W), _ptr(y), M, K, N)
    return y


def moe_gemm_gate_up_silu_q8(x_packed, g_qs, g_d, u_qs, u_d, qs_stride, d_stride, expert_offsets, TK, E, H, E_ffn, h_packed=None, sorted_idx=None):
    """sorted_idx (int32 [TK]): x_packed is the unsorted [T, H] matrix and the rows are gathered while they are loaded."""
    h_packed = _out(h_packed, (TK, E_ffn), torch.float16, x_packed)
    if sorted_idx is not None:
        _call("mx_moe_gemm_gate_up_silu_q8_gather", _f16(x_packed), _ptr(sorted_idx), x_packed.numel() // H, _u8(g_qs), _ptr(g_d), _u8(u_qs), _ptr(u_d),
              qs_stride, d_stride, _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn, TK)
        return h_packed
    _call("mx_moe_gemm_gate_up_silu_q8", _f16(x_packed), _u8(g_qs), _ptr(g_d), _u8(u_qs), _ptr(u_d), qs_stride, d_stride,
          _ptr(expert_offsets), _ptr(h_packed), E, H, E_ffn, TK)
    return h_packed


def moe_gemm_down_q8(h_packed, d_qs, d_d, qs_stride, d_stride, expert_offsets, sorted_w, TK, E, H, E_ffn, out_packed=None):
    out_packed = _out(out_packed, (TK, H), torch.float16, h_packed)
    _call("mx_moe_gemm_down_q8", _f16(h_packed), _u8(d_qs), _ptr(d_d), qs_stride, d_stride, _ptr(expert_offsets), _f16(sorted_w),
          _ptr(out_packed), E, H, E_ffn, TK)
    return out_packed


def gemm_q8_rows(fmt, xq8s, wargs, M, K, N, y=None):
    """Dense int-dot GEMM over block_q8_1s rows: fmt in ('q4_K', 'q6_K', 'q8_0_soa'); wargs = weight tensors in C-ABI order."""
    y = _out(y, (M, N), torch.float16, xq8s)
    _call("mx_gemm_%s_q8" % fmt, _u8(xq8s), *[_ptr(w) for w in wargs], _ptr(y), M, K, N)
    return y
