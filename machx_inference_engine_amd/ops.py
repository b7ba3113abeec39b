"""Host-side mirror of the reference's `src/ops` quantized-matmul functions.

Same names, argument order and meaning as `namespace ie` (include/ie/ops.hpp,
include/ie/moe_q8.hpp); device pointers become torch tensors on a HIP device,
the queue becomes torch's current stream, and a violated precondition raises
MxError instead of silently doing nothing.  Outputs are allocated here when the
caller does not pass them (the reference's callers own all buffers).
"""
import torch

from . import lib

Q81X_BYTES, Q81S_BYTES = 40, 48
BLOCK = {"q8_0": (32, 34), "q4_K": (256, 144), "q6_K": (256, 210), "mxfp4": (32, 17)}


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


# ---------------------------------------------------------------- dequant
def dequant(fmt, packed, n_elements, out=None, dtype=torch.float16):
    out = _out(out, (n_elements,), dtype, packed)
    _call("mx_dequant_%s%s" % (fmt, "" if dtype == torch.float16 else "_f32"), _u8(packed), _ptr(out), n_elements)
    return out


def dequant_to_Bt(fmt, W, K, N, Bt=None):
    Bt = _out(Bt, (K, N), torch.float16, W)
    _call("mx_dequant_%s_to_Bt" % fmt, _u8(W), _ptr(Bt), K, N)
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


def gemv_q6_K_q8_batched(x_q8, W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q6_K_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_q8_0_q8_batched(x_q8, W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q8_0_q8_batched", x_q8, (_u8(W),), K, N, T, y)


def gemv_q8_0_soa_q8_batched(x_q8, qs_W, d_W, K, N, T, y=None):
    return _gemv_q8("mx_gemv_q8_0_soa_q8_batched", x_q8, (_u8(qs_W), _ptr(d_W)), K, N, T, y)


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
