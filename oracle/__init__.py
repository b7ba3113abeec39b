"""ctypes front end of the CPU oracle (oracle/mxq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.

All array arguments and results are numpy arrays; packed weights are uint8
arrays holding raw GGUF blocks.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
Q8_0, Q4_K, Q6_K, MXFP4, Q5_K, Q4_0 = 0, 1, 2, 3, 4, 5   # Q5_K: no encoder (see synth_q5_K)
FMT_NAMES = {Q8_0: "q8_0", Q4_K: "q4_K", Q6_K: "q6_K", MXFP4: "mxfp4", Q5_K: "q5_K", Q4_0: "q4_0"}
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q6_K: 256, MXFP4: 32, Q5_K: 256, Q4_0: 32}
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q6_K: 210, MXFP4: 17, Q5_K: 176, Q4_0: 18}
Q8_1X_BYTES, Q8_1S_BYTES = 40, 48


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is mounted)."""
    so = os.path.join(_HERE, "libmxq_oracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-s", "-B" if force else "-s"])
    return so


def _load():
    so = os.path.join(_HERE, "libmxq_oracle.so")
    if not os.path.exists(so):
        build()
    return C.CDLL(so)


_lib = _load()
_vp, _u32, _u64, _i64, _sz, _f = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int64, C.c_size_t, C.c_float


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype, fn.argtypes = res, list(args)
    return fn


_fp16_to_fp32_n = _sig("orc_fp16_to_fp32_n", None, _vp, _vp, _sz)
_fp32_to_fp16_n = _sig("orc_fp32_to_fp16_n", None, _vp, _vp, _sz)
_rng_normal = _sig("orc_rng_normal", None, _u64, _u64, _sz, _f, _f, _vp)
_rng_uniform = _sig("orc_rng_uniform", None, _u64, _u64, _sz, _f, _f, _vp)
_rng_bytes = _sig("orc_rng_bytes", None, _u64, _u64, _sz, _vp)
_gsm = _sig("orc_get_scale_min_k4", None, C.c_int, _vp, _vp, _vp)
_dequant = _sig("orc_dequant", None, C.c_int, _vp, _sz, _vp)
_dequant_bt = _sig("orc_dequant_to_Bt", None, C.c_int, _vp, _u32, _u32, _vp)
_quant_rows = _sig("orc_quantize_rows", None, C.c_int, _vp, _vp, _i64, _i64)
_q8_1 = _sig("orc_quantize_q8_1", None, _vp, _vp, _i64)
_q8_1s = _sig("orc_quantize_q8_1s", None, _vp, _vp, _i64)
_gemv_f32 = _sig("orc_gemv_f32chain", None, C.c_int, _vp, _vp, _vp, _u32, _u32, _u32)
_gemv_f64 = _sig("orc_gemv_f64", None, C.c_int, _vp, _vp, _vp, _u32, _u32, _u32, C.c_int)
_gemv_q8 = _sig("orc_gemv_q8chain", None, C.c_int, _vp, _vp, _vp, _u32, _u32, _u32)
_gemv_q8s = _sig("orc_gemv_q8schain", None, C.c_int, _vp, _vp, _vp, _u32, _u32, _u32)
_int_codes = _sig("orc_int_codes", None, C.c_int, _vp, _u32, _vp)
_route = _sig("orc_route_from_logits", None, _vp, _u32, _u32, _vp, _vp)
_pack = _sig("orc_build_moe_packing", None, _vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp)
_rp_mx = _sig("orc_repack_mxfp4_to_soa", None, _vp, _sz, _vp, _vp)
_rp_q8 = _sig("orc_repack_q8_0_to_soa", None, _vp, _sz, _vp, _vp)
_swiglu = _sig("orc_swiglu", _f, _f, _f)
_swiglu_oai = _sig("orc_swiglu_oai", _f, _f, _f, _f, _f)
e8m0_half = _sig("orc_e8m0_half", _f, C.c_uint8)


def _p(a):
    return a.ctypes.data_as(_vp)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ---------------------------------------------------------------- fp16 / rng
def fp16_to_fp32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    _fp16_to_fp32_n(_p(h), _p(out), h.size)
    return out


def fp32_to_fp16(f):
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    _fp32_to_fp16_n(_p(f), _p(out), f.size)
    return out


def round_fp16(f):
    return fp16_to_fp32(fp32_to_fp16(f))


def normal(seed, shape, mean=0.0, std=1.0, offset=0):
    out = np.empty(shape, np.float32)
    _rng_normal(seed, offset, out.size, mean, std, _p(out))
    return out


def uniform(seed, shape, lo=0.0, hi=1.0, offset=0):
    out = np.empty(shape, np.float32)
    _rng_uniform(seed, offset, out.size, lo, hi, _p(out))
    return out


def rand_bytes(seed, n, offset=0):
    out = np.empty(n, np.uint8)
    _rng_bytes(seed, offset, n, _p(out))
    return out


# ---------------------------------------------------------------- formats
def get_scale_min_k4(j, scales12):
    s = _c(scales12, np.uint8)
    sc, mn = C.c_uint8(), C.c_uint8()
    _gsm(j, _p(s), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


def row_bytes(fmt, K):
    return K // BLOCK_ELEMS[fmt] * BLOCK_BYTES[fmt]


def dequant(fmt, packed, n_elems=None):
    packed = _c(packed, np.uint8)
    if n_elems is None:
        n_elems = packed.size // BLOCK_BYTES[fmt] * BLOCK_ELEMS[fmt]
    out = np.empty(n_elems, np.float32)
    _dequant(fmt, _p(packed), n_elems, _p(out))
    return out


def dequant_to_Bt(fmt, packed, K, N):
    packed = _c(packed, np.uint8)
    out = np.empty((K, N), np.uint16)
    _dequant_bt(fmt, _p(packed), K, N, _p(out))
    return out


def quantize(fmt, x):
    """x: [rows, K] fp32 -> uint8 [rows, row_bytes]."""
    x = _c(x, np.float32)
    if x.ndim == 1:
        x = x[None, :]
    rows, K = x.shape
    assert K % BLOCK_ELEMS[fmt] == 0
    out = np.zeros((rows, row_bytes(fmt, K)), np.uint8)
    _quant_rows(fmt, _p(x), _p(out), rows, K)
    return out


def synth_q5_K(x, seed):
    """Valid Q5_K blocks for tests: the Q4_K encoding of x (header, scales, nibbles) plus seeded fifth bits.
    {d, dmin, scales[12], qh[32], qs[128]} (include/ie/quant_blocks.hpp:79-85).  -> uint8 [rows, K/256*176]."""
    b4 = quantize(Q4_K, x)
    rows = b4.shape[0]
    b4 = b4.reshape(-1, 144)
    qh = rand_bytes(seed, b4.shape[0] * 32).reshape(-1, 32)
    return np.concatenate([b4[:, :16], qh, b4[:, 16:]], axis=1).reshape(rows, -1)


def quantize_q8_1(x):
    """x fp32 (values already at the precision the kernel sees) -> uint8 [n/32*40]."""
    x = _c(x, np.float32).ravel()
    out = np.zeros(x.size // 32 * Q8_1X_BYTES, np.uint8)
    _q8_1(_p(x), _p(out), x.size)
    return out


def quantize_q8_1s(x):
    x = _c(x, np.float32).ravel()
    out = np.zeros(x.size // 32 * Q8_1S_BYTES, np.uint8)
    _q8_1s(_p(x), _p(out), x.size)
    return out


def q8_1_fields(buf):
    """Split a block_q8_1x stream into (d[nb], s[nb], qs[nb,32])."""
    b = _c(buf, np.uint8).reshape(-1, Q8_1X_BYTES)
    return (b[:, 0:4].copy().view(np.float32).ravel(), b[:, 4:8].copy().view(np.float32).ravel(),
            b[:, 8:40].copy().view(np.int8))


def q8_1s_fields(buf):
    b = _c(buf, np.uint8).reshape(-1, Q8_1S_BYTES)
    hdr = b[:, 0:16].copy().view(np.float32)
    return hdr[:, 0], hdr[:, 1], hdr[:, 2], hdr[:, 3], b[:, 16:48].copy().view(np.int8)


def int_codes(fmt, row, K):
    row = _c(row, np.uint8)
    out = np.empty(K, np.int8)
    _int_codes(fmt, _p(row), K, _p(out))
    return out


# ---------------------------------------------------------------- matmul references
def gemv_f32chain(fmt, W, x, K, N):
    """The reference's CPU path: fp32 dequant + sequential fp32 dot.  x [T,K] -> y [T,N] fp32."""
    W, x = _c(W, np.uint8), _c(x, np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], N), np.float32)
    _gemv_f32(fmt, _p(W), _p(x), _p(y), K, N, x.shape[0])
    return y


def gemv_f64(fmt, W, x, K, N, round_w_fp16=False):
    W, x = _c(W, np.uint8), _c(x, np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], N), np.float64)
    _gemv_f64(fmt, _p(W), _p(x), _p(y), K, N, x.shape[0], int(round_w_fp16))
    return y


def gemv_q8chain(fmt, W, xq8, K, N):
    """xq8: block_q8_1x stream of T rows -> y [T,N] fp64."""
    W, xq8 = _c(W, np.uint8), _c(xq8, np.uint8)
    T = xq8.size // (K // 32 * Q8_1X_BYTES)
    y = np.empty((T, N), np.float64)
    _gemv_q8(fmt, _p(W), _p(xq8), _p(y), K, N, T)
    return y


def gemv_q8schain(fmt, W, xq8s, K, N):
    """xq8s: block_q8_1s stream of T rows -> y [T,N] fp64; the K-quant min terms use the stored half sums."""
    W, xq8s = _c(W, np.uint8), _c(xq8s, np.uint8)
    T = xq8s.size // (K // 32 * Q8_1S_BYTES)
    y = np.empty((T, N), np.float64)
    _gemv_q8s(fmt, _p(W), _p(xq8s), _p(y), K, N, T)
    return y


def swiglu(g, u):
    return np.array([_swiglu(float(a), float(b)) for a, b in zip(np.ravel(g), np.ravel(u))], np.float32).reshape(np.shape(g))


def swiglu_np(g, u):
    g64 = np.asarray(g, np.float64)
    return ((g64 / (1.0 + np.exp(-g64))).astype(np.float32) * np.asarray(u, np.float32)).astype(np.float32)


def swiglu_oai_np(g, u, alpha=1.702, limit=7.0):
    x = np.minimum(np.asarray(g, np.float32), np.float32(limit)).astype(np.float64)
    z = np.clip(np.asarray(u, np.float32), -limit, limit).astype(np.float32)
    return ((x / (1.0 + np.exp(alpha * -x))).astype(np.float32) * (z + np.float32(1.0))).astype(np.float32)


# ---------------------------------------------------------------- MoE
def route_from_logits(logits, k):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    ids = np.empty((T, k), np.int32)
    w = np.empty((T, k), np.float32)
    for t in range(T):
        _route(_p(logits[t]), E, k, _p(ids[t]), _p(w[t]))
    return ids, w


def build_moe_packing(topk_ids, topk_w, E):
    ids, w = _c(topk_ids, np.int32), _c(topk_w, np.float32)
    T, K = ids.shape
    off = np.empty(E + 1, np.uint32)
    sorted_idx = np.empty(T * K, np.int32)
    wp = np.empty(T * K, np.float32)
    tk2p = np.empty(T * K, np.int32)
    _pack(_p(ids), _p(w), T, K, E, _p(off), _p(sorted_idx), _p(wp), _p(tk2p))
    return off, sorted_idx, wp, tk2p


def repack_mxfp4_to_soa(blocks):
    blocks = _c(blocks, np.uint8).ravel()
    nb = blocks.size // 17
    qs, e = np.empty(nb * 16, np.uint8), np.empty(nb, np.uint8)
    _rp_mx(_p(blocks), nb, _p(qs), _p(e))
    return qs, e


def repack_q8_0_to_soa(blocks):
    blocks = _c(blocks, np.uint8).ravel()
    nb = blocks.size // 34
    qs, d = np.empty(nb * 32, np.int8), np.empty(nb, np.uint16)
    _rp_q8(_p(blocks), nb, _p(qs), _p(d))
    return qs, d


# ---------------------------------------------------------------- K-quant repacks (numpy restatements)
def repack_kquant_streams(fmt, bank, n_experts, nblocks_per_expert):
    """Per expert region: the nb blocks' fields gathered into per-field streams, region size unchanged.
    Q4_K: qs[128] x nb | scales[12] x nb | {d,dmin}[4] x nb; Q6_K: ql[128] x nb | qh[64] x nb |
    scales[16] x nb | d[2] x nb  (include/ie/quant_soa.hpp:33-51,127-157; with one region and
    nb = N*K/256 the Q4_K form is repack_q4_K_to_reorder, src/ops/gemv_q8dot.cpp:134-147).
    Pinned against the reference's own repack_moe_q{4,6}k_soa_host where oracle/_ref is built."""
    bs = BLOCK_BYTES[fmt]
    b = _c(bank, np.uint8).reshape(n_experts, nblocks_per_expert, bs)
    fields = [(16, 144), (4, 16), (0, 4)] if fmt == Q4_K else [(0, 128), (128, 192), (192, 208), (208, 210)]
    return np.concatenate([b[:, :, lo:hi].reshape(n_experts, -1) for lo, hi in fields], axis=1).ravel()


def q4_K_codes(W):
    """AoS Q4_K blocks -> (q [nb,256] uint8 natural order, sc [nb,8], mn [nb,8], d [nb] u16, dmin [nb] u16);
    element 64g + 32h + l is nibble h of qs[32g + l] (include/ie/dequant_ref.hpp:38-53)."""
    b = _c(W, np.uint8).reshape(-1, 144)
    qs = b[:, 16:].reshape(-1, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 256)
    s = b[:, 4:16]
    sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)], axis=1)    # get_scale_min_k4, all j at once
    mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], axis=1)
    return q, sc, mn, b[:, 0:2].copy().view(np.uint16).ravel(), b[:, 2:4].copy().view(np.uint16).ravel()


def q6_K_codes(W):
    """AoS Q6_K blocks -> (q6u [nb,256] uint8 in 0..63, natural order, sc [nb,16] int8, d [nb] u16);
    element 128h + 32s + l: low nibble = nibble (s>>1) of ql[64h + 32(s&1) + l], high bits
    (qh[32h + l] >> 2s) & 3 (include/ie/dequant_ref.hpp:78-96)."""
    b = _c(W, np.uint8).reshape(-1, 210)
    ql = b[:, :128].reshape(-1, 2, 2, 32)          # [nb, h, s&1, l]
    qh = b[:, 128:192].reshape(-1, 2, 1, 32)
    q = np.empty((b.shape[0], 2, 4, 32), np.uint8)
    for s_ in range(4):
        lo = (ql[:, :, s_ & 1] >> 4) if s_ & 2 else (ql[:, :, s_ & 1] & 15)
        q[:, :, s_] = lo | (((qh[:, :, 0] >> (2 * s_)) & 3) << 4)
    return q.reshape(-1, 256), b[:, 192:208].copy().view(np.int8), b[:, 208:210].copy().view(np.uint16).ravel()


def repack_q4_K_to_soa(W):
    """-> (q4_q, q4_sc, q4_mn, q4_d, q4_dmin): natural-order nibble plane (element k = nibble k&1 of byte
    k/2), unpacked per-32 scale / min, per-256 d / dmin (src/ops/gemv_q4_soa.cpp:18-28,115-151)."""
    q, sc, mn, d, dmin = q4_K_codes(W)
    return (q[:, 0::2] | (q[:, 1::2] << 4)).ravel(), sc.astype(np.int8).ravel(), mn.astype(np.int8).ravel(), d, dmin


def repack_q6_K_to_soa(W):
    """-> (q6_lo, q6_hi, q6_sc, q6_d): low nibbles two per byte, high bit pairs four per byte (element k =
    bits 2*(k&3) of byte k/4), per-16 int8 scales, per-256 d (src/ops/gemv_q6_soa.cpp:62-126)."""
    q, sc, d = q6_K_codes(W)
    lo, hi = q & 15, q >> 4
    return ((lo[:, 0::2] | (lo[:, 1::2] << 4)).ravel(), (hi[:, 0::4] | (hi[:, 1::4] << 2) | (hi[:, 2::4] << 4) | (hi[:, 3::4] << 6)).ravel(),
            sc.ravel(), d)


def dequant_q4_soa(planes):
    """value = (d * s_raw) * q4 - dmin * m_raw in fp32, element order natural (src/ops/gemv_q4_soa.cpp:30-35)."""
    q, sc, mn, d, dmin = planes
    codes = np.stack([q & 15, q >> 4], axis=1).reshape(-1, 256).astype(np.float32)
    d1 = (fp16_to_fp32(d)[:, None] * sc.reshape(-1, 8).astype(np.float32)).astype(np.float32)
    m1 = (fp16_to_fp32(dmin)[:, None] * mn.reshape(-1, 8).astype(np.float32)).astype(np.float32)
    return ((np.repeat(d1, 32, axis=1) * codes).astype(np.float32) - np.repeat(m1, 32, axis=1)).astype(np.float32).ravel()


def dequant_q6_soa(planes):
    """value = (d * sc) * (q6u - 32) in fp32 (src/ops/gemv_q6_soa.cpp:415-444)."""
    lo, hi, sc, d = planes
    l4 = np.stack([lo & 15, lo >> 4], axis=1).reshape(-1, 256)
    h2 = np.stack([(hi >> (2 * i)) & 3 for i in range(4)], axis=1).reshape(-1, 256)
    q = (l4 | (h2 << 4)).astype(np.int32) - 32
    ds = (fp16_to_fp32(d)[:, None] * sc.reshape(-1, 16).astype(np.float32)).astype(np.float32)
    return (np.repeat(ds, 16, axis=1) * q.astype(np.float32)).astype(np.float32).ravel()


# ---------------------------------------------------------------- the reference, where built
def load_ref():
    """oracle/_ref/libmxref.so (the reference's own host code) or None when it was not built."""
    so = os.path.join(_HERE, "_ref", "libmxref.so")
    if not os.path.exists(so):
        return None
    r = C.CDLL(so)
    r.ref_fp16_to_fp32.restype, r.ref_fp16_to_fp32.argtypes = _f, [C.c_uint16]
    r.ref_fp32_to_fp16.restype, r.ref_fp32_to_fp16.argtypes = C.c_uint16, [_f]
    r.ref_get_scale_min_k4.restype, r.ref_get_scale_min_k4.argtypes = None, [C.c_int, _vp, _vp, _vp]
    r.ref_dequant.restype, r.ref_dequant.argtypes = C.c_int, [C.c_int, _vp, _sz, _vp]
    r.ref_quantize_row_q4_K.restype, r.ref_quantize_row_q4_K.argtypes = None, [_vp, _vp, _i64]
    r.ref_quantize_row_q6_K.restype, r.ref_quantize_row_q6_K.argtypes = None, [_vp, _vp, _i64]
    r.ref_dp4a_us.restype, r.ref_dp4a_us.argtypes = C.c_int32, [_u32, C.c_int32, C.c_int32]
    r.ref_dp4a_ss.restype, r.ref_dp4a_ss.argtypes = C.c_int32, [C.c_int32, C.c_int32, C.c_int32]
    r.ref_build_moe_packing.restype = None
    r.ref_build_moe_packing.argtypes = [_vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]
    r.ref_repack_moe_q4k_soa.restype, r.ref_repack_moe_q4k_soa.argtypes = None, [_vp, _vp, _u32, _u64]
    r.ref_repack_moe_q6k_soa.restype, r.ref_repack_moe_q6k_soa.argtypes = None, [_vp, _vp, _u32, _u64]
    r.ref_gemv_cpu.restype, r.ref_gemv_cpu.argtypes = C.c_int, [C.c_int, _vp, _vp, _vp, _u32, _u32]
    return r


# ---------------------------------------------------------------- parity metrics
def parity(got, ref, abs_floor=0.0):
    """Metrics used by every parity test.

    abs_floor : extra absolute floor of the denominator; fp16 outputs use 2^-14 (the
              smallest normal half): below it the output format itself has absolute,
              not relative, precision.

    max_rel : max_i |g-r| / max(|r_i|, 1e-2*rms(r))  -- elementwise relative error
              with a floor at 1 % of the signal RMS (outputs that cancel to ~0 carry
              no relative information; the reference's own tests floor the
              denominator the same way: tests/unit/gemv_q4k_test.cpp:199-205,
              tests/unit/q8dot_test.cpp:112-135)
    cos     : cosine similarity
    max_abs_over_rms : max |g-r| / rms(r)
    n_under_rms_floor / n_under_abs_floor : elements whose |r| lies below 1 % of the RMS / below abs_floor
              (their error was divided by the floor, not by |r|)
    """
    g = np.asarray(got, np.float64).ravel()
    r = np.asarray(ref, np.float64).ravel()
    rms = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
    if rms == 0.0:
        return {"max_rel": float(np.max(np.abs(g))) if g.size else 0.0, "cos": 1.0, "max_abs_over_rms": 0.0, "rms": 0.0,
                "n": int(r.size), "n_under_rms_floor": int(r.size), "n_under_abs_floor": int(r.size)}
    err = np.abs(g - r)
    floor = max(1e-2 * rms, abs_floor)
    return {"max_rel": float(np.max(err / np.maximum(np.abs(r), floor))),
            "cos": float(np.dot(g, r) / (np.linalg.norm(g) * np.linalg.norm(r) + 1e-300)),
            "max_abs_over_rms": float(err.max() / rms), "rms": rms, "n": int(r.size),
            # how many elements were compared against a floored denominator instead of their own magnitude
            "n_under_rms_floor": int(np.sum(np.abs(r) < 1e-2 * rms)),
            "n_under_abs_floor": int(np.sum(np.abs(r) < abs_floor)) if abs_floor > 0 else 0}
