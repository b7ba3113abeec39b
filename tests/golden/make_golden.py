"""Writes tests/golden/ref_vectors.npz from the reference's own host code.

Run in a container where the reference tree is mounted and oracle/_ref was built
(`make -C oracle`).  Inputs come from the oracle's counter-based RNG (seeds
below); expected outputs come from oracle/_ref/libmxref.so, i.e. from
ie::ref::dequant_*, ie::quantize_row_q4_K/q6_K, ie::build_moe_packing, ie::repack_moe_q{4,6}k_soa_host,
ie::fp16_to_fp32/fp32_to_fp16 and ie::ref::get_scale_min_k4 compiled from the
reference sources.  Only data is stored: inputs and the reference's outputs.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle as O  # noqa: E402


def sane_blocks(fmt, seed, nb):
    """Random block bytes with the fp16 scale fields forced finite (exponent < 31)."""
    bb = O.BLOCK_BYTES[fmt]
    raw = O.rand_bytes(seed, nb * bb).reshape(nb, bb).copy()
    for off in {O.Q8_0: [1], O.Q4_K: [1, 3], O.Q6_K: [209], O.Q5_K: [1, 3]}[fmt]:
        raw[:, off] &= 0xBB  # clear one exponent bit: never Inf/NaN, keeps sign and subnormals
    return raw


def main():
    r = O.load_ref()
    if r is None:
        raise SystemExit("oracle/_ref/libmxref.so not built (reference tree not mounted?)")
    out = {}
    for fmt in (O.Q8_0, O.Q4_K, O.Q6_K, O.Q5_K):
        nb = 96
        raw = sane_blocks(fmt, 0xC0FFEE + fmt, nb)
        raw[0] = 0  # all-zero block
        n = nb * O.BLOCK_ELEMS[fmt]
        y = np.empty(n, np.float32)
        assert r.ref_dequant(fmt, raw.ctypes.data, n, y.ctypes.data) == 0
        out["deq_in_%s" % O.FMT_NAMES[fmt]] = raw
        out["deq_out_%s" % O.FMT_NAMES[fmt]] = y
    # encoders: N(0,0.02) rows plus edge rows
    x = O.normal(0x51CE, (12, 512), 0.0, 0.02)
    x[1, :256] = 0.0            # all-zero super-block
    x[2, 256:] = 0.0125         # constant block
    x[3] *= 1000.0              # large magnitude
    x[4, ::2] = 0.0             # half zeros
    x[5] = np.abs(x[5])         # all positive (min clamps to 0)
    x[6] = -np.abs(x[6])        # all negative
    x[7, 100] = 5.0             # outlier
    for fmt, fn in ((O.Q4_K, r.ref_quantize_row_q4_K), (O.Q6_K, r.ref_quantize_row_q6_K)):
        enc = np.zeros((x.shape[0], O.row_bytes(fmt, 512)), np.uint8)
        for i in range(x.shape[0]):
            fn(x[i].ctypes.data, enc[i].ctypes.data, 512)
        out["enc_out_%s" % O.FMT_NAMES[fmt]] = enc
    out["enc_in"] = x
    # scale/min unpack
    tabs = O.rand_bytes(0x5CA1E, 64 * 12).reshape(64, 12).copy()
    import ctypes as C
    sm = np.zeros((64, 8, 2), np.uint8)
    for i in range(64):
        for j in range(8):
            a, b = C.c_uint8(), C.c_uint8()
            r.ref_get_scale_min_k4(j, tabs[i].ctypes.data, C.byref(a), C.byref(b))
            sm[i, j] = (a.value, b.value)
    out["k4_in"], out["k4_out"] = tabs, sm
    # fp16 conversions: every half pattern that is not NaN; a fp32 sample incl. ties
    h = np.arange(65536, dtype=np.uint16)
    h = h[~np.isnan(h.view(np.float16))]
    out["h2f_in"] = h
    out["h2f_out"] = np.array([r.ref_fp16_to_fp32(int(v)) for v in h], np.float32)
    f = np.concatenate([O.normal(0xF16, 4096, 0, 1), O.normal(0xF17, 2048, 0, 1e-6), O.normal(0xF18, 2048, 0, 3e4),
                        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, 2.9802322e-8, 2.9802326e-8, 5.9604645e-8,
                                  6.1035156e-5, 6.0975552e-5, 1.0009766, 1.0004883, 1.0014648], np.float32)]).astype(np.float32)
    out["f2h_in"] = f
    out["f2h_out"] = np.array([r.ref_fp32_to_fp16(float(v)) for v in f], np.uint16)
    # MoE packing: T=9 tokens, top-3 of 7 experts (expert 5 unused)
    ids = np.array([[0, 2, 6], [1, 2, 3], [0, 1, 2], [2, 4, 6], [0, 3, 4], [1, 4, 6], [2, 3, 6], [0, 2, 4], [1, 2, 6]], np.int32)
    w = O.uniform(0x9AC, ids.shape, 0.05, 1.0)
    off = np.zeros(8, np.uint32)
    si, wp, t2p = np.zeros(27, np.int32), np.zeros(27, np.float32), np.zeros(27, np.int32)
    r.ref_build_moe_packing(ids.ctypes.data, w.ctypes.data, 9, 3, 7, off.ctypes.data, si.ctypes.data, wp.ctypes.data, t2p.ctypes.data)
    out.update(pack_ids=ids, pack_w=w, pack_off=off, pack_sorted=si, pack_wp=wp, pack_t2p=t2p)
    # dp4a
    a = O.rand_bytes(0xD4, 4 * 256).view(np.uint32).copy()
    b = O.rand_bytes(0xD5, 4 * 256).view(np.int32).copy()
    out["dp4a_a"], out["dp4a_b"] = a, b
    out["dp4a_us"] = np.array([r.ref_dp4a_us(int(x), int(y), 7) for x, y in zip(a, b)], np.int32)
    out["dp4a_ss"] = np.array([r.ref_dp4a_ss(int(np.int32(x)), int(y), -3) for x, y in zip(a.view(np.int32), b)], np.int32)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_vectors.npz")
    # per-expert stream repacks (ie::repack_moe_q4k_soa_host / _q6k_soa_host, include/ie/quant_soa.hpp:127-157)
    for fmt, fn in ((O.Q4_K, r.ref_repack_moe_q4k_soa), (O.Q6_K, r.ref_repack_moe_q6k_soa)):
        E, nb = 3, 20
        bank = O.rand_bytes(0x50A50A + fmt, E * nb * O.BLOCK_BYTES[fmt])
        soa = np.empty_like(bank)
        fn(bank.ctypes.data, soa.ctypes.data, E, nb)
        out["soa_in_%s" % O.FMT_NAMES[fmt]] = bank
        out["soa_out_%s" % O.FMT_NAMES[fmt]] = soa
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
