"""Pins the CPU oracle (oracle/mxq_oracle.c) before anything is compared with it:
against the golden vectors written from the reference's own host code
(tests/golden/ref_vectors.npz), against oracle/_ref where it is built, and
against closed forms / brute force for what those leave open."""
import numpy as np
import pytest

import oracle as O

FMTS3 = (O.Q8_0, O.Q4_K, O.Q6_K)
FMTS_REF = FMTS3 + (O.Q5_K,)   # formats the reference's host headers can dequantize


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ---------------------------------------------------------------- fp16
def test_fp16_to_fp32_exhaustive_vs_numpy_and_golden(golden):
    h = np.arange(65536, dtype=np.uint16)
    mine, npy = O.fp16_to_fp32(h), h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(npy)
    assert np.array_equal(bits(mine)[ok], bits(npy)[ok])
    assert np.isnan(mine[~ok]).all()
    assert np.array_equal(bits(O.fp16_to_fp32(golden["h2f_in"])), bits(golden["h2f_out"]))


def test_fp32_to_fp16_vs_numpy_ties_and_golden(golden):
    assert np.array_equal(O.fp32_to_fp16(golden["f2h_in"]), golden["f2h_out"])
    hf = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo, hi = O.fp16_to_fp32(hf).astype(np.float64), O.fp16_to_fp32(hf + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)  # exact: every midpoint fits fp32
    x = np.concatenate([mid, -mid, np.nextafter(mid, np.float32(1e9)), np.nextafter(mid, np.float32(-1e9)),
                        O.normal(11, 100000, 0, 1), O.normal(12, 50000, 0, 1e-5), O.normal(13, 50000, 0, 2e4)])
    with np.errstate(over="ignore"):
        assert np.array_equal(O.fp32_to_fp16(x), x.astype(np.float16).view(np.uint16))


# ---------------------------------------------------------------- dequant
@pytest.mark.parametrize("fmt", FMTS_REF)
def test_dequant_matches_reference_golden(golden, fmt):
    name = O.FMT_NAMES[fmt]
    assert np.array_equal(bits(O.dequant(fmt, golden["deq_in_" + name])), bits(golden["deq_out_" + name]))


@pytest.mark.parametrize("fmt", FMTS_REF)
def test_dequant_matches_ref_build_random(fmt):
    r = O.load_ref()
    if r is None:
        pytest.skip("oracle/_ref not built here")
    nb = 2048
    raw = O.rand_bytes(900 + fmt, nb * O.BLOCK_BYTES[fmt])
    n = nb * O.BLOCK_ELEMS[fmt]
    ref = np.empty(n, np.float32)
    r.ref_dequant(fmt, raw.ctypes.data, n, ref.ctypes.data)
    mine = O.dequant(fmt, raw)
    assert ((bits(mine) == bits(ref)) | (np.isnan(mine) & np.isnan(ref))).all()


def test_get_scale_min_k4_golden(golden):
    for tab, exp in zip(golden["k4_in"], golden["k4_out"]):
        for j in range(8):
            assert O.get_scale_min_k4(j, tab) == tuple(exp[j])


def test_dequant_closed_forms():
    # Q8_0: d = 1.0 -> y = q
    b = np.zeros(34, np.uint8)
    b[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    b[2:] = np.arange(-16, 16, dtype=np.int8).view(np.uint8)
    assert np.array_equal(O.dequant(O.Q8_0, b), np.arange(-16, 16, dtype=np.float32))
    # Q4_K: d = 0.5, dmin = 0.25, all scales 1 / mins 0 (j<4 bytes = 1, j>=4 low nibble 1) -> y = 0.5 * nibble
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([0x3800], np.uint16).view(np.uint8)
    b[2:4] = np.array([0x3400], np.uint16).view(np.uint8)
    b[4:8] = 1      # sc 0..3 = 1
    b[8:12] = 0     # m 0..3 = 0 ; high bits of sc/m 4..7 = 0
    b[12:16] = 1    # sc 4..7 = 1 (low nibble), m 4..7 = 0
    nib = (np.arange(256) * 7 + 3) % 16
    for e in range(256):
        g, hi, l = e // 64, (e // 32) % 2, e % 32
        b[16 + 32 * g + l] |= nib[e] << (4 * hi)
    assert np.array_equal(O.dequant(O.Q4_K, b), 0.5 * nib.astype(np.float32))
    # ... and with mins: sc=2, m=3 for sub-block 5 only: y = (0.5*2)*q - 0.25*3
    b[4 + 5 + 4] = 2 | (3 << 4)
    y = O.dequant(O.Q4_K, b)
    assert np.array_equal(y[160:192], 1.0 * nib[160:192] - 0.75)
    assert np.array_equal(y[:160], 0.5 * nib[:160].astype(np.float32))
    # Q5_K: same scales, d = 0.5: y = 0.5 * q5, the fifth bit of element 64g + 32hi + l in bit 2g + hi of qh[l]
    b5 = np.zeros(176, np.uint8)
    b5[0:2] = np.array([0x3800], np.uint16).view(np.uint8)
    b5[2:4] = np.array([0x3400], np.uint16).view(np.uint8)
    b5[4:8] = 1
    b5[12:16] = 1
    q5 = (np.arange(256) * 11 + 5) % 32
    for e in range(256):
        g, hi, l = e // 64, (e // 32) % 2, e % 32
        b5[48 + 32 * g + l] |= (q5[e] & 15) << (4 * hi)
        b5[16 + l] |= (q5[e] >> 4) << (2 * g + hi)
    assert np.array_equal(O.dequant(O.Q5_K, b5), 0.5 * q5.astype(np.float32))
    b5[4 + 2 + 4] = 3        # min of sub-block 2 = 3 -> y = 0.5 * q - 0.75 there only
    y = O.dequant(O.Q5_K, b5)
    assert np.array_equal(y[64:96], 0.5 * q5[64:96] - 0.75) and np.array_equal(y[:64], 0.5 * q5[:64].astype(np.float32))
    # Q6_K: d = 1, scales = 1 -> y = q - 32 with q the 6-bit code of element e
    b = np.zeros(210, np.uint8)
    b[192:208] = 1
    b[208:210] = np.array([0x3C00], np.uint16).view(np.uint8)
    code = (np.arange(256) * 37 + 11) % 64
    for e in range(256):
        h, sub, l = e // 128, (e // 32) % 4, e % 32
        b[64 * h + 32 * (sub & 1) + l] |= (code[e] & 15) << (4 * (sub >> 1))
        b[128 + 32 * h + l] |= (code[e] >> 4) << (2 * sub)
    assert np.array_equal(O.dequant(O.Q6_K, b), code.astype(np.float32) - 32)
    # per-16 scales: scale index 8h + 2sub + l/16
    b[192:208] = np.arange(1, 17, dtype=np.uint8)
    y = O.dequant(O.Q6_K, b)
    for e in (0, 15, 16, 31, 32, 100, 128, 200, 255):
        h, sub, l = e // 128, (e // 32) % 4, e % 32
        assert y[e] == (8 * h + 2 * sub + l // 16 + 1) * (code[e] - 32.0)


def test_mxfp4_closed_forms():
    """MXFP4 has no host routine in the reference headers; pinned by the format's
    definition: value = 2^(e-128) * {0,1,2,3,4,6,8,12} i.e. at e=127 the true E2M1
    table {0,.5,1,1.5,2,3,4,6}; e in {0,1} are fp32 denormals 2^-128, 2^-127
    (tests/mxfp4_dequant_test.cpp:37-64 exponent list)."""
    e2m1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], np.float32)
    for e in (0, 1, 2, 3, 64, 126, 127, 128, 200, 254, 255):
        assert O.e8m0_half(e) == 2.0 ** (e - 128)   # exact power of two, denormal for e < 2
        for seed in range(4):  # the reference test's make_block(e, seed) nibble pattern
            b = np.zeros(17, np.uint8)
            b[0] = e
            lo = (seed + np.arange(16)) & 15
            hi = (seed + np.arange(16) + 7) & 15
            b[1:] = lo | (hi << 4)
            y = O.dequant(O.MXFP4, b)
            with np.errstate(over="ignore"):  # e >= 254 overflows fp32 to inf for the large codes, as fp32 must
                exp = (np.concatenate([e2m1[lo], e2m1[hi]]).astype(np.float64) * 2.0 * 2.0 ** (e - 128)).astype(np.float32)
            assert np.array_equal(y, exp), (e, seed)
    assert O.e8m0_half(0) == 2.0 ** -128 and O.e8m0_half(1) == 2.0 ** -127 and O.e8m0_half(127) == 0.5


def test_q4_0_closed_forms_and_round_trip():
    """Q4_0 has no host routine in the reference; pinned by its definition (include/ie/quant_blocks.hpp:32-43,
    src/ops/gemv_q4_0.cpp:3-8): w[j] = d * ((qs[j] & 15) - 8), w[j+16] = d * ((qs[j] >> 4) - 8)."""
    b = np.zeros(18, np.uint8)
    b[0:2] = np.array([0x4000], np.uint16).view(np.uint8)       # d = 2.0
    b[2:] = (np.arange(16) | ((15 - np.arange(16)) << 4)).astype(np.uint8)
    y = O.dequant(O.Q4_0, b)
    assert np.array_equal(y[:16], 2.0 * (np.arange(16) - 8)) and np.array_equal(y[16:], 2.0 * (7 - np.arange(16)))
    # encoder (fixture generator): error at most |d|/2 except where x/d + 8 clamps at 15, and the extreme maps to code 0
    x = O.normal(77, (64, 256), 0.0, 0.02)
    w = O.quantize(O.Q4_0, x)
    yq = O.dequant(O.Q4_0, w).reshape(x.shape)
    d = np.abs(O.fp16_to_fp32(w.reshape(-1, 18)[:, :2].copy().view(np.uint16).ravel())).reshape(64, 8)
    err = np.abs(yq - x).reshape(64, 8, 32)
    inside = np.abs(x).reshape(64, 8, 32) <= 7.0 * d[:, :, None]          # codes 1..15 reach +-7 d; beyond that the code clamps
    tol = 2.0 ** -7                                                        # d is stored as fp16, the codes were chosen with the fp32 d
    assert (err <= d[:, :, None] * (1.0 + tol)).all() and (err[inside] <= (d[:, :, None] * (0.5 + tol) * np.ones_like(err))[inside]).all()
    codes = O.int_codes(O.Q4_0, w[0], 256)
    assert codes.min() >= -8 and codes.max() <= 7
    assert np.array_equal(codes.astype(np.float32) * np.repeat(O.fp16_to_fp32(w[0].reshape(-1, 18)[:, :2].copy().view(np.uint16).ravel()), 32), yq[0])
    # Q5_K codes: 5-bit code c with (d*sc)*c - dmin*m == dequant (include/ie/dequant_ref.hpp:55-75)
    w5 = O.synth_q5_K(O.normal(78, (1, 512), 0.0, 0.02), 79)
    c5 = O.int_codes(O.Q5_K, w5[0], 512).astype(np.int64)
    assert c5.min() >= 0 and c5.max() <= 31 and c5.max() > 15
    blk = w5[0].reshape(-1, 176)
    for b in range(2):
        d, dmin = O.fp16_to_fp32(blk[b, 0:4].copy().view(np.uint16))
        for j in range(8):
            sc, mn = O.get_scale_min_k4(j, blk[b, 4:16])
            exp = (np.float32(d) * np.float32(sc)) * c5[256 * b + 32 * j:256 * b + 32 * j + 32].astype(np.float32) - np.float32(dmin) * np.float32(mn)
            assert np.array_equal(exp.astype(np.float32), O.dequant(O.Q5_K, w5[0])[256 * b + 32 * j:256 * b + 32 * j + 32])


# ---------------------------------------------------------------- encoders
@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K))
def test_encoders_bit_identical_to_reference_golden(golden, fmt):
    assert np.array_equal(O.quantize(fmt, golden["enc_in"]), golden["enc_out_" + O.FMT_NAMES[fmt]])


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K))
def test_encoders_bit_identical_to_ref_build_large(fmt):
    r = O.load_ref()
    if r is None:
        pytest.skip("oracle/_ref not built here")
    x = O.normal(77 + fmt, (256, 1024), 0.0, 0.02)
    fn = r.ref_quantize_row_q4_K if fmt == O.Q4_K else r.ref_quantize_row_q6_K
    ref = np.zeros((256, O.row_bytes(fmt, 1024)), np.uint8)
    for i in range(256):
        fn(x[i].ctypes.data, ref[i].ctypes.data, 1024)
    assert np.array_equal(O.quantize(fmt, x), ref)


def test_encode_decode_error_bounds():
    # reference bounds: Q6_K max err < 2 % of absmax, Q4_K < 10 % (tests/quantize_q6k_test.cpp:53-54,78-79)
    x = O.normal(5, (32, 2048), 0.0, 0.02)
    for fmt, bound in ((O.Q6_K, 0.02), (O.Q4_K, 0.10), (O.Q8_0, 0.005), (O.MXFP4, 0.26)):
        y = O.dequant(fmt, O.quantize(fmt, x)).reshape(x.shape)
        assert np.abs(y - x).max() < bound * np.abs(x).max(), O.FMT_NAMES[fmt]
    z = np.zeros((1, 512), np.float32)
    for fmt in (O.Q8_0, O.Q4_K, O.Q6_K, O.MXFP4):
        assert not O.dequant(fmt, O.quantize(fmt, z)).any()


def test_q8_0_and_mxfp4_encoder_invariants():
    x = O.normal(6, (4, 256), 0.0, 0.02)
    q = O.quantize(O.Q8_0, x).reshape(-1, 34)
    d = O.fp16_to_fp32(q[:, :2].copy().view(np.uint16).ravel())
    qs = q[:, 2:].view(np.int8)
    assert np.abs(qs).max(axis=1).min() == 127          # amax element hits +-127
    xb = x.reshape(-1, 32)
    assert np.allclose(d, np.abs(xb).max(axis=1) / 127, rtol=1e-3)
    m = O.quantize(O.MXFP4, x).reshape(-1, 17)
    y = O.dequant(O.MXFP4, m).reshape(-1, 32)
    scale = np.array([O.e8m0_half(int(e)) for e in m[:, 0]])
    assert (np.abs(xb).max(axis=1) <= 12 * scale).all() and (np.abs(xb).max(axis=1) > 6 * scale).all()
    # nearest code: error at most half the largest code gap (2 units below 8, 4 above) -> <= 2*scale
    assert (np.abs(y - xb) <= 2.0 * scale[:, None] + 1e-12).all()


# ---------------------------------------------------------------- activation quantizers
def test_quantize_q8_1_invariants_and_rounding():
    x = O.round_fp16(O.normal(21, 32 * 64, 0.0, 1.0))
    x[32:64] = 0.0
    x[64:96] = np.linspace(-1, 1, 32, dtype=np.float32)
    d, s, q = O.q8_1_fields(O.quantize_q8_1(x))
    xb = x.reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    assert np.array_equal(d, (amax / np.float32(127.0)).astype(np.float32))
    assert np.abs(q).max() <= 127 and (np.abs(q).max(axis=1)[amax > 0] == 127).all()
    assert np.array_equal(s, d * q.sum(axis=1).astype(np.float32))
    assert d[1] == 0 and not q[1].any() and s[1] == 0
    inv = np.where(amax > 0, np.float32(127.0) / np.where(amax > 0, amax, 1), 0).astype(np.float32)
    v = (xb * inv[:, None]).astype(np.float32)
    exp = np.where(v >= 0, np.floor(v + np.float32(0.5)), -np.floor(-v + np.float32(0.5)))  # half away from zero
    assert np.array_equal(q.astype(np.float32), exp)
    # a tie: amax = 127 -> inv = 1, v = 2.5 -> 3 ; -2.5 -> -3
    t = np.zeros(32, np.float32)
    t[0], t[1], t[2] = 127.0, 2.5, -2.5
    assert tuple(O.q8_1_fields(O.quantize_q8_1(t))[2][0][:3]) == (127, 3, -3)
    d2, s0, s1, pad, q2 = O.q8_1s_fields(O.quantize_q8_1s(x))
    assert np.array_equal(d2, d) and np.array_equal(q2, q) and not pad.any()
    assert np.array_equal(s0, d * q[:, :16].sum(axis=1).astype(np.float32))
    assert np.array_equal(s1, d * q[:, 16:].sum(axis=1).astype(np.float32))


# ---------------------------------------------------------------- matmul references
@pytest.mark.parametrize("fmt", (O.Q8_0, O.Q4_K, O.Q6_K, O.MXFP4))
def test_reference_gemv_chains_brute_force(fmt):
    K, N, T = 512, 6, 2
    W = O.quantize(fmt, O.normal(31 + fmt, (N, K), 0.0, 0.02))
    x = O.round_fp16(O.normal(41, (T, K), 0.0, 1.0))
    Wd = O.dequant(fmt, W).reshape(N, K)
    # float chain: sequential fp32 dot, exactly as the reference test loops it
    y = O.gemv_f32chain(fmt, W, x, K, N)
    for t in range(T):
        for n in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + np.float32(x[t, k] * Wd[n, k]))
            assert y[t, n] == acc
    assert np.allclose(O.gemv_f64(fmt, W, x, K, N), x.astype(np.float64) @ Wd.astype(np.float64).T, rtol=1e-12, atol=1e-14)
    # q8 chain equals (dequant W) @ (d8 * q8) in fp64, and its integer part equals the brute-force int dot
    xq = O.quantize_q8_1(x)
    d8, _, q8 = O.q8_1_fields(xq)
    xdq = (d8[:, None].astype(np.float64) * q8.astype(np.float64)).reshape(T, K)
    assert np.allclose(O.gemv_q8chain(fmt, W, xq, K, N), xdq @ Wd.astype(np.float64).T, rtol=1e-12, atol=1e-14)
    codes = np.stack([O.int_codes(fmt, W[n], K) for n in range(N)]).astype(np.int64)
    # codes reproduce the dequantized values for the symmetric formats: W = scale * code
    if fmt in (O.Q8_0, O.MXFP4):
        scale = Wd.reshape(N, K // 32, 32)
        c = codes.reshape(N, K // 32, 32)
        nz = c != 0
        ratio = np.where(nz, scale / np.where(nz, c, 1), 0)
        assert all(len(set(r[m].tolist())) <= 1 for r, m in zip(ratio.reshape(-1, 32), nz.reshape(-1, 32)))
    # linearity in x
    y2 = O.gemv_f64(fmt, W, 2 * x, K, N)
    assert np.allclose(y2, 2 * O.gemv_f64(fmt, W, x, K, N), rtol=1e-12)


def test_gemv_identity_like_weights():
    # Q8_0 row n = one-hot at k=n with q=127, d=1/127 -> y[n] = x[n]
    K = N = 64
    Wf = np.eye(N, K, dtype=np.float32)
    W = O.quantize(O.Q8_0, Wf)
    x = O.round_fp16(O.normal(3, (1, K)))
    y = O.gemv_f64(O.Q8_0, W, x, K, N)[0]
    d = O.fp16_to_fp32(np.array([O.fp32_to_fp16(np.float32(1 / 127))]))[0]
    assert np.allclose(y, x[0].astype(np.float64) * float(d) * 127, rtol=1e-12)


# ---------------------------------------------------------------- MoE host logic
def test_route_from_logits_textbook():
    logits = O.normal(55, (16, 32))
    ids, w = O.route_from_logits(logits, 4)
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    for t in range(16):
        top = np.sort(np.argsort(-p[t], kind="stable")[:4])
        assert np.array_equal(ids[t], top)
        assert np.allclose(w[t], p[t, top] / p[t, top].sum(), rtol=1e-5)
        assert abs(w[t].sum() - 1) < 1e-5


def test_build_moe_packing_golden_and_invariants(golden):
    off, si, wp, t2p = O.build_moe_packing(golden["pack_ids"], golden["pack_w"], 7)
    assert np.array_equal(off, golden["pack_off"]) and np.array_equal(si, golden["pack_sorted"])
    assert np.array_equal(wp, golden["pack_wp"]) and np.array_equal(t2p, golden["pack_t2p"])
    # invariants on a larger random routing
    T, K, E = 200, 8, 128
    ids = np.stack([np.sort(np.argsort(O.uniform(1000 + t, E))[:K]) for t in range(T)]).astype(np.int32)
    w = O.uniform(7, (T, K), 0.1, 1.0)
    off, si, wp, t2p = O.build_moe_packing(ids, w, E)
    assert off[0] == 0 and off[-1] == T * K and (np.diff(off.astype(np.int64)) >= 0).all()
    assert sorted(t2p.tolist()) == list(range(T * K))
    for e in range(E):
        seg = si[off[e]:off[e + 1]]
        assert (np.diff(seg) >= 0).all()            # stable: token order kept inside an expert
        assert all(e in ids[t] for t in seg)
    assert np.array_equal(wp[t2p], w.ravel()) and np.array_equal(si[t2p], np.repeat(np.arange(T), K))
    r = O.load_ref()
    if r is not None:
        o2, s2, w2, p2 = np.zeros(E + 1, np.uint32), np.zeros(T * K, np.int32), np.zeros(T * K, np.float32), np.zeros(T * K, np.int32)
        r.ref_build_moe_packing(ids.ctypes.data, w.ctypes.data, T, K, E, o2.ctypes.data, s2.ctypes.data, w2.ctypes.data, p2.ctypes.data)
        assert np.array_equal(off, o2) and np.array_equal(si, s2) and np.array_equal(wp, w2) and np.array_equal(t2p, p2)


def test_repacks_reconstruct():
    x = O.normal(8, (3, 128), 0, 0.02)
    for fmt, rp, plane in ((O.MXFP4, O.repack_mxfp4_to_soa, 16), (O.Q8_0, O.repack_q8_0_to_soa, 32)):
        blk = O.quantize(fmt, x).reshape(-1, O.BLOCK_BYTES[fmt])
        qs, hd = rp(blk)
        if fmt == O.MXFP4:
            assert np.array_equal(hd, blk[:, 0]) and np.array_equal(qs.reshape(-1, 16), blk[:, 1:])
        else:
            assert np.array_equal(hd, blk[:, :2].copy().view(np.uint16).ravel())
            assert np.array_equal(qs.reshape(-1, 32).view(np.uint8), blk[:, 2:])


def test_dp4a_semantics_golden(golden):
    """The int dot used by the kernels (4 x int8 products + c) against the reference's dp4a_us / dp4a_ss."""
    a, b = golden["dp4a_a"], golden["dp4a_b"]
    ab = a.view(np.uint8).reshape(-1, 4).astype(np.int64)
    bs = b.view(np.int8).reshape(-1, 4).astype(np.int64)
    assert np.array_equal((ab * bs).sum(axis=1) + 7, golden["dp4a_us"])
    assert np.array_equal((a.view(np.int8).reshape(-1, 4).astype(np.int64) * bs).sum(axis=1) - 3, golden["dp4a_ss"])


# ---------------------------------------------------------------- activation epilogues
def _both_swiglu(g, u):
    """The C and the numpy restatement of swiglu on the same scalars."""
    return float(O.swiglu([g], [u])[0]), float(O.swiglu_np(np.float32([g]), np.float32([u]))[0])


def _both_oai(g, u, alpha=1.702, limit=7.0):
    return (float(O._swiglu_oai(float(g), float(u), float(alpha), float(limit))),
            float(O.swiglu_oai_np(np.float32([g]), np.float32([u]), alpha, limit)[0]))


def test_swiglu_known_answers():
    """swiglu = (g * sigmoid(g)) * u (src/ops/elementwise.cpp:449-466).  Expected values are literals
    (sigmoid(1) = 0.7310585786300049, ...), not a retyped formula: a dropped factor, sigmoid(-g) for
    sigmoid(g) or swapped operands each fail one line."""
    cases = [((0.0, 3.0), 0.0),                        # silu(0) = 0 whatever u
             ((1.0, 1.0), 0.7310585786300049),          # silu(1)
             ((1.0, -2.0), -1.4621171572600098),        # linear in u, sign kept
             ((-1.0, 2.0), -0.5378828427399902),        # silu(-1) = -0.26894142..., not +
             ((30.0, 0.5), 15.0),                       # large gate: g * u
             ((-30.0, 1.0), -2.8072868906517896e-12),   # large negative gate: -> -0
             ((2.0, 0.0), 0.0)]
    for (g, u), want in cases:
        for got in _both_swiglu(g, u):
            assert got == pytest.approx(want, rel=2e-6, abs=1e-18), (g, u, got, want)
    # not symmetric in its operands
    assert _both_swiglu(2.0, 1.0)[0] != pytest.approx(_both_swiglu(1.0, 2.0)[0], rel=1e-3)


def test_swiglu_oai_known_answers():
    """swiglu_oai: x = min(gate, limit) (clamped ABOVE only), z = clamp(up, -limit, limit),
    out = (x * sigmoid(alpha x)) * (z + 1), alpha = 1.702, limit = 7 (src/ops/elementwise.cpp:468-492)."""
    x7 = 6.999953128303318        # 7 * sigmoid(1.702 * 7)
    cases = [((8.0, 0.0), x7),                          # gate above the limit -> x = 7 exactly
             ((7.0, 0.0), x7),
             ((100.0, 0.0), x7),
             ((-8.0, 0.0), -9.766428865730381e-06),     # gate below -limit is NOT clamped (clamped would give -4.687e-05)
             ((8.0, 8.0), x7 * 8.0),                    # up above the limit -> z = 7, factor 8
             ((8.0, -8.0), x7 * -6.0),                  # up below -limit -> z = -7, factor -6
             ((8.0, 100.0), x7 * 8.0),
             ((3.0, -1.0), 0.0),                        # z + 1 = 0
             ((1.0, 0.0), 0.8457957659328212),          # sigmoid(1.702): pins alpha
             ((0.5, 1.0), 2 * 0.35038843660638014),     # (z + 1) = 2
             ((-2.5, 0.5), 1.5 * -0.03498616504857008),
             ((0.0, 5.0), 0.0)]
    for (g, u), want in cases:
        for got in _both_oai(g, u):
            assert got == pytest.approx(want, rel=2e-6, abs=1e-12), (g, u, got, want)
    # the one-sided clamp, side by side: a two-sided clamp of the gate would make these two equal
    lo8, lo7 = _both_oai(-8.0, 0.0)[1], _both_oai(-7.0, 0.0)[1]
    assert lo7 == pytest.approx(-4.687169668280189e-05, rel=2e-6) and abs(lo8) < 0.25 * abs(lo7)
    # alpha and limit are arguments, not constants: alpha = 1 gives plain sigmoid, limit = 2 clamps at 2
    for got in _both_oai(1.0, 0.0, alpha=1.0):
        assert got == pytest.approx(0.7310585786300049, rel=2e-6)
    for got in _both_oai(5.0, 9.0, alpha=1.702, limit=2.0):
        assert got == pytest.approx(2.0 / (1.0 + 0.03324004351101861) * 3.0, rel=2e-6)   # exp(-1.702 * 2) = 0.0332400435110


def test_swiglu_c_and_numpy_forms_agree():
    g, u = O.normal(71, 4000, 0, 6), O.normal(72, 4000, 0, 6)
    assert np.allclose(O.swiglu(g, u), O.swiglu_np(g, u), rtol=3e-7, atol=0)
    c = np.float32([O._swiglu_oai(float(a), float(b), 1.702, 7.0) for a, b in zip(g, u)])
    assert np.allclose(c, O.swiglu_oai_np(g, u), rtol=2e-6, atol=0)   # alpha is a float in C, a double in numpy
    assert (np.abs(g) > 7).sum() > 100 and (g < -7).sum() > 30 and (np.abs(u) > 7).sum() > 100   # both clamps exercised


# ---------------------------------------------------------------- q8_1s chain (stored half sums)
def _q8s_rows(x):
    """fp32 rows [T, K] -> (block_q8_1s stream, block_q8_1x stream) of the same quants."""
    return (np.concatenate([O.quantize_q8_1s(r) for r in x]), np.concatenate([O.quantize_q8_1(r) for r in x]))


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0, O.MXFP4, O.Q4_0))
def test_q8schain_equals_q8chain_on_quantizer_output(fmt):
    """The quantizer stores s0 + s1 = d * sum(q) up to fp32 rounding, so both chains give the same sums to ~1e-6."""
    K, N, T = 512, 24, 3
    x = O.round_fp16(O.normal(500 + fmt, (T, K)))
    W = O.quantize(fmt, O.normal(510 + fmt, (N, K), 0, 0.02))
    xs, xx = _q8s_rows(x)
    a, b = O.gemv_q8schain(fmt, W, xs, K, N), O.gemv_q8chain(fmt, W, xx, K, N)
    rms = np.sqrt(np.mean(b * b))
    assert np.abs(a - b).max() <= 2e-6 * rms, (fmt, np.abs(a - b).max() / rms)


def test_q8schain_uses_the_stored_sums():
    """Doctored sums that no quantizer would write show which field the min term reads."""
    K, N = 256, 1
    # Q4_K: every scale 0, every min 1, d = dmin = 1  ->  weight = -1 everywhere, y = -(sum over blocks of s0 + s1)
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[4 + 4:4 + 8] = 1                 # mins of sub-blocks 0..3 (low 6 bits of bytes 4..7)
    blk[4 + 8:4 + 12] = 1 << 4           # mins of sub-blocks 4..7 (high nibbles of bytes 8..11)
    assert np.array_equal(O.dequant(O.Q4_K, blk), np.full(256, -1.0, np.float32))
    xs = np.zeros((8, 48), np.uint8)
    hdr = np.zeros((8, 4), np.float32)
    hdr[:, 0] = 0.5                                         # d8 (irrelevant: the scales are 0)
    hdr[:, 1] = np.arange(8) + 1.0                          # s0 = 1..8
    hdr[:, 2] = 100.0 * (np.arange(8) + 1.0)                # s1 = 100..800
    hdr[:, 3] = 1e9                                         # pad: never read
    xs[:, :16] = hdr.view(np.uint8)
    xs[:, 16:] = 3                                          # quants: multiplied by scale 0
    assert O.gemv_q8schain(O.Q4_K, blk, xs.ravel(), K, N)[0, 0] == -(36.0 + 3600.0)
    # Q6_K: d = 1, every scale 1, all codes 0 (value -32)  ->  y = sum over 16-groups of (d8 * 0 - 32 * s_half)
    b6 = np.zeros(210, np.uint8)
    b6[192:208] = 1
    b6[208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    assert np.array_equal(O.dequant(O.Q6_K, b6), np.full(256, -32.0, np.float32))
    assert O.gemv_q8schain(O.Q6_K, b6, xs.ravel(), K, N)[0, 0] == -32.0 * (36.0 + 3600.0)
    # per-group scale indexing: scale 2 on the second half of block 3 only
    b6[192 + 3 * 2 + 1] = 2
    assert O.gemv_q8schain(O.Q6_K, b6, xs.ravel(), K, N)[0, 0] == -32.0 * (36.0 + 3600.0 + 400.0)
    # and the integer part: one quant 1 facing code 0 (u = 0): nothing; code 5 in element 0 of block 0: d8 * 5 * q
    b6[0] = 5
    xs[0, 16] = 7
    assert O.gemv_q8schain(O.Q6_K, b6, xs.ravel(), K, N)[0, 0] == -32.0 * (36.0 + 3600.0 + 400.0) + 0.5 * 5 * 7
