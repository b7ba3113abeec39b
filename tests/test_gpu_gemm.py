"""GPU parity: prefill quant-GEMM on the matrix cores (BASELINE config 3) and the
expert-grouped GEMM (config 5) against the oracle: fp16 activations times
fp16-rounded dequantized weights, accumulated in fp64 (the reference's XMX /
dequant+GEMM arithmetic, src/ops/gemm_q4k_xmx.cpp:107-108).  Gate 1e-3 / 0.99999."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host, weights

pytestmark = pytest.mark.gpu


def f16(a):
    return O.round_fp16(np.asarray(a, np.float32))


@pytest.mark.parametrize("M,K,N", [(128, 256, 256), (1, 512, 64), (300, 1024, 520), (129, 768, 33), (512, 4096, 1024)])
def test_gemm_q4_K(mx, M, K, N):
    if K % 256:
        K = K // 256 * 256
    W = weights(O.Q4_K, 2000 + N, N, K)
    A = f16(O.normal(2001 + M, (M, K)))
    ref = O.gemv_f64(O.Q4_K, W, A, K, N, round_w_fp16=True)
    got = host(mx.ops.gemm_q4_K(dev(A).half(), dev(W), M, K, N)).astype(np.float32)
    check(got, ref, "gemm_q4_K M=%d K=%d N=%d" % (M, K, N))
    # equals M independent GEMVs on the same rounded weights (rows are independent)
    if M >= 2:
        one = host(mx.ops.gemm_q4_K(dev(A[1:2]).half(), dev(W), 1, K, N)).astype(np.float32)
        check(one[0], ref[1], "row 1 alone")


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
@pytest.mark.parametrize("M,K,N", [(8, 4096, 512), (64, 2048, 260), (200, 3072, 768), (512, 7168, 256)])
def test_gemm_k_slices(mx, fmt, M, K, N):
    """Launches with too few output tiles for the chip run as K slices plus a launch that adds the slices in order:
    4 slices of 128-token tiles (M <= 64), 2..8 slices of 64-token tiles, a last slice shorter than the others
    (K = 3072: 24 chunks in 3 slices; K = 7168: 56 chunks in 7).  Against the oracle, and the same bits from launch to launch."""
    W = weights(fmt, 2100 + N, N, K)
    A = f16(O.normal(2101 + M, (M, K)))
    ref = O.gemv_f64(fmt, W, A, K, N, round_w_fp16=True)
    fn = getattr(mx.ops, "gemm_%s" % O.FMT_NAMES[fmt])
    a_d, w_d = dev(A).half(), dev(W)
    got = fn(a_d, w_d, M, K, N)
    check(host(got).astype(np.float32), ref, "gemm %s M=%d K=%d N=%d" % (O.FMT_NAMES[fmt], M, K, N))
    for _ in range(3):
        assert torch.equal(fn(a_d, w_d, M, K, N), got), "K-sliced GEMM differs from launch to launch"


@pytest.mark.parametrize("M,K,N", [(128, 128, 256), (260, 768, 2048), (77, 2048, 768)])
def test_gemm_q8_0_soa(mx, M, K, N):
    W = weights(O.Q8_0, 2100 + N, N, K)
    qs, d = O.repack_q8_0_to_soa(W)
    A = f16(O.normal(2101 + M, (M, K)))
    ref = O.gemv_f64(O.Q8_0, W, A, K, N, round_w_fp16=True)
    got = host(mx.ops.gemm_q8_0_soa(dev(A).half(), dev(qs), dev(d), M, K, N)).astype(np.float32)
    check(got, ref, "gemm_q8_0_soa M=%d K=%d N=%d" % (M, K, N))


def onehot_weights_through_gemm(gemm, K, N):
    """A = rows of the identity: Y[t, n] is the kernel's own fp16 weight W16[n, k0 + t]."""
    out = np.zeros((N, K), np.float32)
    for k0 in range(0, K, 128):
        n = min(128, K - k0)
        A = np.zeros((128, K), np.float32)
        A[np.arange(n), k0 + np.arange(n)] = 1.0
        out[:, k0:k0 + n] = host(gemm(dev(A).half())).astype(np.float32).T[:, :n]
    return out


def q5k_blocks(seed, N, K):
    """Q5_K blocks from Q4_K ones: same header and nibbles, seeded high bits (the oracle has no Q5_K quantizer)."""
    b4 = O.quantize(O.Q4_K, O.normal(seed, (N, K), 0.0, 0.02)).reshape(-1, 144)
    return np.ascontiguousarray(np.concatenate([b4[:, :16], O.rand_bytes(seed + 1, b4.shape[0] * 32).reshape(-1, 32), b4[:, 16:]], axis=1)).reshape(-1)


@pytest.mark.parametrize("fmt,K", [("q4_K", 512), ("q6_K", 512), ("q8_0", 256), ("q5_K", 512), ("mxfp4", 320)])
def test_gemm_weight_fragments_bit_exact(mx, fmt, K):
    """The fp16 weights the GEMM multiplies by equal half(reference dequant) element for element
    (include/ie/dequant_ref.hpp), read back through one-hot activations.  MXFP4 at K = 320: the row ends half way
    through its last 128-element chunk, as K = 2880 does."""
    F = {"q4_K": O.Q4_K, "q6_K": O.Q6_K, "q8_0": O.Q8_0, "q5_K": O.Q5_K, "mxfp4": O.MXFP4}[fmt]
    N = 256
    if fmt == "q5_K":
        W = q5k_blocks(2300, N, K)
    elif fmt == "mxfp4":
        W = O.quantize(F, O.normal(2300, (N, K), 0.0, 0.02))
        # a few blocks at exponents where half(value) is zero, subnormal or near the top of the fp16 range (finite: a
        # weight that is inf would turn the one-hot read-back of its whole row into nan)
        Wb = W.reshape(-1, 17)
        Wb[:8, 0] = np.array([0, 1, 100, 112, 126, 127, 139, 140], np.uint8)
    else:
        W = weights(F, 2300, N, K)
    ref = f16(O.dequant(F, W, N * K).reshape(N, K))
    if fmt == "mxfp4":
        qs, e = O.repack_mxfp4_to_soa(W)
        fn = lambda A, _W, M, K_, N_: mx.ops.gemm_mxfp4_soa(A, dev(qs), dev(e), M, K_, N_)
    else:
        fn = {"q4_K": mx.ops.gemm_q4_K, "q6_K": mx.ops.gemm_q6_K, "q8_0": mx.ops.gemm_q8_0, "q5_K": mx.ops.gemm_q5_K}[fmt]
    got = onehot_weights_through_gemm(lambda A: fn(A, dev(W), 128, K, N), K, N)
    # value equality: a zero weight may come out as +0 where the reference expression gives -0
    # (Q6_K code 32 under a negative scale); the sign of a zero cannot change a dot product
    n_bad = int((got != ref.astype(np.float32)).sum())
    assert n_bad == 0, "%d of %d weights differ" % (n_bad, got.size)
    if fmt == "q8_0":
        qs, d = O.repack_q8_0_to_soa(W)
        got = onehot_weights_through_gemm(lambda A: mx.ops.gemm_q8_0_soa(A, dev(qs), dev(d), 128, K, N), K, N)
        assert np.array_equal(got, ref.astype(np.float32))


@pytest.mark.parametrize("M,K,N", [(128, 256, 256), (1, 512, 64), (300, 1024, 520), (129, 768, 33), (512, 4096, 1024)])
def test_gemm_q6_K(mx, M, K, N):
    W = weights(O.Q6_K, 2200 + N, N, K)
    A = f16(O.normal(2201 + M, (M, K)))
    ref = O.gemv_f64(O.Q6_K, W, A, K, N, round_w_fp16=True)
    got = host(mx.ops.gemm_q6_K(dev(A).half(), dev(W), M, K, N)).astype(np.float32)
    check(got, ref, "gemm_q6_K M=%d K=%d N=%d" % (M, K, N))


@pytest.mark.parametrize("M,K,N", [(128, 128, 256), (260, 768, 2048), (77, 2048, 768)])
def test_gemm_q8_0_aos(mx, M, K, N):
    W = weights(O.Q8_0, 2100 + N, N, K)
    A = f16(O.normal(2101 + M, (M, K)))
    ref = O.gemv_f64(O.Q8_0, W, A, K, N, round_w_fp16=True)
    got = host(mx.ops.gemm_q8_0(dev(A).half(), dev(W), M, K, N)).astype(np.float32)
    check(got, ref, "gemm_q8_0 M=%d K=%d N=%d" % (M, K, N))
    qs, d = O.repack_q8_0_to_soa(W)
    soa = host(mx.ops.gemm_q8_0_soa(dev(A).half(), dev(qs), dev(d), M, K, N)).astype(np.float32)
    assert np.array_equal(got, soa), "AoS and SoA entry points multiply the same fp16 weights in the same order"


def test_gemm_rejects_bad_shapes(mx):
    A = torch.zeros((4, 300), dtype=torch.float16, device="cuda")
    W = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    with pytest.raises(mx.MxError):
        mx.ops.gemm_q4_K(A, W, 4, 300, 4)     # K % 256 != 0: the reference would silently do nothing


def zipf_routing(seed, T, E, Kt, s=1.1):
    """Expert popularity ~ rank^-s (seeded permutation of ranks), Kt distinct experts per token
    sampled without replacement, router weights from a seeded softmax; ascending expert id per token."""
    rng = np.random.default_rng(seed)
    p = (np.arange(1, E + 1, dtype=np.float64) ** -s)
    p = p[rng.permutation(E)]
    p /= p.sum()
    ids = np.stack([np.sort(rng.choice(E, size=Kt, replace=False, p=p)) for _ in range(T)]).astype(np.int32)
    lg = O.normal(seed + 1, (T, Kt))
    w = np.exp(lg - lg.max(axis=1, keepdims=True))
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return ids, w


@pytest.mark.parametrize("T,E,Kt,H,EF", [(64, 8, 2, 256, 128), (300, 16, 4, 512, 384), (512, 128, 8, 256, 128)])
def test_moe_grouped_gemm_q8(mx, T, E, Kt, H, EF):
    """Qwen3-MoE style layer at reduced size: Zipf(1.1) routing gives experts with 0, 1 and hundreds of rows."""
    ops = mx.ops
    mk = lambda seed, N, K: np.stack([O.quantize(O.Q8_0, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
    Wg, Wu, Wd = mk(3000, EF, H), mk(4000, EF, H), mk(5000, H, EF)
    gq, gd = O.repack_q8_0_to_soa(Wg)
    uq, ud = O.repack_q8_0_to_soa(Wu)
    dq, dd = O.repack_q8_0_to_soa(Wd)
    x = f16(O.normal(6000, (T, H)))
    ids, w = zipf_routing(7000, T, E, Kt)
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    TK = T * Kt
    counts = np.diff(off.astype(np.int64))
    print("rows per expert: min %d max %d, empty %d" % (counts.min(), counts.max(), (counts == 0).sum()))
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, H)
    hp = ops.moe_gemm_gate_up_silu_q8(xp, dev(gq), dev(gd), dev(uq), dev(ud), EF * H, EF * H // 32, dev(off), TK, E, H, EF)
    # the gather folded into the row loads: the unsorted rows and the sorted -> source index, the same bits
    hp_g = ops.moe_gemm_gate_up_silu_q8(dev(x).half(), dev(gq), dev(gd), dev(uq), dev(ud), EF * H, EF * H // 32, dev(off), TK, E, H, EF, sorted_idx=dev(si))
    assert torch.equal(hp_g, hp), "gather form differs from gather_rows + grouped GEMM"
    hp_h = host(hp).astype(np.float32)
    xs = x[si]
    h_ref = np.zeros((TK, EF), np.float32)
    for e in range(E):
        if counts[e]:
            rows = slice(off[e], off[e + 1])
            g = O.gemv_f64(O.Q8_0, Wg[e], xs[rows], H, EF, round_w_fp16=True)
            u = O.gemv_f64(O.Q8_0, Wu[e], xs[rows], H, EF, round_w_fp16=True)
            h_ref[rows] = O.swiglu_np(g.astype(np.float32), u.astype(np.float32))
    check(hp_h, h_ref, "moe grouped gate_up silu (MFMA)")
    wp16 = dev(wp).half()
    op = ops.moe_gemm_down_q8(hp, dev(dq), dev(dd), H * EF, H * EF // 32, dev(off), wp16, TK, E, H, EF)
    o_ref = np.zeros((TK, H), np.float64)
    for e in range(E):
        if counts[e]:
            rows = slice(off[e], off[e + 1])
            o_ref[rows] = O.gemv_f64(O.Q8_0, Wd[e], hp_h[rows], EF, H, round_w_fp16=True) * f16(wp[rows])[:, None]
    check(host(op).astype(np.float32), o_ref, "moe grouped down (MFMA)")
    y = ops.moe_prefill_reduce_sum(op, dev(t2p.astype(np.uint32)), T, Kt, H)
    y_ref = host(op).astype(np.float32)[t2p].reshape(T, Kt, H).sum(axis=1)
    check(host(y).astype(np.float32), y_ref, "reduce_sum")
    # the int-dot grouped GEMV path on the same layer agrees at the activation-quantisation noise level
    hq = ops.moe_prefill_gate_up_silu_q8(ops.quantize_q8_1(xp), dev(gq), dev(gd), dev(uq), dev(ud), EF * H, EF * H // 32, dev(off), TK, E, H, EF)
    a, b = host(hq).astype(np.float64), hp_h.astype(np.float64)
    assert np.abs(a - b).max() / np.sqrt(np.mean(b * b)) < 0.2   # q8 activation noise through silu(g)*u


@pytest.mark.parametrize("H,EF", [(640, 256), (384, 128)])
def test_moe_grouped_gemm_q8_tile_boundaries(mx, H, EF):
    """Expert row counts on both sides of every tile class of the grouped kernel (empty, 1, 31..33, 63..65,
    127..129, 192/193, 256) and K depths of 1, 2, 3 and 5 chunks (the small-tile path walks K three chunks at a time)."""
    ops = mx.ops
    counts = np.array([0, 1, 63, 64, 65, 127, 128, 129, 192, 193, 256, 0, 31, 33, 32], np.int64)
    E, Kt = len(counts), 1
    ids = np.repeat(np.arange(E), counts).astype(np.int32)
    ids = ids[np.random.default_rng(11).permutation(ids.size)].reshape(-1, 1)
    T = ids.shape[0]
    w = O.uniform(12, (T, 1), 0.5, 1.5).astype(np.float32)
    mk = lambda seed, N, K: np.stack([O.quantize(O.Q8_0, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
    Wg, Wu, Wd = mk(3100, EF, H), mk(4100, EF, H), mk(5100, H, EF)
    gq, gd = O.repack_q8_0_to_soa(Wg)
    uq, ud = O.repack_q8_0_to_soa(Wu)
    dq, dd = O.repack_q8_0_to_soa(Wd)
    x = f16(O.normal(6100, (T, H)))
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    assert np.array_equal(np.diff(off.astype(np.int64)), counts)
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), T, H)
    hp = ops.moe_gemm_gate_up_silu_q8(xp, dev(gq), dev(gd), dev(uq), dev(ud), EF * H, EF * H // 32, dev(off), T, E, H, EF)
    hp_h = host(hp).astype(np.float32)
    xs = x[si]
    h_ref = np.zeros((T, EF), np.float32)
    o_ref = np.zeros((T, H), np.float64)
    for e in range(E):
        if counts[e]:
            rows = slice(off[e], off[e + 1])
            g = O.gemv_f64(O.Q8_0, Wg[e], xs[rows], H, EF, round_w_fp16=True)
            u = O.gemv_f64(O.Q8_0, Wu[e], xs[rows], H, EF, round_w_fp16=True)
            h_ref[rows] = O.swiglu_np(g.astype(np.float32), u.astype(np.float32))
            o_ref[rows] = O.gemv_f64(O.Q8_0, Wd[e], hp_h[rows], EF, H, round_w_fp16=True) * f16(wp[rows])[:, None]
    check(hp_h, h_ref, "grouped gate_up silu, boundary row counts")
    op = ops.moe_gemm_down_q8(hp, dev(dq), dev(dd), H * EF, H * EF // 32, dev(off), dev(wp).half(), T, E, H, EF)
    check(host(op).astype(np.float32), o_ref, "grouped down, boundary row counts")
    # per expert as well: a wrong row range shows up as one expert's rows being off, which a global norm can hide
    op_h = host(op).astype(np.float64)
    for e in range(E):
        if counts[e]:
            rows = slice(off[e], off[e + 1])
            err = np.abs(op_h[rows] - o_ref[rows]).max() / max(np.sqrt(np.mean(o_ref[rows] ** 2)), 1e-30)
            assert err < 5e-2, (e, counts[e], err)


@pytest.mark.parametrize("T,E,Kt,H,EF", [(64, 8, 2, 256, 256), (300, 16, 4, 512, 256)])
def test_moe_grouped_gemm_kquant(mx, T, E, Kt, H, EF):
    """Q4_K gate/up + Q4_K or Q6_K down expert banks (AoS, expert-major) through the grouped GEMM
    (moe_prefill_gate_up_silu_q4k, moe_prefill_down_packed_q4k/_q6k, include/ie/ops.hpp:922-983)."""
    ops = mx.ops
    mk = lambda F, seed, N, K: np.stack([O.quantize(F, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
    Wg, Wu = mk(O.Q4_K, 3100, EF, H), mk(O.Q4_K, 4100, EF, H)
    x = f16(O.normal(6100, (T, H)))
    ids, w = zipf_routing(7100, T, E, Kt)
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    TK = T * Kt
    counts = np.diff(off.astype(np.int64))
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, H)
    stride_gu = Wg[0].size
    hp = ops.moe_gemm_gate_up_silu_q4k(xp, dev(Wg), dev(Wu), dev(off), TK, E, H, EF, stride_gu)
    hp_h = host(hp).astype(np.float32)
    xs = x[si]
    h_ref = np.zeros((TK, EF), np.float32)
    for e in range(E):
        if counts[e]:
            rows = slice(off[e], off[e + 1])
            g = O.gemv_f64(O.Q4_K, Wg[e], xs[rows], H, EF, round_w_fp16=True)
            u = O.gemv_f64(O.Q4_K, Wu[e], xs[rows], H, EF, round_w_fp16=True)
            h_ref[rows] = O.swiglu_np(g.astype(np.float32), u.astype(np.float32))
    check(hp_h, h_ref, "moe grouped gate_up silu q4k (MFMA)")
    # soa = 1: the same blocks as per-field streams per expert region: the same fragments, so the same bits
    nb_gu = EF * H // 256
    Wg_s, Wu_s = ops.repack_moe_kquant_soa("q4k", Wg, E, nb_gu), ops.repack_moe_kquant_soa("q4k", Wu, E, nb_gu)
    hp_s = ops.moe_gemm_gate_up_silu_q4k(xp, dev(Wg_s), dev(Wu_s), dev(off), TK, E, H, EF, stride_gu, soa=True)
    assert torch.equal(hp_s, hp), "soa gate/up differs from the AoS bank"
    for soa, (a, b) in ((False, (Wg, Wu)), (True, (Wg_s, Wu_s))):
        hp_g = ops.moe_gemm_gate_up_silu_q4k(dev(x).half(), dev(a), dev(b), dev(off), TK, E, H, EF, stride_gu, soa=soa, sorted_idx=dev(si))
        assert torch.equal(hp_g, hp), "gather form differs from gather_rows + grouped GEMM"
    for fmt, F in (("q4k", O.Q4_K), ("q6k", O.Q6_K)):
        Wd = mk(F, 5100, H, EF)
        o_ref = np.zeros((TK, H), np.float64)
        for e in range(E):
            if counts[e]:
                rows = slice(off[e], off[e + 1])
                o_ref[rows] = O.gemv_f64(F, Wd[e], hp_h[rows], EF, H, round_w_fp16=True)
        op = ops.moe_gemm_down_kquant(fmt, hp, dev(Wd), dev(off), None, TK, E, H, EF, Wd[0].size)
        check(host(op).astype(np.float32), o_ref, "moe grouped down %s unweighted (MFMA)" % fmt)
        opw = ops.moe_gemm_down_kquant(fmt, hp, dev(Wd), dev(off), dev(wp).half(), TK, E, H, EF, Wd[0].size)
        check(host(opw).astype(np.float32), o_ref * f16(wp)[:, None], "moe grouped down %s weighted (MFMA)" % fmt)
        Wd_s = ops.repack_moe_kquant_soa(fmt, Wd, E, H * EF // 256)
        opw_s = ops.moe_gemm_down_kquant(fmt, hp, dev(Wd_s), dev(off), dev(wp).half(), TK, E, H, EF, Wd[0].size, soa=True)
        assert torch.equal(opw_s, opw), "soa down %s differs from the AoS bank" % fmt
        # unweighted rows + moe_prefill_reduce (weights applied there) == the reference's two-step path
        y = ops.moe_prefill_reduce(op, dev(t2p.astype(np.uint32)), dev(wp).half(), torch.zeros((T, H), dtype=torch.float16, device="cuda"), T, Kt, H)
        y_ref = (host(op).astype(np.float32) * f16(wp)[:, None])[t2p].reshape(T, Kt, H).sum(axis=1)
        check(host(y).astype(np.float32), y_ref, "prefill_reduce over %s rows" % fmt, max_rel=2e-3)
        # accumulate form: fp32 atomics into y_fp32[token], then the fp32 -> fp16 merge (include/ie/ops.hpp:930-962)
        y32 = torch.zeros((T, H), dtype=torch.float32, device="cuda")
        ops.moe_prefill_down_kquant_accum(fmt, hp, dev(Wd), dev(off), dev(si.astype(np.int32)), dev(wp).half(), y32, TK, E, H, EF, Wd[0].size)
        a_ref = np.zeros((T, H), np.float64)
        np.add.at(a_ref, si, o_ref * f16(wp)[:, None])
        check(host(y32), a_ref, "moe down %s accumulate form (fp32 atomics)" % fmt, abs_floor=0.0)
        y0 = f16(O.normal(7200, (T, H)))
        ym = ops.moe_prefill_merge_fp32_to_fp16(y32, dev(y0).half())
        assert np.array_equal(host(ym), (y0 + host(y32)).astype(np.float16))


@pytest.mark.parametrize("M,N,K", [(1, 8, 32), (33, 130, 288), (256, 512, 2048), (200, 135, 73), (129, 257, 1000)])
def test_gemm_fp16_plain(mx, M, N, K):
    """gemm_fp16 (fp32 C, the hand-tiled kernel; ragged M, N and K into an exactly sized C) and gemm_fp16_onednn (fp16 y,
    the vendor library): A[M,K] . B[K,N], fp32 accumulation (include/ie/ops.hpp:275-286,460-465), against fp64 on the
    same fp16 operands."""
    A = O.round_fp16(O.normal(3000 + M, (M, K), 0.0, 1.0))
    B = O.round_fp16(O.normal(3001 + N, (K, N), 0.0, 0.05))
    ref = A.astype(np.float64) @ B.astype(np.float64)
    guard = torch.full((M * N + 64,), 7.0, dtype=torch.float32, device="cuda")   # C sized exactly, canaries behind it
    C = mx.ops.gemm_fp16(dev(A).half(), dev(B).half(), M, N, K, C=guard[:M * N].view(M, N))
    assert bool((guard[M * N:] == 7.0).all()), "gemm_fp16 wrote past C"
    check(host(C).ravel(), ref.ravel(), "gemm_fp16 fp32 out", abs_floor=0.0, max_rel=2e-4)
    y = mx.ops.gemm_fp16(dev(A).half(), dev(B).half(), M, N, K, out_dtype=torch.float16)
    check(host(y).astype(np.float32).ravel(), ref.ravel(), "gemm_fp16_onednn fp16 out")


def test_q5_K_prefill_route(mx):
    """The reference's Q5_K prefill: dequant_q5_K_to_Bt + gemm_fp16_onednn (include/ie/dequant.hpp:81-86)."""
    M, N, K = 48, 96, 512
    W = O.quantize(O.Q4_K, O.normal(3100, (N, K), 0.0, 0.02))
    # Q5_K blocks from Q4_K ones: same header and nibbles, seeded high bits (the oracle has no Q5_K quantizer)
    b4 = W.reshape(-1, 144)
    b5 = np.concatenate([b4[:, :16], O.rand_bytes(3101, b4.shape[0] * 32).reshape(-1, 32), b4[:, 16:]], axis=1)
    A = O.round_fp16(O.normal(3102, (M, K), 0.0, 1.0))
    Bt = mx.ops.dequant_to_Bt("q5_K", dev(b5), K, N)
    wd = O.round_fp16(O.dequant(O.Q5_K, b5)).reshape(N, K)
    assert np.array_equal(host(Bt).astype(np.float32), wd.T)
    y = mx.ops.gemm_fp16(dev(A).half(), Bt, M, N, K, out_dtype=torch.float16)
    check(host(y).astype(np.float32).ravel(), (A.astype(np.float64) @ wd.T.astype(np.float64)).ravel(), "q5_K dequant + gemm_fp16")


@pytest.mark.parametrize("M,K,N", [(128, 512, 256), (77, 2880, 520), (300, 2880, 2880)])
def test_gemm_mxfp4_and_q5_K_fused(mx, M, K, N):
    """MXFP4 planes (K = 2880: 22 chunks and a half) and Q5_K blocks through the fused kernel, against fp64 over
    half(dequant) weights; and against the reference's own route (dequant to [K, N] fp16 + plain GEMM) on the same bits."""
    A = f16(O.normal(8100 + M, (M, K)))
    W = O.quantize(O.MXFP4, O.normal(8101 + N, (N, K), 0.0, 0.02))
    qs, e = O.repack_mxfp4_to_soa(W)
    ref = O.gemv_f64(O.MXFP4, W, A, K, N, round_w_fp16=True)
    got = mx.ops.gemm_mxfp4_soa(dev(A).half(), dev(qs), dev(e), M, K, N)
    check(host(got).astype(np.float32), ref, "gemm_mxfp4_soa M=%d K=%d N=%d" % (M, K, N))
    bt = mx.ops.dequant_soa_to_Bt("mxfp4_soa", (dev(qs), dev(e)), K, N)
    two = mx.ops.gemm_fp16(dev(A).half(), bt, M, N, K, out_dtype=torch.float16)
    check(host(got).astype(np.float32).ravel(), host(two).astype(np.float32).ravel(), "fused vs dequant + GEMM (mxfp4)", max_rel=2e-3)
    if K % 256 == 0:
        W5 = q5k_blocks(8200 + N, N, K)
        ref5 = O.gemv_f64(O.Q5_K, W5, A, K, N, round_w_fp16=True)
        got5 = mx.ops.gemm_q5_K(dev(A).half(), dev(W5), M, K, N)
        check(host(got5).astype(np.float32), ref5, "gemm_q5_K M=%d K=%d N=%d" % (M, K, N))


@pytest.mark.parametrize("T,E,Kt,H,EF", [(64, 8, 2, 320, 192), (96, 32, 4, 2880, 2880)])
def test_moe_grouped_gemm_mxfp4(mx, T, E, Kt, H, EF):
    """gpt-oss expert banks through the grouped matrix-core GEMM on fp16 rows: half(swiglu_oai(half(g + b), half(u + b)))
    and half(half(acc) + b), against the float chain (fp64 over half(dequant) weights) at H = EF = 2880."""
    from test_gpu_moe import make_experts, route
    ops = mx.ops
    Wg, gq, ge, qs_st, e_st = make_experts(O.MXFP4, 100, E, EF, H)
    Wu, uq, ue, _, _ = make_experts(O.MXFP4, 200, E, EF, H)
    Wd, dq, de, dqs_st, de_st = make_experts(O.MXFP4, 300, E, H, EF)
    bg, bu, bd = O.normal(1, (E, EF)), O.normal(2, (E, EF)), O.normal(3, (E, H))
    x = f16(O.normal(4, (T, H)))
    ids, w = route(5, T, E, Kt)
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    TK = T * Kt
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, H)
    hp = ops.moe_gemm_gate_up_oai_mxfp4(xp, dev(gq), dev(ge), dev(uq), dev(ue), qs_st, e_st, dev(bg), dev(bu), dev(off), TK, E, H, EF)
    hp_g = ops.moe_gemm_gate_up_oai_mxfp4(dev(x).half(), dev(gq), dev(ge), dev(uq), dev(ue), qs_st, e_st, dev(bg), dev(bu), dev(off), TK, E, H, EF,
                                          sorted_idx=dev(si))
    assert torch.equal(hp_g, hp), "gather form differs from gather_rows + grouped GEMM"
    hp_h = host(hp).astype(np.float32)
    xs = x[si]
    rows = np.arange(TK) if TK <= 256 else np.random.default_rng(9).choice(TK, 48, replace=False)
    exp_of = np.searchsorted(off, rows, side="right") - 1
    lo, hi = [], []
    for r_, e_ in zip(rows, exp_of):
        g = O.gemv_f64(O.MXFP4, Wg[e_], xs[r_:r_ + 1], H, EF, round_w_fp16=True)[0].astype(np.float64) + bg[e_]
        u = O.gemv_f64(O.MXFP4, Wu[e_], xs[r_:r_ + 1], H, EF, round_w_fp16=True)[0].astype(np.float64) + bu[e_]
        inf = np.float16(np.inf)
        gc = [np.nextafter(f16(g).astype(np.float16), -inf), f16(g).astype(np.float16), np.nextafter(f16(g).astype(np.float16), inf)]
        uc = [np.nextafter(f16(u).astype(np.float16), -inf), f16(u).astype(np.float16), np.nextafter(f16(u).astype(np.float16), inf)]
        outs = [f16(O.swiglu_oai_np(a.astype(np.float32), b.astype(np.float32))) for a in gc for b in uc]
        lo.append(np.min(outs, axis=0)); hi.append(np.max(outs, axis=0))
    got16 = hp_h[rows].astype(np.float16)
    inf = np.float16(np.inf)
    ok = (got16 >= np.nextafter(np.stack(lo).astype(np.float16), -inf)) & (got16 <= np.nextafter(np.stack(hi).astype(np.float16), inf))
    print("grouped mxfp4 gate/up (MFMA): %d / %d inside the one-ulp envelope of the chain" % (ok.sum(), ok.size), flush=True)
    assert ok.mean() > 0.9995, ok.mean()
    op = ops.moe_gemm_down_mxfp4(hp, dev(dq), dev(de), dqs_st, de_st, dev(bd), dev(off), TK, E, H, EF)
    # out = half(half(acc) + bias): the sum can cancel, so the gate is the set of values the chain can produce when
    # half(acc) moves by the accumulation-order noise and one fp16 ulp (as in test_gpu_moe), plus closeness in rms terms
    from test_gpu_moe import f16_candidates, sum_noise, check_envelope
    lo, hi, ctr = [], [], []
    for r_, e_ in zip(rows, exp_of):
        acc = O.gemv_f64(O.MXFP4, Wd[e_], hp_h[r_:r_ + 1], EF, H, round_w_fp16=True)[0].astype(np.float64)
        c = [f16(v.astype(np.float32) + bd[e_]) for v in f16_candidates(acc, sum_noise(acc))]
        lo.append(np.min(c, axis=0)); hi.append(np.max(c, axis=0)); ctr.append(c[1])
    op_h = host(op).astype(np.float32)[rows]
    check_envelope(op_h, np.stack(lo), np.stack(hi), "grouped mxfp4 down + bias (MFMA)")
    check(op_h, np.stack(ctr), "  ... against the centre of the envelope", max_rel=1.0)


def test_moe_grouped_gemm_q8_random_shapes(mx):
    """Random expert counts (empty experts, a few rows, several tiles) against random depths and widths, including the
    depths whose scale rows end in a half piece of the LDS scale table (K = 128, 384, 640).  Floating-point kernel: the
    reference is the same product in fp32 on the dequantized (fp16-rounded) weights; relative error against
    |ref| + 2 % of mean |ref| (an output that cancels to nothing carries the fp16 rounding of its terms)."""
    from machx_inference_engine_amd import synth
    ops = mx.ops
    d0 = "cuda:0"
    rng = np.random.default_rng(123)

    def deq(blocks, N, K):
        b = blocks.reshape(N, K // 32, 34)
        d = b[:, :, 0:2].contiguous().view(torch.float16).float()
        q = b[:, :, 2:].contiguous().view(torch.int8).float()
        return (d * q).half().float().reshape(N, K)

    worst = 0.0
    for it in range(12):
        E = int(rng.integers(1, 24))
        H = int(rng.choice([128, 256, 384, 512, 640, 1024, 2048]))
        EF = int(rng.choice([128, 256, 384, 768]))
        counts = rng.integers(0, 140, size=E)
        counts[rng.integers(0, E)] += int(rng.integers(0, 300))
        if counts.sum() == 0:
            counts[0] = 5
        off = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
        TK = int(off[-1])
        g = torch.Generator(device=d0)
        g.manual_seed(it)
        Wg = synth.random_weights("q8_0", E * EF, H, seed=10 + it, device=d0)
        Wu = synth.random_weights("q8_0", E * EF, H, seed=500 + it, device=d0)
        Wd = synth.random_weights("q8_0", E * H, EF, seed=900 + it, device=d0)
        gq, gd = synth.split_q8_0(Wg)
        uq, ud = synth.split_q8_0(Wu)
        dq, dd = synth.split_q8_0(Wd)
        x = (torch.randn((TK, H), device=d0, generator=g) * 0.5).half()
        wp = torch.rand((TK,), device=d0, generator=g).half()
        offd = torch.from_numpy(off).to(d0)
        hp = ops.moe_gemm_gate_up_silu_q8(x, gq, gd, uq, ud, EF * H, EF * H // 32, offd, TK, E, H, EF)
        op = ops.moe_gemm_down_q8(hp, dq, dd, H * EF, H * EF // 32, offd, wp, TK, E, H, EF)
        torch.cuda.synchronize()
        Wgf, Wuf, Wdf = deq(Wg, E * EF, H).reshape(E, EF, H), deq(Wu, E * EF, H).reshape(E, EF, H), deq(Wd, E * H, EF).reshape(E, H, EF)
        for e in range(E):
            lo, hi = int(off[e]), int(off[e + 1])
            if lo == hi:
                continue
            xe = x[lo:hi].float()
            gg, uu = xe @ Wgf[e].T, xe @ Wuf[e].T
            href = (gg / (1 + torch.exp(-gg))) * uu
            e1 = ((hp[lo:hi].float() - href).abs() / (href.abs() + 0.02 * href.abs().mean() + 1e-6)).max().item()
            oref = (hp[lo:hi].float() @ Wdf[e].T) * wp[lo:hi].float()[:, None]
            e2 = ((op[lo:hi].float() - oref).abs() / (oref.abs() + 0.02 * oref.abs().mean() + 1e-6)).max().item()
            worst = max(worst, e1, e2)
            assert e1 < 2e-3 and e2 < 2e-3, (it, E, H, EF, e, lo, hi, e1, e2)
    print("grouped q8_0 GEMM, 12 random layers: worst relative error %.2e" % worst, flush=True)


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
def test_gemm_eight_wave_workgroups(mx, fmt):
    """Dense launches whose 128-token tiles cover between half and all of the CUs (here 2 x 70 = 140 tiles) run
    eight-wave workgroups: waves 4 - 7 walk the second half of K and hand their sums over through LDS.  A ragged second
    token tile, and output columns sampled across every column tile, against the oracle."""
    M, K, N = 160, 2048, 256 * 70
    W = weights(fmt, 2300, N, K)
    A = f16(O.normal(2301, (M, K)))
    fn = getattr(mx.ops, "gemm_%s" % O.FMT_NAMES[fmt])
    got = host(fn(dev(A).half(), dev(W), M, K, N)).astype(np.float32)
    cols = np.unique(np.concatenate([np.arange(0, 96), np.arange(N - 96, N), np.arange(0, N, 37)]))
    ref = O.gemv_f64(fmt, np.ascontiguousarray(W[cols]), A, K, len(cols), round_w_fp16=True)
    check(got[:, cols], ref, "gemm %s, eight-wave workgroups" % O.FMT_NAMES[fmt])
