"""GPU parity at BASELINE.json's full sizes (configs 2, 3 and 5; config 4 at full size lives in
test_gpu_moe.py).  The weights are seeded N(0, 0.02) tensors quantized in HBM by the torch encoders of
machx_inference_engine_amd.synth; a seeded sample of output rows / tokens is recomputed by the oracle from
the same bytes (spot parity at the gate), and size-independent properties cover the rest:
row-slice consistency (a slice of the matrix alone gives the same rows bit for bit), batched ==
single-token results, GEMM rows == the T=1 GEMM of that token."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host
from machx_inference_engine_amd import synth

pytestmark = pytest.mark.gpu

H, FF = 4096, 14336


def f16(a):
    return O.round_fp16(np.asarray(a, np.float32))


def sample_rows(N, n=48, seed=0):
    rng = np.random.default_rng(seed)
    return np.unique(np.concatenate([[0, 1, N // 2, N - 2, N - 1], rng.integers(0, N, n)]))


@pytest.mark.parametrize("K,N", [(H, FF), (FF, H)])
@pytest.mark.parametrize("fmt", ["q6_K", "q8_0"])
def test_config2_gemv_full_size(mx, fmt, K, N):
    ops = mx.ops
    F = {"q6_K": O.Q6_K, "q8_0": O.Q8_0}[fmt]
    W = synth.normal_weights(fmt, N, K, seed=31 + K % 7)
    x = f16(O.normal(4000 + N, (8, K)))
    xq = ops.quantize_q8_1(dev(x).half())
    xq_h = host(xq).reshape(8, -1)
    rows = sample_rows(N)
    W_rows = host(W[torch.from_numpy(rows).cuda()])
    ref = O.gemv_q8chain(F, W_rows, xq_h, K, len(rows))          # [8, len(rows)]
    if fmt == "q8_0":
        qs, d = synth.split_q8_0(W)
        one = lambda xr: ops.gemv_q8_0_soa_q8(xr, qs, d, K, N)
        bat = lambda T: ops.gemv_q8_0_soa_q8_batched(xq[:T * (K // 32) * 40], qs, d, K, N, T)
        aos1 = ops.gemv_q8_0_q8(xq[:(K // 32) * 40], W, K, N)
    else:
        one = lambda xr: ops.gemv_q6_K_q8(xr, W, K, N)
        bat = lambda T: ops.gemv_q6_K_q8_batched(xq[:T * (K // 32) * 40], W, K, N, T)
        aos1 = None
    y1 = one(xq[:(K // 32) * 40])
    check(host(y1).astype(np.float32)[rows], ref[0], "%s %dx%d T=1 sampled rows" % (fmt, N, K))
    if aos1 is not None:
        # GGUF blocks and planes hold the same numbers; their kernels add the per-block terms in different orders
        check(host(aos1).astype(np.float32)[rows], ref[0], "%s %dx%d T=1 GGUF blocks, sampled rows" % (fmt, N, K))
        a, b = host(aos1).astype(np.float32), host(y1).astype(np.float32)
        assert np.mean(a == b) > 0.98 and np.abs(a - b).max() <= 2e-3 * np.abs(b).max()
    for T in (2, 4, 8):
        yT = bat(T)
        check(host(yT).astype(np.float32)[:, rows], ref[:T], "%s T=%d sampled rows" % (fmt, T))
        # every batched row is within fp32 summation noise of its single-token result
        a, b = host(yT[0]).astype(np.float32), host(y1).astype(np.float32)
        assert np.mean(a == b) > 0.98 and np.abs(a - b).max() <= 2e-3 * np.abs(b).max()
    # a slice of the rows computed alone gives the same numbers
    lo, n = N // 3 // 16 * 16, 512
    if fmt == "q8_0":
        ys = ops.gemv_q8_0_soa_q8(xq[:(K // 32) * 40], qs[lo * K:(lo + n) * K], d[lo * (K // 32):(lo + n) * (K // 32)], K, n)
    else:
        ys = ops.gemv_q6_K_q8(xq[:(K // 32) * 40], W[lo:lo + n], K, n)
    assert torch.equal(ys, y1[lo:lo + n])


_W3 = {}


def _config3_weights(K, N):
    if (K, N) not in _W3:
        _W3[(K, N)] = synth.normal_weights("q4_K", N, K, seed=41)
    return _W3[(K, N)]


@pytest.mark.parametrize("T", [2048, 512, 4096])
@pytest.mark.parametrize("K,N", [(H, FF), (FF, H)])
def test_config3_gemm_full_size(mx, K, N, T):
    """T = 512 on N = 4096 runs 64-token tiles in K slices (another launch than 2048 / 4096)."""
    ops = mx.ops
    W = _config3_weights(K, N)
    A = f16(O.normal(4100 + N, (T, K), 0.0, 1.0))
    Ad = dev(A).half()
    Y = ops.gemm_q4_K(Ad, W, T, K, N)
    rows = sample_rows(N, 40, 1)
    toks = sample_rows(T, 12, 2)
    W_rows = host(W[torch.from_numpy(rows).cuda()])
    ref = O.gemv_f64(O.Q4_K, W_rows, A[toks], K, len(rows), round_w_fp16=True)
    got = host(Y).astype(np.float32)[np.ix_(toks, rows)]
    check(got, ref, "gemm_q4_K T=%d K=%d N=%d sampled" % (T, K, N))
    # token rows are independent: a single-token GEMM reproduces its row up to fp32 summation order (a launch this
    # small runs as K slices whose partial sums are added afterwards): within one fp16 ulp of the value or of the row's rms
    t = int(toks[3])
    y1 = host(ops.gemm_q4_K(Ad[t:t + 1], W, 1, K, N)).astype(np.float32)[0]
    yt = host(Y[t]).astype(np.float32)
    rms = float(np.sqrt(np.mean(yt.astype(np.float64) ** 2)))
    assert np.all(np.abs(y1 - yt) <= np.maximum(np.abs(yt), rms) * 2.0 ** -9), "a token row depends on the batch it is in"
    # full 128-token tiles of a batch that is not sliced keep the accumulation order: identical bits
    Y3 = ops.gemm_q4_K(Ad[:1024], W, 1024, K, N) if N > 8192 and T >= 1024 else None
    if Y3 is not None:
        assert torch.equal(Y3, Y[:1024])
    # and the last, partial token tile (T not a multiple of 128) leaves the others untouched
    Y2 = ops.gemm_q4_K(Ad[:T - 37], W, T - 37, K, N)
    assert torch.equal(Y2, Y[:T - 37])


def test_config5_grouped_gemm_full_size(mx):
    ops = mx.ops
    E, Kt, Hm, EF, T = 128, 8, 2048, 768, 2048
    gate = synth.normal_weights("q8_0", E * EF, Hm, 51)
    up = synth.normal_weights("q8_0", E * EF, Hm, 52)
    down = synth.normal_weights("q8_0", E * Hm, EF, 53)
    gq, gd = synth.split_q8_0(gate); uq, ud = synth.split_q8_0(up); dq, dd = synth.split_q8_0(down)
    rng = np.random.default_rng(5)
    p = np.arange(1, E + 1, dtype=np.float64) ** -1.1
    p = p[rng.permutation(E)]; p /= p.sum()
    ids = np.stack([np.sort(rng.choice(E, size=Kt, replace=False, p=p)) for _ in range(T)]).astype(np.int32)
    w = f16(rng.random((T, Kt)).astype(np.float32) + 0.1)
    w = f16(w / w.sum(axis=1, keepdims=True))
    x = f16(O.normal(4200, (T, Hm)))
    TK = T * Kt
    # routing -> packing entirely on the device, checked against the host counting sort
    off, si, wp, t2p = ops.moe_build_packing_device(dev(ids), dev(w).half(), E)
    off_r, si_r, wp_r, t2p_r = O.build_moe_packing(ids, w, E)
    assert np.array_equal(host(off).view(np.uint32), off_r) and np.array_equal(host(si), si_r) and np.array_equal(host(t2p), t2p_r)
    xp = ops.moe_gather_rows(dev(x).half(), si, TK, Hm)
    hp = ops.moe_gemm_gate_up_silu_q8(xp, gq, gd, uq, ud, EF * Hm, EF * Hm // 32, off, TK, E, Hm, EF)
    op = ops.moe_gemm_down_q8(hp, dq, dd, Hm * EF, Hm * EF // 32, off, wp, TK, E, Hm, EF)
    y = ops.moe_prefill_reduce_sum(op, t2p, T, Kt, Hm)
    hp_h, op_h = host(hp).astype(np.float32), host(op).astype(np.float32)
    # sampled packed rows against the oracle, expert by expert (largest, smallest and a few others)
    counts = np.diff(off_r.astype(np.int64))
    experts = np.unique(np.concatenate([[int(np.argmax(counts)), int(np.argmin(np.where(counts > 0, counts, 1 << 30)))], rng.integers(0, E, 6)]))
    g_h, u_h, d_h = host(gate).reshape(E, EF, -1), host(up).reshape(E, EF, -1), host(down).reshape(E, Hm, -1)
    xs = x[si_r]
    for e in experts:
        if counts[e] == 0:
            continue
        rr = off_r[e] + np.unique(np.concatenate([[0, counts[e] - 1], rng.integers(0, counts[e], 3)]))
        g = O.gemv_f64(O.Q8_0, g_h[e], xs[rr], Hm, EF, round_w_fp16=True)
        u = O.gemv_f64(O.Q8_0, u_h[e], xs[rr], Hm, EF, round_w_fp16=True)
        check(hp_h[rr], O.swiglu_np(g.astype(np.float32), u.astype(np.float32)), "C5 gate_up expert %d (%d rows)" % (e, counts[e]))
        o = O.gemv_f64(O.Q8_0, d_h[e], hp_h[rr], EF, Hm, round_w_fp16=True) * wp_r[rr][:, None]
        check(op_h[rr], o, "C5 down expert %d" % e)
    y_ref = op_h[t2p_r].reshape(T, Kt, Hm).sum(axis=1)
    check(host(y).astype(np.float32), y_ref, "C5 reduce_sum")
    assert np.isfinite(hp_h).all() and np.isfinite(op_h).all()
    # ---- the same layer through the reference's own q8 signatures (include/ie/moe_q8.hpp:51-72): block_q8_1x rows in,
    # int-dot on the matrix cores, against the q8-chain oracle
    xq = ops.quantize_q8_1(xp)
    hq8 = ops.moe_prefill_gate_up_silu_q8(xq, gq, gd, uq, ud, EF * Hm, EF * Hm // 32, off, TK, E, Hm, EF)
    hqq = ops.quantize_q8_1(hq8)
    oq8 = ops.moe_prefill_down_q8(hqq, dq, dd, Hm * EF, Hm * EF // 32, off, wp, TK, E, Hm, EF)
    xq_h, hq_h = host(xq).reshape(TK, -1), host(hqq).reshape(TK, -1)
    hq8_h, oq8_h = host(hq8).astype(np.float32), host(oq8).astype(np.float32)
    assert np.array_equal(hq_h.ravel(), O.quantize_q8_1(hq8_h))
    for e in experts:
        if counts[e] == 0:
            continue
        rr = off_r[e] + np.unique(np.concatenate([[0, counts[e] - 1], rng.integers(0, counts[e], 3)]))
        g = O.gemv_q8chain(O.Q8_0, g_h[e], xq_h[rr], Hm, EF)
        u = O.gemv_q8chain(O.Q8_0, u_h[e], xq_h[rr], Hm, EF)
        check(hq8_h[rr], O.swiglu_np(g.astype(np.float32), u.astype(np.float32)), "C5 q8 rows, gate_up expert %d (%d rows)" % (e, counts[e]))
        o = O.gemv_q8chain(O.Q8_0, d_h[e], hq_h[rr], EF, Hm) * wp_r[rr][:, None]
        check(oq8_h[rr], o, "C5 q8 rows, down expert %d" % e)
    # rows of experts nobody sampled: finite, and every row written (the buffers come from torch.empty)
    assert np.isfinite(hq8_h).all() and np.isfinite(oq8_h).all()
