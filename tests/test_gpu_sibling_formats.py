"""GPU parity for the sibling formats on the shared kernels: Q4_0 (Gemma-4 QAT; GGUF blocks and SoA
planes, int-dot and fp16-activation GEMV, multi-bank launch, matrix-core GEMM, transposed dequant) and
Q5_K (int-dot and fp16-activation GEMV).  Gate: max_rel <= 1e-3, cosine >= 0.99999; dequant bit-exact."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host, weights

pytestmark = pytest.mark.gpu


def acts(seed, T, K):
    return O.round_fp16(O.normal(seed, (T, K), 0.0, 1.0))


@pytest.mark.parametrize("K,N", [(32, 5), (2880, 130), (4096, 300), (8192 + 32, 17)])
def test_gemv_q4_0(mx, K, N):
    ops = mx.ops
    W = weights(O.Q4_0, 6000 + K, N, K)
    x = acts(6001, 1, K)
    xq = O.quantize_q8_1(x)
    ref = O.gemv_q8chain(O.Q4_0, W, xq, K, N)[0]
    qs, d = ops.repack_q4_0_to_soa(W, K, N)
    assert np.array_equal(qs.reshape(-1, 16), W.reshape(-1, 18)[:, 2:]) and np.array_equal(d, W.reshape(-1, 18)[:, :2].copy().view(np.uint16).ravel())
    y_soa = ops.gemv_q4_0_soa_q8(dev(xq), dev(qs), dev(d), K, N)
    check(host(y_soa).astype(np.float32), ref, "gemv_q4_0_soa_q8 K=%d N=%d" % (K, N))
    assert torch.equal(ops.gemv_q4_0_q8(dev(xq), dev(W), K, N), y_soa)          # GGUF blocks: same units, same fold
    y16 = ops.gemv_q4_0(dev(x[0]).half(), dev(W), K, N)
    check(host(y16).astype(np.float32), O.gemv_f64(O.Q4_0, W, x, K, N)[0], "gemv_q4_0 (fp16 activations)")


@pytest.mark.parametrize("T", (2, 3, 8, 16))
def test_gemv_q4_0_soa_batched(mx, T):
    K, N = 2048, 130
    W = weights(O.Q4_0, 6100, N, K)
    xq = O.quantize_q8_1(acts(6101 + T, T, K))
    qs, d = mx.ops.repack_q4_0_to_soa(W, K, N)
    y = host(mx.ops.gemv_q4_0_soa_q8(dev(xq), dev(qs), dev(d), K, N, T)).astype(np.float32)
    ref = O.gemv_q8chain(O.Q4_0, W, xq, K, N)
    for t in range(T):
        check(y[t], ref[t], "gemv_q4_0_soa_q8_batched T=%d row %d" % (T, t))


@pytest.mark.parametrize("Ns", [(512,), (1024, 96), (700, 33, 130)])
def test_gemv_q4_0_soa_multi(mx, Ns):
    """Up to three projections sharing x_q8 in one launch (include/ie/ops.hpp:577-592): each output equals
    the single-bank kernel's, bit for bit (same row walk)."""
    K = 2560
    ops = mx.ops
    xq = dev(O.quantize_q8_1(acts(6200, 1, K)))
    banks, singles = [], []
    for i, N in enumerate(Ns):
        qs, d = ops.repack_q4_0_to_soa(weights(O.Q4_0, 6201 + i, N, K), K, N)
        banks.append((dev(qs), dev(d), N))
        singles.append(ops.gemv_q4_0_soa_q8(xq, banks[-1][0], banks[-1][1], K, N))
    for y, s in zip(ops.gemv_q4_0_soa_q8_multi(xq, banks, K), singles):
        assert torch.equal(y, s)


@pytest.mark.parametrize("M,K,N", [(1, 128, 8), (70, 512, 200), (300, 2048, 520)])
def test_gemm_q4_0_and_Bt(mx, M, K, N):
    ops = mx.ops
    W = weights(O.Q4_0, 6300 + M, N, K)
    A = acts(6301, M, K)
    y = ops.gemm_q4_0(dev(A).half(), dev(W), M, K, N)
    check(host(y).astype(np.float32).ravel(), O.gemv_f64(O.Q4_0, W, A, K, N, round_w_fp16=True).ravel(), "gemm_q4_0 M=%d" % M)
    bt = ops.dequant_to_Bt("q4_0", dev(W), K, N)
    assert np.array_equal(host(bt).view(np.uint16), O.dequant_to_Bt(O.Q4_0, W, K, N))
    qs, d = ops.repack_q4_0_to_soa(W, K, N)
    assert torch.equal(ops.dequant_soa_to_Bt("q4_0_soa", [dev(qs), dev(d)], K, N), bt)
    # the reference's prefill route for this format: Bt + dense GEMM
    y2 = ops.gemm_fp16(dev(A).half(), bt, M, N, K, out_dtype=torch.float16)
    check(host(y2).astype(np.float32).ravel(), host(y).astype(np.float32).ravel(), "Bt + gemm_fp16 vs fused", max_rel=2e-3)


@pytest.mark.parametrize("T", (1, 2, 8))
@pytest.mark.parametrize("K,N", [(256, 5), (2048, 130), (5120, 64)])
def test_gemv_q5_K(mx, K, N, T):
    ops = mx.ops
    W = O.synth_q5_K(O.normal(6400 + K, (N, K), 0.0, 0.02), 6401)
    x = acts(6402 + T, T, K)
    xq = O.quantize_q8_1(x)
    y = host(ops.gemv_q5_K_q8(dev(xq), dev(W), K, N, T)).astype(np.float32).reshape(T, N)
    ref = O.gemv_q8chain(O.Q5_K, W, xq, K, N)
    for t in range(T):
        check(y[t], ref[t], "gemv_q5_K_q8 K=%d T=%d row %d" % (K, T, t))
    if T == 1:
        y16 = ops.gemv_q5_K(dev(x[0]).half(), dev(W), K, N)
        check(host(y16).astype(np.float32), O.gemv_f64(O.Q5_K, W, x, K, N)[0], "gemv_q5_K (fp16 activations)")


@pytest.mark.parametrize("T,E,Kt,K,N", [(40, 6, 2, 736, 200), (96, 8, 2, 1024, 512)])
def test_moe_prefill_proj_q4_0(mx, T, E, Kt, K, N):
    """moe_prefill_proj_q4_0_q8 / _soa_q8 / _xmx (include/ie/ops.hpp:166-204): plain projections of expert-sorted rows
    through Q4_0 experts; the int-dot forms against the q8-chain oracle expert by expert, the matrix-core form against
    the float chain with fp16-rounded weights."""
    ops = mx.ops
    Ws = np.stack([weights(O.Q4_0, 6500 + e, N, K) for e in range(E)])
    x = acts(6510, T, K)
    rng = np.random.default_rng(6511)
    ids = np.stack([np.sort(rng.choice(E, size=Kt, replace=False)) for _ in range(T)]).astype(np.int32)
    off, si, wp, t2p = ops.build_moe_packing(ids, np.full(ids.shape, 0.5, np.float32), E)
    TK = T * Kt
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, K)
    xq_s = ops.quantize_q8_1s(xp)
    xq_x = host(ops.quantize_q8_1(xp)).reshape(TK, -1)      # same quants and d in the 40-byte layout, for the oracle
    stride = Ws[0].size
    got = ops.moe_prefill_proj_q4_0("q8", xq_s, dev(Ws), dev(off), TK, E, K, N, stride)
    ref = np.zeros((TK, N), np.float64)
    for e in range(E):
        if off[e + 1] > off[e]:
            ref[off[e]:off[e + 1]] = O.gemv_q8chain(O.Q4_0, Ws[e], xq_x[off[e]:off[e + 1]], K, N)
    check(host(got).astype(np.float32).ravel(), ref.ravel(), "moe_prefill_proj_q4_0_q8")
    planes = [ops.repack_q4_0_to_soa(Ws[e], K, N) for e in range(E)]
    qs_bank, d_bank = np.concatenate([p[0] for p in planes]), np.concatenate([p[1] for p in planes])
    got_soa = ops.moe_prefill_proj_q4_0("soa_q8", xq_s, (dev(qs_bank), dev(d_bank)), dev(off), TK, E, K, N, (N * K // 2, N * K // 32))
    assert torch.equal(got_soa, got)
    if K % 128 == 0:
        got_x = ops.moe_prefill_proj_q4_0("xmx", xp, dev(Ws), dev(off), TK, E, K, N, stride)
        xs = x[si]
        ref_x = np.zeros((TK, N), np.float64)
        for e in range(E):
            if off[e + 1] > off[e]:
                ref_x[off[e]:off[e + 1]] = O.gemv_f64(O.Q4_0, Ws[e], xs[off[e]:off[e + 1]], K, N, round_w_fp16=True)
        check(host(got_x).astype(np.float32).ravel(), ref_x.ravel(), "moe_prefill_proj_q4_0_xmx")


@pytest.mark.parametrize("M,K,N", [(1, 64, 8), (5, 736, 130), (37, 2048, 300), (300, 1056, 200)])
def test_gemm_q4_0_q8(mx, M, K, N):
    """gemm_q4_0_q8 (include/ie/ops.hpp:538-548): int-dot GEMM over block_q8_1s rows, any M, any K % 32 == 0."""
    W = weights(O.Q4_0, 6600 + M, N, K)
    x = acts(6601, M, K)
    xq_s = mx.ops.quantize_q8_1s(dev(x).half())
    y = mx.ops.gemm_q4_0_q8(xq_s, dev(W), M, K, N)
    ref = O.gemv_q8chain(O.Q4_0, W, O.quantize_q8_1(x), K, N)
    check(host(y).astype(np.float32).ravel(), ref.ravel(), "gemm_q4_0_q8 M=%d" % M)


@pytest.mark.parametrize("M,K,N", [(7, 512, 96), (70, 1024, 260), (600, 2048, 512)])
def test_gemm_q8_rows_dense(mx, M, K, N):
    """Dense int-dot GEMM over block_q8_1s rows for Q4_K / Q6_K / Q8_0 planes (int8 matrix cores, token tiles dealt over
    workgroups): every row against the q8 chain with the stored half sums (the arithmetic of mx_gemv_*_q8s)."""
    x = acts(6700 + M, M, K)
    xq_s = mx.ops.quantize_q8_1s(dev(x).half())
    xq_h = host(xq_s)
    for fmt, F in (("q4_K", O.Q4_K), ("q6_K", O.Q6_K)):
        W = weights(F, 6701 + N, N, K)
        y = mx.ops.gemm_q8_rows(fmt, xq_s, (dev(W),), M, K, N)
        ref = O.gemv_q8schain(F, W, xq_h, K, N)
        check(host(y).astype(np.float32).ravel(), ref.ravel(), "gemm_%s_q8 M=%d" % (fmt, M))
    W = weights(O.Q8_0, 6702 + N, N, K)
    qs, d = O.repack_q8_0_to_soa(W)
    y = mx.ops.gemm_q8_rows("q8_0_soa", xq_s, (dev(qs), dev(d)), M, K, N)
    ref = O.gemv_q8chain(O.Q8_0, W, O.quantize_q8_1(x), K, N)
    check(host(y).astype(np.float32).ravel(), ref.ravel(), "gemm_q8_0_soa_q8 M=%d" % M)
