"""The entry points that keep their scratch in a library-owned device array (split-K batched GEMV, K-sliced dense
GEMM) against their caller-workspace twins, through the C ABI: same bits, on two calls in a row of which the second
is smaller (the array keeps the first call's contents), after a poisoned workspace, and against the oracle."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host
from machx_inference_engine_amd import synth

pytestmark = pytest.mark.gpu


def f16(a):
    return O.round_fp16(np.asarray(a, np.float32))


def test_split_k_gemv_static_scratch_equals_workspace_form(mx):
    ops = mx.ops
    ops.init()
    K, N1, T1, N2, T2 = 14336, 4096, 8, 1000, 3          # second call: fewer rows, fewer tokens
    W = synth.normal_weights("q8_0", N1, K, seed=61)
    qs, d = synth.split_q8_0(W)
    x = f16(O.normal(6100, (T1, K)))
    xq = ops.quantize_q8_1(dev(x).half())
    rb = K // 32 * 40
    for (N, T) in ((N1, T1), (N2, T2)):
        need = ops.gemv_batched_ws_bytes(K, N, T)
        assert need >= 2 * T * N * 4            # these shapes split K over at least two ranges
        ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
        y_static = ops.gemv_q8_0_soa_q8_batched(xq[:T * rb], qs[:N * K], d[:N * (K // 32)], K, N, T)
        y_ws = ops.gemv_q8_batched_ws("q8_0_soa", xq[:T * rb], (qs[:N * K], d[:N * (K // 32)]), K, N, T, ws)
        assert torch.equal(y_static, y_ws), "static-scratch and workspace forms differ (N=%d T=%d)" % (N, T)
        assert torch.isfinite(y_ws.float()).all()
        rows = np.unique(np.concatenate([[0, N - 1], np.random.default_rng(N).integers(0, N, 24)]))
        ref = O.gemv_q8chain(O.Q8_0, host(W[torch.from_numpy(rows).cuda()]), host(xq[:T * rb]), K, len(rows))
        check(host(y_static).astype(np.float32)[:, rows], ref, "split-K GEMV, library scratch, N=%d T=%d" % (N, T))
    # the GGUF-block formats share the path
    for fmt, F in (("q6_K", O.Q6_K), ("q4_K", O.Q4_K)):
        Wk = synth.normal_weights(fmt, N2, K, seed=62)
        ws = torch.full((ops.gemv_batched_ws_bytes(K, N2, T2) // 4,), float("nan"), dtype=torch.float32, device="cuda")
        a = getattr(ops, "gemv_%s_q8_batched" % fmt)(xq[:T2 * rb], Wk, K, N2, T2)
        b = ops.gemv_q8_batched_ws(fmt, xq[:T2 * rb], (Wk,), K, N2, T2, ws)
        assert torch.equal(a, b), fmt
    # a workspace that is too small is refused, nothing is launched
    with pytest.raises(mx.ops.MxError):
        ops.gemv_q8_batched_ws("q8_0_soa", xq, (qs, d), K, N1, T1, torch.empty(1024, dtype=torch.float32, device="cuda"))


def test_k_sliced_gemm_static_scratch_equals_workspace_form(mx):
    ops = mx.ops
    K, N = 14336, 4096
    W = synth.normal_weights("q4_K", N, K, seed=63)
    A = f16(O.normal(6300, (256, K)))
    Ad = dev(A).half()
    for M in (256, 100):                                   # both are K-sliced; the second is smaller
        need = ops.gemm_ws_bytes(M, K, N)
        assert need == 8 * M * N * 4
        ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
        y_static = ops.gemm_q4_K(Ad[:M], W, M, K, N)
        y_ws = ops.gemm_ws("q4_K", Ad[:M], (W,), M, K, N, ws)
        assert torch.isfinite(y_ws.float()).all()
        # a workspace of the static scratch's capacity (8 Mi floats) gives the same launch, hence the same bits; a roomier one
        # may take more slices and differ by fp32 summation order
        ws_same = torch.full((8 << 20,), float("nan"), dtype=torch.float32, device="cuda")
        assert torch.equal(y_static, ops.gemm_ws("q4_K", Ad[:M], (W,), M, K, N, ws_same)), "same capacity, different bits (M=%d)" % M
        rows = np.unique(np.random.default_rng(M).integers(0, N, 32))
        ref = O.gemv_f64(O.Q4_K, host(W[torch.from_numpy(rows).cuda()]), A[:M], K, len(rows), round_w_fp16=True)
        check(host(y_static).astype(np.float32)[:, rows], ref, "K-sliced GEMM, library scratch, M=%d" % M)
        check(host(y_ws).astype(np.float32)[:, rows], ref, "K-sliced GEMM, caller workspace, M=%d" % M)
    # no workspace at all is legal: the launch is not sliced
    y0 = ops.gemm_ws("q4_K", Ad[:100], (W,), 100, K, N, None)
    rows = np.arange(0, N, 131)
    check(host(y0).astype(np.float32)[:, rows], O.gemv_f64(O.Q4_K, host(W[torch.from_numpy(rows).cuda()]), A[:100], K, len(rows), round_w_fp16=True),
          "unsliced GEMM (no workspace)")
