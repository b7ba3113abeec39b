"""GPU parity for the repacked K-quant layouts: the three-region Q4_K "reorder" streams, the
natural-order Q4_K / Q6_K planes and the per-expert stream regions.  A repack moves bits and never
changes a weight, so every result is checked against the AoS kernels on the same weights (bit for
bit where the arithmetic order is the same) and against the q8-chain oracle."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host, weights

pytestmark = pytest.mark.gpu


def acts_q8(seed, T, K):
    return O.quantize_q8_1(O.round_fp16(O.normal(seed, (T, K), 0.0, 1.0)))


@pytest.mark.parametrize("K,N", [(256, 5), (2048, 130), (4096, 300), (14336, 64)])
def test_gemv_q4_K_reorder_and_soa(mx, K, N):
    """gemv_q4_K_reorder_q8 (src/ops/gemv_q8dot.cpp:152-256) and gemv_q4_soa_q8 (src/ops/gemv_q4_soa.cpp:
    160-312): same units, products and fold as the AoS kernel, so bit-identical to it."""
    ops = mx.ops
    W = weights(O.Q4_K, 2000 + K, N, K)
    xq = acts_q8(2001, 1, K)
    y_aos = ops.gemv_q4_K_q8(dev(xq), dev(W), K, N)
    check(host(y_aos).astype(np.float32), O.gemv_q8chain(O.Q4_K, W, xq, K, N)[0], "gemv_q4_K_q8")
    y_re = ops.gemv_q4_K_reorder_q8(dev(xq), dev(ops.repack_q4_K_to_reorder(W, K, N)), K, N)
    assert torch.equal(y_re, y_aos)
    y_soa = ops.gemv_q4_soa_q8(dev(xq), [dev(p) for p in ops.repack_q4_K_to_soa(W, K, N)], K, N)
    assert torch.equal(y_soa, y_aos)


@pytest.mark.parametrize("T", (1, 2, 4, 8, 16))
@pytest.mark.parametrize("K,N", [(256, 5), (2048, 130), (4096, 300), (14336, 64)])
def test_gemv_q6_soa(mx, K, N, T):
    """gemv_q6_soa_q8 / _batched (src/ops/gemv_q6_soa.cpp:137-407): natural-order bit planes; the partial
    sums group differently from the AoS kernel, so the gate is the q8-chain oracle."""
    ops = mx.ops
    W = weights(O.Q6_K, 2100 + K, N, K)
    xq = acts_q8(2101 + T, T, K)
    planes = [dev(p) for p in ops.repack_q6_K_to_soa(W, K, N)]
    y = host(ops.gemv_q6_soa_q8(dev(xq), planes, K, N, T)).astype(np.float32).reshape(T, N)
    ref = O.gemv_q8chain(O.Q6_K, W, xq, K, N)
    for t in range(T):
        check(y[t], ref[t], "gemv_q6_soa_q8 K=%d N=%d T=%d row %d" % (K, N, T, t))
    if T == 1:
        # two plane sets in one launch: each half equals the single launch bit for bit
        W2 = weights(O.Q6_K, 2150 + K, N, K)
        planes2 = [dev(p) for p in ops.repack_q6_K_to_soa(W2, K, N)]
        ya, yb = ops.gemv_q8_x2("q6_soa", dev(xq), planes, planes2, K, N)
        assert np.array_equal(host(ya).astype(np.float32), y[0])
        check(host(yb).astype(np.float32), O.gemv_q8chain(O.Q6_K, W2, xq, K, N)[0], "gemv_q6_soa_q8_x2 second matrix K=%d N=%d" % (K, N))


@pytest.mark.parametrize("K,N", [(256, 3), (1024, 70), (2880 // 32 * 32 + 256 - 2880 % 256, 9)])
def test_dequant_repacked_to_Bt_bit_exact(mx, K, N):
    """dequant_q4_moe_soa_to_Bt / dequant_q6_K_soa_to_Bt (include/ie/dequant.hpp:64-80), dequant_q4_soa_to_Bt /
    dequant_q6_soa_to_Bt (include/ie/ops.hpp:421-458), dequant_mxfp4_soa_to_Bt (include/ie/dequant.hpp:60-63):
    bit-identical to the AoS transposed dequant, which is bit-exact against the oracle."""
    ops = mx.ops
    W4, W6 = weights(O.Q4_K, 2200, N, K), weights(O.Q6_K, 2201, N, K)
    nb = N * K // 256
    bt4 = ops.dequant_to_Bt("q4_K", dev(W4), K, N)
    assert np.array_equal(host(bt4).view(np.uint16), O.dequant_to_Bt(O.Q4_K, W4, K, N))
    bt6 = ops.dequant_to_Bt("q6_K", dev(W6), K, N)
    assert torch.equal(ops.dequant_soa_to_Bt("q4_moe_soa", [dev(ops.repack_moe_kquant_soa("q4k", W4, 1, nb))], K, N), bt4)
    assert torch.equal(ops.dequant_soa_to_Bt("q6_K_soa", [dev(ops.repack_moe_kquant_soa("q6k", W6, 1, nb))], K, N), bt6)
    assert torch.equal(ops.dequant_soa_to_Bt("q4_soa", [dev(p) for p in ops.repack_q4_K_to_soa(W4, K, N)], K, N), bt4)
    assert torch.equal(ops.dequant_soa_to_Bt("q6_soa", [dev(p) for p in ops.repack_q6_K_to_soa(W6, K, N)], K, N), bt6)
    Km = K + 32                                                   # MXFP4: K % 32 == 0 only
    Wm = weights(O.MXFP4, 2202, N, Km)
    qs, e = O.repack_mxfp4_to_soa(Wm)
    assert torch.equal(ops.dequant_soa_to_Bt("mxfp4_soa", [dev(qs), dev(e)], Km, N), ops.dequant_to_Bt("mxfp4", dev(Wm), Km, N))
