"""GPU parity: device-side MoE routing / packing (src/ops/moe.cpp:22-216,366-446,
src/model/qwen3moe_pack.cpp) and the fused normalisation -> block_q8_1x producers
(src/ops/elementwise.cpp:136-191, src/ops/deltanet.cpp:73-130)."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host

pytestmark = pytest.mark.gpu


def f16(a):
    return O.round_fp16(np.asarray(a, np.float32))


@pytest.mark.parametrize("T,E,k,H", [(1, 256, 8, 2048), (5, 128, 8, 512), (33, 32, 4, 2880), (2, 1000, 64, 256)])
def test_moe_router(mx, T, E, k, H):
    x = f16(O.normal(9100, (T, H)))
    Wg = O.normal(9101, (E, H), 0.0, 0.05).astype(np.float32)
    idx, w = mx.ops.moe_router(dev(x).half(), dev(Wg), E, k)
    logits = (x.astype(np.float64) @ Wg.astype(np.float64).T).astype(np.float32)
    ids_ref, w_ref = O.route_from_logits(logits, k)
    idx_h, w_h = host(idx), host(w).astype(np.float32)
    # a pick may differ only where two probabilities tie within fp32 noise of the logits
    same = (idx_h == ids_ref).all(axis=1)
    assert same.mean() >= 0.9, "routing disagrees on %d of %d tokens" % ((~same).sum(), T)
    assert (np.diff(idx_h, axis=1) > 0).all(), "expert ids ascending and distinct"
    np.testing.assert_allclose(w_h.sum(axis=1), 1.0, atol=4e-3)
    check(w_h[same], w_ref[same], "router weights", max_rel=2e-3)


@pytest.mark.parametrize("T,E,k", [(1, 32, 4), (7, 128, 8), (3, 1024, 16)])
def test_moe_topk_from_logits(mx, T, E, k):
    logits = f16(O.normal(9200, (T, E), 0.0, 2.0))
    idx, w = mx.ops.moe_topk_from_logits(dev(logits).half(), k)
    ids_ref, w_ref = O.route_from_logits(logits, k)
    idx_h = host(idx)
    same = (idx_h == ids_ref).all(axis=1)
    # fp16 logits tie exactly now and then; the reference breaks an exact tie towards the higher id
    for t in np.where(~same)[0]:
        a, b = set(idx_h[t]) - set(ids_ref[t]), set(ids_ref[t]) - set(idx_h[t])
        assert len(a) == len(b) and sorted(logits[t, list(a)]) == sorted(logits[t, list(b)]), "differs beyond an exact tie"
    check(host(w).astype(np.float32)[same], w_ref[same], "topk weights", max_rel=2e-3)


def test_moe_topk_tie_goes_to_higher_id(mx):
    logits = np.zeros((1, 64), np.float32)
    logits[0, [3, 9, 20, 41]] = 1.0          # four-way exact tie, k = 2 -> ids 20 and 41
    idx, w = mx.ops.moe_topk_from_logits(dev(logits).half(), 2)
    assert host(idx).tolist() == [[20, 41]]
    np.testing.assert_allclose(host(w).astype(np.float32), [[0.5, 0.5]], atol=1e-3)


@pytest.mark.parametrize("T,E,K", [(1, 32, 4), (64, 8, 2), (300, 128, 8), (2048, 128, 8)])
def test_moe_packing_device_equals_host(mx, T, E, K):
    rng = np.random.default_rng(T + E)
    p = np.arange(1, E + 1, dtype=np.float64) ** -1.1
    p /= p.sum()
    ids = np.stack([np.sort(rng.choice(E, size=K, replace=False, p=p)) for _ in range(T)]).astype(np.int32)
    w = f16(rng.random((T, K)).astype(np.float32))
    off_r, si_r, wp_r, t2p_r = O.build_moe_packing(ids, w, E)
    for decode in ([False, True] if T == 1 else [False]):
        off, si, wp, t2p = mx.ops.moe_build_packing_device(dev(ids), dev(w).half(), E, decode=decode)
        assert np.array_equal(host(off).view(np.uint32), off_r)
        assert np.array_equal(host(si), si_r)
        assert np.array_equal(host(t2p), t2p_r)
        assert np.array_equal(host(wp).astype(np.float32), wp_r)


def ref_q8_of(y_half):
    return O.quantize_q8_1(y_half.astype(np.float32))


@pytest.mark.parametrize("rows,hidden", [(1, 4096), (3, 2880), (17, 128), (2, 8192)])
def test_rms_norm_f32w_q8(mx, rows, hidden):
    x = f16(O.normal(9300, (rows, hidden)))
    w = (1.0 + O.normal(9301, (hidden,), 0.0, 0.1)).astype(np.float32)
    eps = 1e-6
    y, q8 = mx.ops.rms_norm_f32w_q8(dev(x).half(), dev(w), eps)
    y_h = host(y)
    xd = x.astype(np.float64)
    ref = xd / np.sqrt((xd * xd).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)
    check(y_h.astype(np.float32), ref, "rms_norm_f32w_q8 y", max_rel=1.5e-3)   # 1 fp16 ulp + rsqrt
    assert np.array_equal(host(q8), ref_q8_of(y_h).reshape(-1)), "q8 stream == quantize_q8_1(y)"
    assert np.array_equal(host(q8), host(mx.ops.quantize_q8_1(y))), "q8 stream == the standalone quantizer on y"


@pytest.mark.parametrize("rows,hidden", [(32, 128), (5, 256), (1, 4096)])
def test_gated_rms_norm_q8(mx, rows, hidden):
    x = O.normal(9400, (rows, hidden)).astype(np.float32)
    z = f16(O.normal(9401, (rows, hidden)))
    w = f16(1.0 + O.normal(9402, (hidden,), 0.0, 0.1))
    eps = 1e-6
    y, q8 = mx.ops.gated_rms_norm_q8(dev(x), dev(z).half(), dev(w).half(), eps)
    y_h = host(y)
    xd, zd = x.astype(np.float64), z.astype(np.float64)
    ref = w.astype(np.float64) * (xd / np.sqrt((xd * xd).mean(axis=1, keepdims=True) + eps)) * (zd / (1.0 + np.exp(-zd)))
    check(y_h.astype(np.float32), ref, "gated_rms_norm_q8 y", max_rel=1.5e-3)
    assert np.array_equal(host(q8), ref_q8_of(y_h).reshape(-1))


@pytest.mark.parametrize("n", [32, 2880 * 4, 768 * 131])
@pytest.mark.parametrize("oai", [False, True])
def test_swiglu_q8(mx, n, oai):
    """swiglu / swiglu_oai (src/ops/elementwise.cpp:449-492) with the fused block_q8_1x emitter: y against the
    closed form in fp64, the stream bit-identical to quantize_q8_1 of the rounded y."""
    g = f16(O.normal(9500 + n, (n,), 0.0, 3.0))        # sigma 3: the OAI clamp at 7 is exercised
    u = f16(O.normal(9501 + n, (n,), 0.0, 3.0))
    y, q8 = mx.ops.swiglu_q8(dev(g).half(), dev(u).half(), oai=oai)
    y_h = host(y)
    gd, ud = g.astype(np.float64), u.astype(np.float64)
    if oai:
        x, z = np.minimum(gd, 7.0), np.clip(ud, -7.0, 7.0)
        ref = x / (1.0 + np.exp(-1.702 * x)) * (z + 1.0)
    else:
        ref = gd / (1.0 + np.exp(-gd)) * ud
    check(y_h.astype(np.float32), ref, "swiglu%s y" % ("_oai" if oai else ""), max_rel=1.5e-3)
    assert np.array_equal(host(q8), ref_q8_of(y_h).reshape(-1)), "q8 stream == quantize_q8_1(y)"
    _, q8_only = mx.ops.swiglu_q8(dev(g).half(), dev(u).half(), oai=oai, want_y=False)
    assert torch.equal(q8_only, q8)
