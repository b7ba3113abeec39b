"""GPU parity: decode GEMV (T = 1 and batched) for Q4_K / Q6_K / Q8_0 / MXFP4,
int-dot kernels against the q8-chain oracle, float-activation kernels against
the float-chain oracle.  Gate: max_rel <= 1e-3 and cosine >= 0.99999."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host, weights

pytestmark = pytest.mark.gpu


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def acts(seed, T, K):
    """fp32 N(0,1) activations rounded to fp16 (what the fp16 entry points see)."""
    return O.round_fp16(O.normal(seed, (T, K), 0.0, 1.0))


def run_q8(mx, fmt, W, xq, K, N, T):
    name = O.FMT_NAMES[fmt]
    Wd, xd = dev(W), dev(xq)
    if fmt == O.MXFP4:
        qs, e = O.repack_mxfp4_to_soa(W)
        f = mx.ops.gemv_mxfp4_soa_q8 if T == 1 else mx.ops.gemv_mxfp4_soa_q8_batched
        args = (xd, dev(qs), dev(e), K, N) + ((T,) if T > 1 else ())
        return host(f(*args)).astype(np.float32)
    f = getattr(mx.ops, "gemv_%s_q8%s" % (name, "" if T == 1 else "_batched"))
    args = (xd, Wd, K, N) + ((T,) if T > 1 else ())
    return host(f(*args)).astype(np.float32)


SHAPES = [(256, 8), (512, 70), (2048, 512), (4096, 300), (2816, 33), (7936, 17)]


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0, O.MXFP4))
@pytest.mark.parametrize("K,N", SHAPES)
def test_gemv_q8_small_shapes(mx, fmt, K, N):
    if fmt in (O.Q8_0, O.MXFP4) and K == 2816:
        K = 2880  # K % 32 == 0 but not % 256 (gpt-oss hidden)
    if fmt in (O.Q8_0, O.MXFP4) and K == 7936:
        K = 7936 + 32  # K % 64 == 32: the last 64-element unit is half empty
    W = weights(fmt, 100 + fmt, N, K)
    x = acts(200 + K, 1, K)
    xq = host(mx.ops.quantize_q8_1(dev(x).half()))
    assert np.array_equal(xq, O.quantize_q8_1(x))
    ref = O.gemv_q8chain(fmt, W, xq, K, N)
    got = run_q8(mx, fmt, W, xq, K, N, 1)
    check(got, ref[0], "gemv_%s_q8 K=%d N=%d" % (O.FMT_NAMES[fmt], K, N))


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0, O.MXFP4))
@pytest.mark.parametrize("T", (2, 3, 4, 5, 7, 8, 11, 16))
def test_gemv_q8_batched(mx, fmt, T):
    K, N = (2880, 130) if fmt == O.MXFP4 else (2048, 130)
    W = weights(fmt, 300 + fmt, N, K)
    x = acts(400 + T, T, K)
    xq = O.quantize_q8_1(x)
    ref = O.gemv_q8chain(fmt, W, xq, K, N)
    got = run_q8(mx, fmt, W, xq, K, N, T)
    assert got.shape == (T, N)
    check(got, ref, "gemv_%s_q8_batched T=%d" % (O.FMT_NAMES[fmt], T))
    # per-row numerics identical to the T=1 kernel's gate (row t alone)
    one = run_q8(mx, fmt, W, xq[: K // 32 * 40], K, N, 1)
    check(one, ref[0], "row 0 alone")


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
def test_gemv_q8_multi_tile_K(mx, fmt):
    """K large enough that the activation is staged in several LDS tiles (T=8, K=14336)."""
    K, N, T = 14336, 64, 8
    W = weights(fmt, 500 + fmt, N, K)
    xq = O.quantize_q8_1(acts(501, T, K))
    check(run_q8(mx, fmt, W, xq, K, N, T), O.gemv_q8chain(fmt, W, xq, K, N), "multi-tile %s" % O.FMT_NAMES[fmt])


def test_gemv_q8_0_soa_matches_aos(mx):
    K, N = 4096, 96
    W = weights(O.Q8_0, 600, N, K)
    xq = O.quantize_q8_1(acts(601, 4, K))
    qs, d = O.repack_q8_0_to_soa(W)
    ref = O.gemv_q8chain(O.Q8_0, W, xq, K, N)
    soa1 = host(mx.ops.gemv_q8_0_soa_q8(dev(xq[: K // 32 * 40]), dev(qs), dev(d), K, N)).astype(np.float32)
    check(soa1, ref[0], "gemv_q8_0_soa_q8")
    soa4 = host(mx.ops.gemv_q8_0_soa_q8_batched(dev(xq), dev(qs), dev(d), K, N, 4)).astype(np.float32)
    check(soa4, ref, "gemv_q8_0_soa_q8_batched")
    aos4 = run_q8(mx, O.Q8_0, W, xq, K, N, 4)
    check(aos4, ref, "gemv_q8_0_q8_batched (GGUF blocks)")
    # the same products; planes and blocks are walked in different orders, so the fp32 sums differ in their last bits
    assert np.mean(aos4 == soa4) > 0.95 and np.abs(aos4 - soa4).max() <= 2e-3 * np.abs(ref).max()
    # a K outside the interleaved walk's reach (not a multiple of 512) takes the plain unit walk: the same bits as the blocks
    K2 = 4096 + 64
    W2 = weights(O.Q8_0, 602, N, K2)
    xq2 = O.quantize_q8_1(acts(603, 2, K2))
    qs2, d2 = O.repack_q8_0_to_soa(W2)
    soa2 = host(mx.ops.gemv_q8_0_soa_q8_batched(dev(xq2), dev(qs2), dev(d2), K2, N, 2)).astype(np.float32)
    check(soa2, O.gemv_q8chain(O.Q8_0, W2, xq2, K2, N), "gemv_q8_0_soa_q8_batched, K = %d" % K2)
    assert np.array_equal(run_q8(mx, O.Q8_0, W2, xq2, K2, N, 2), soa2)


def test_gemv_mxfp4_x2_bias(mx):
    K, N = 2880, 200
    Wg, Wu = weights(O.MXFP4, 700, N, K), weights(O.MXFP4, 701, N, K)
    xq = O.quantize_q8_1(acts(702, 1, K))
    bg, bu = O.normal(703, N), O.normal(704, N)
    gq, ge = O.repack_mxfp4_to_soa(Wg)
    uq, ue = O.repack_mxfp4_to_soa(Wu)
    gy, uy = mx.ops.gemv_mxfp4_soa_q8_x2(dev(xq), dev(gq), dev(ge), dev(uq), dev(ue), dev(bg), dev(bu), K, N)
    check(host(gy).astype(np.float32), O.gemv_q8chain(O.MXFP4, Wg, xq, K, N)[0] + bg, "x2 gate")
    check(host(uy).astype(np.float32), O.gemv_q8chain(O.MXFP4, Wu, xq, K, N)[0] + bu, "x2 up")
    gy2, uy2 = mx.ops.gemv_mxfp4_soa_q8_x2(dev(xq), dev(gq), dev(ge), dev(uq), dev(ue), None, None, K, N)
    assert np.array_equal(host(gy2), host(mx.ops.gemv_mxfp4_soa_q8(dev(xq), dev(gq), dev(ge), K, N)))


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
@pytest.mark.parametrize("K,N", [(256, 8), (2048, 300), (4096, 512)])
def test_gemv_float_activation(mx, fmt, K, N):
    """W4A16-style kernels vs the reference's CPU path (fp32 dequant + fp32 dot) and its fp64 twin."""
    name = O.FMT_NAMES[fmt]
    W = weights(fmt, 800 + fmt, N, K)
    x16 = acts(801, 1, K)
    ref64 = O.gemv_f64(fmt, W, x16, K, N)[0]
    got16 = host(getattr(mx.ops, "gemv_" + name)(dev(x16[0]).half(), dev(W), K, N)).astype(np.float32)
    check(got16, ref64, "gemv_%s fp16" % name)
    x32 = O.normal(802, (1, K), 0.0, 1.0)
    got32 = host(getattr(mx.ops, "gemv_" + name)(dev(x32[0]), dev(W), K, N))
    check(got32, O.gemv_f64(fmt, W, x32, K, N)[0], "gemv_%s fp32" % name, max_rel=1e-4)
    # the reference's own sequential-fp32 CPU result sits within fp32 accumulation noise of ours
    check(got32, O.gemv_f32chain(fmt, W, x32, K, N)[0], "vs fp32 chain", max_rel=2e-4)


def test_gemv_mxfp4_f16(mx):
    K, N = 2880, 256
    W = weights(O.MXFP4, 900, N, K)
    x = acts(901, 1, K)
    qs, e = O.repack_mxfp4_to_soa(W)
    got = host(mx.ops.gemv_mxfp4_soa_f16(dev(x[0]).half(), dev(qs), dev(e), K, N)).astype(np.float32)
    check(got, O.gemv_f64(O.MXFP4, W, x, K, N)[0], "gemv_mxfp4_soa_f16")


def test_gemv_q8_fp32_out_tight(mx):
    """fp32-output twins: the fp32 fold must sit within 2e-5 of the fp64 q8-chain."""
    K, N = 4096, 256
    for fmt in (O.Q4_K, O.Q6_K, O.Q8_0):
        W = weights(fmt, 1000 + fmt, N, K)
        xq = O.quantize_q8_1(acts(1001, 1, K))
        got = host(mx.ops.gemv_q8_f32(O.FMT_NAMES[fmt], dev(xq), dev(W), K, N))
        check(got, O.gemv_q8chain(fmt, W, xq, K, N)[0], "gemv_%s_q8_f32" % O.FMT_NAMES[fmt], max_rel=1e-4)


def test_gemv_integer_part_exact(mx):
    """Weights with unit scales make the fold exact, so the kernel's integer dot
    must equal the brute-force int64 dot bit for bit (Q8_0: d = 1)."""
    K, N = 1024, 40
    qs = (O.rand_bytes(1100, N * K).view(np.int8)).reshape(N, K)
    blk = np.zeros((N, K // 32, 34), np.uint8)
    blk[:, :, 0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    blk[:, :, 2:] = qs.reshape(N, K // 32, 32).view(np.uint8)
    xq = np.zeros((K // 32, 40), np.uint8)
    q8 = O.rand_bytes(1101, K).view(np.int8).reshape(K // 32, 32)
    xq[:, 0:4] = np.array([1.0], np.float32).view(np.uint8)
    xq[:, 8:] = q8.view(np.uint8)
    got = host(mx.ops.gemv_q8_f32("q8_0", dev(xq.ravel()), dev(blk.reshape(N, -1)), K, N))
    exact = qs.astype(np.int64) @ q8.reshape(K).astype(np.int64)
    assert np.array_equal(got.astype(np.int64), exact)   # |sum| < 2^24, so fp32 holds it exactly


def test_full_size_properties_config1(mx):
    """BASELINE config 1 at full size (Q4_K 4096x4096): linearity in the
    activation scale and agreement between the int-dot and float chains at the
    activation-quantisation noise level (max_err/rms < 3e-2, tests/unit/q8dot_test.cpp:120-135)."""
    K = N = 4096
    W = weights(O.Q4_K, 1200, N, K)
    x = acts(1201, 1, K)
    Wd = dev(W)
    yq = host(mx.ops.gemv_q4_K_q8(mx.ops.quantize_q8_1(dev(x).half()), Wd, K, N)).astype(np.float64)
    yf = host(mx.ops.gemv_q4_K(dev(x[0]), Wd, K, N)).astype(np.float64)
    rms = np.sqrt(np.mean(yf ** 2))
    assert np.abs(yq - yf).max() / rms < 3e-2
    y2 = host(mx.ops.gemv_q4_K(dev(2 * x[0]), Wd, K, N)).astype(np.float64)
    assert np.allclose(y2, 2 * yf, rtol=1e-6, atol=1e-6 * rms)
    check(yf, O.gemv_f64(O.Q4_K, W, x, K, N)[0], "config1 float chain", max_rel=1e-4)
    check(yq, O.gemv_q8chain(O.Q4_K, W, O.quantize_q8_1(x), K, N)[0], "config1 q8 chain")


@pytest.mark.parametrize("fmt,K,N,T", [("q4_K", 1024, 96, 5), ("q4_K", 4096, 256, 16), ("q6_K", 2048, 130, 3), ("q6_K", 768, 64, 8)])
def test_gemv_kquant_q8s_batched(mx, fmt, K, N, T):
    """block_q8_1s activation rows (stored half sums, src/ops/gemv_q8dot.cpp:483-597) at the gate against
    the q8-chain oracle.  Q6_K folds per 16 elements, so s0 / s1 are exactly the numbers the
    block_q8_1x form recomputes (bit-identical); Q4_K folds per 32 with s0 + s1, one more fp32
    rounding than d * float(sum32)."""
    F = {"q4_K": O.Q4_K, "q6_K": O.Q6_K}[fmt]
    W = weights(F, 700 + N, N, K)
    x = O.normal(701 + T, (T, K)).astype(np.float32)
    xd = dev(x)
    xq, xqs = mx.ops.quantize_q8_1(xd), mx.ops.quantize_q8_1s(xd)
    a = mx.ops.gemv_kquant_q8s_batched(fmt, xqs, dev(W), K, N, T)
    b = getattr(mx.ops, "gemv_%s_q8_batched" % fmt)(xq, dev(W), K, N, T)
    if fmt == "q6_K":
        assert torch.equal(a, b)
    else:
        assert (a == b).float().mean().item() > 0.99
    ref = O.gemv_q8schain(F, W, host(xqs), K, N)      # min terms on the stored half sums, as the kernel folds them
    check(host(a).astype(np.float32), ref, "%s q8s batched T=%d" % (fmt, T))


@pytest.mark.parametrize("K,N", [(2048, 32), (4096, 1000)])
def test_gemv_q4_K_dual_and_down_accum(mx, K, N):
    """gemv_q4_K_dual == two single GEMVs, bit for bit (same kernel, same order);
    gemv_q4_K_down_accum: y = half(float(y) + float(sh_g) * acc) (src/ops/gemv_q4k.cpp:398-472)."""
    Wa, Wb = weights(O.Q4_K, 1100, N, K), weights(O.Q4_K, 1101, N, K)
    x16 = acts(1102, 1, K)
    xd = dev(x16[0]).half()
    ya, yb = mx.ops.gemv_q4_K_dual(xd, dev(Wa), dev(Wb), K, N)
    assert torch.equal(ya, mx.ops.gemv_q4_K(xd, dev(Wa), K, N)) and torch.equal(yb, mx.ops.gemv_q4_K(xd, dev(Wb), K, N))
    check(host(yb).astype(np.float32), O.gemv_f64(O.Q4_K, Wb, x16, K, N)[0], "dual second output")
    y0 = O.round_fp16(O.normal(1103, (N,), 0.0, 1.0))
    g = O.round_fp16(np.array([0.37], np.float32))
    y = mx.ops.gemv_q4_K_down_accum(xd, dev(Wa), dev(g).half(), dev(y0).half(), K, N)
    ref = y0.astype(np.float64) + float(g[0]) * O.gemv_f64(O.Q4_K, Wa, x16, K, N)[0]
    check(host(y).astype(np.float32), ref, "down_accum")


@pytest.mark.parametrize("K,N", [(2048, 512), (4096, 33)])
def test_gemv_q4_K_shexp_gate_up(mx, K, N):
    """y_h = half(silu(W_gate.A) * (W_up.A)) with fp32 sums, plus the gate scalar
    sigmoid(W_shg . A) from the extra workgroup (src/ops/gemv_q4k.cpp:288-395)."""
    Wg, Wu = weights(O.Q4_K, 1200, N, K), weights(O.Q4_K, 1201, N, K)
    x16 = acts(1202, 1, K)
    wshg = O.normal(1203, (K,), 0.0, 0.03)
    y_h, sh_g = mx.ops.gemv_q4_K_shexp_gate_up(dev(x16[0]).half(), dev(Wg), dev(Wu), dev(wshg), K, N)
    g = O.gemv_f64(O.Q4_K, Wg, x16, K, N)[0]
    u = O.gemv_f64(O.Q4_K, Wu, x16, K, N)[0]
    check(host(y_h).astype(np.float32), g / (1.0 + np.exp(-g)) * u, "shexp silu(g)*u")
    dot = float(np.dot(x16[0].astype(np.float64), wshg.astype(np.float64)))
    ref_g = 1.0 / (1.0 + np.exp(-dot))
    assert abs(float(host(sh_g)[0]) - ref_g) <= 1e-3 * ref_g + 2.0 ** -11


@pytest.mark.parametrize("K,N", [(2048, 32), (2048, 48)])
def test_gemv_q4_K_dual_ssm_gbeta(mx, K, N):
    """alpha/beta sums round through fp16, then g = A_log * softplus(a + dt_bias), beta = sigmoid(b)
    (src/ops/gemv_q4k.cpp:480-590).  The fp16 rounding point is checked by feeding the kernel's own
    dual GEMV outputs (bit-identical sums) through the closed form."""
    Wa, Wb = weights(O.Q4_K, 1210, N, K), weights(O.Q4_K, 1211, N, K)
    x16 = acts(1212, 1, K)
    A_log = -np.exp(O.normal(1213, (N,), 0.0, 0.5)).astype(np.float32)
    dt_bias = O.normal(1214, (N,), 0.0, 1.0)
    xd = dev(x16[0]).half()
    g, beta = mx.ops.gemv_q4_K_dual_ssm_gbeta(xd, dev(Wa), dev(Wb), dev(A_log), dev(dt_bias), K, N)
    ya, yb = mx.ops.gemv_q4_K_dual(xd, dev(Wa), dev(Wb), K, N)
    a = host(ya).astype(np.float64) + dt_bias.astype(np.float64)
    ref_g = A_log.astype(np.float64) * (np.maximum(a, 0.0) + np.log1p(np.exp(-np.abs(a))))
    ref_b = 1.0 / (1.0 + np.exp(-host(yb).astype(np.float64)))
    assert np.max(np.abs(host(g) - ref_g)) <= 1e-5 * np.max(np.abs(ref_g))
    assert np.max(np.abs(host(beta) - ref_b)) <= 1e-5
    # and the sums themselves against the float-chain oracle
    check(host(ya).astype(np.float32), O.gemv_f64(O.Q4_K, Wa, x16, K, N)[0], "alpha sums")


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
def test_gemv_q8_x2_equals_two_single_launches(mx, fmt):
    """Fused gate + up (the launch shape of gemv_mxfp4_soa_q8_x2, include/ie/ops.hpp:503-513): each output is
    bit-identical to the single-matrix kernel's, which is gated against the oracle above."""
    K, N = 2048, 300
    name = O.FMT_NAMES[fmt]
    Wa, Wb = weights(fmt, 1400 + fmt, N, K), weights(fmt, 1410 + fmt, N, K)
    xq = dev(O.quantize_q8_1(acts(1420, 1, K)))
    single = getattr(mx.ops, "gemv_%s_q8" % name)
    ya, yb = mx.ops.gemv_q8_x2(name, xq, dev(Wa), dev(Wb), K, N)
    assert torch.equal(ya, single(xq, dev(Wa), K, N)) and torch.equal(yb, single(xq, dev(Wb), K, N))
    if fmt == O.Q8_0:
        sa, sb = [tuple(dev(p) for p in O.repack_q8_0_to_soa(W)) for W in (Wa, Wb)]
        ya2, yb2 = mx.ops.gemv_q8_x2("q8_0_soa", xq, sa, sb, K, N)
        assert torch.equal(ya2, mx.ops.gemv_q8_0_soa_q8(xq, sa[0], sa[1], K, N)) and torch.equal(yb2, mx.ops.gemv_q8_0_soa_q8(xq, sb[0], sb[1], K, N))


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
@pytest.mark.parametrize("K,N", [(2048, 320), (4096, 1056), (1280, 96), (14336, 64)])
def test_decode_ffn_forms_equal_the_launch_chain(mx, fmt, K, N):
    """gate + up + SwiGLU in one launch, and GEMVs that quantize the fp16 activation row while staging it: the bits of
    quantize_q8_1 -> gemv x2 -> swiglu and of quantize_q8_1 -> gemv, whose parts are gated against the oracle above.
    K = 2048 / 4096 / 1280 walk 32, 64 and 16 lanes per row (1280 leaves lanes of the last round without a unit);
    K = 14336 with few rows is the down-projection shape (Q8_0 planes: the workgroup-wide walk in both forms)."""
    ops = mx.ops
    name = O.FMT_NAMES[fmt]
    Wg, Wu = weights(fmt, 1600 + fmt, N, K), weights(fmt, 1610 + fmt, N, K)
    x16 = dev(acts(1620 + K, 1, K)).half()
    xq = ops.quantize_q8_1(x16)
    forms = [(name, dev(Wg), dev(Wu))]
    if fmt == O.Q8_0:
        forms.append(("q8_0_soa",) + tuple(tuple(dev(p) for p in O.repack_q8_0_to_soa(W)) for W in (Wg, Wu)))
    for nm, g_w, u_w in forms:
        g, u = ops.gemv_q8_x2(nm, xq, g_w, u_w, K, N)
        h_chain, hq_chain = ops.swiglu_q8(g, u)
        h1 = ops.gemv_x2_silu(nm, xq, g_w, u_w, K, N)
        h2 = ops.gemv_x2_silu(nm, x16.reshape(-1), g_w, u_w, K, N)
        assert torch.equal(h1, h2), "%s: fused gate/up/silu on the fp16 row != on the q8 row" % nm
        if K < 8192:   # long rows of a short matrix: the separate launches walk a row with the whole workgroup, another summation order
            assert torch.equal(h1, h_chain), "%s: fused gate/up/silu != the launch chain" % nm
        single = (lambda w: ops.gemv_q8_0_soa_q8(xq, w[0], w[1], K, N)) if nm == "q8_0_soa" else (lambda w: getattr(ops, "gemv_%s_q8" % nm)(xq, w, K, N))
        assert torch.equal(ops.gemv_f16q8(nm, x16.reshape(-1), g_w, K, N), single(g_w)), "%s: gemv on the fp16 row != quantize + gemv" % nm
    # and the fused result against the oracle chain directly (q8-chain dots, fp16 roundings of g and u, SwiGLU)
    xq_h = host(xq)
    g_ref = f16(O.gemv_q8chain(fmt, Wg, xq_h, K, N)[0]).astype(np.float32)
    u_ref = f16(O.gemv_q8chain(fmt, Wu, xq_h, K, N)[0]).astype(np.float32)
    check(host(h1).astype(np.float32), O.swiglu_np(g_ref, u_ref), "fused gate/up/silu vs oracle", max_rel=3e-3)


@pytest.mark.parametrize("fmt,K", [(O.Q4_K, 14336), (O.Q8_0, 14336), (O.Q8_0, 14368), (O.Q8_0, 8192 + 96), (O.Q4_K, 8192)])
def test_gemv_long_rows_few_of_them(mx, fmt, K):
    """T = 1 on long rows with few of them takes the kernel that keeps two rounds of loads rotating; K = 14368 and 8288
    leave a half unit and lanes without a unit in the last round.  Against the q8-chain oracle, AoS and SoA forms."""
    N = 300
    W = weights(fmt, 1800 + fmt, N, K)
    xq = O.quantize_q8_1(acts(1810 + K, 1, K))
    ref = O.gemv_q8chain(fmt, W, xq, K, N)
    name = O.FMT_NAMES[fmt]
    got = getattr(mx.ops, "gemv_%s_q8" % name)(dev(xq), dev(W), K, N)
    check(host(got).astype(np.float32), ref[0], "gemv_%s_q8 K=%d N=%d" % (name, K, N))
    if fmt == O.Q8_0:
        qs, d = (dev(p) for p in O.repack_q8_0_to_soa(W))
        got2 = mx.ops.gemv_q8_0_soa_q8(dev(xq), qs, d, K, N)
        check(host(got2).astype(np.float32), ref[0], "gemv_q8_0_soa_q8 K=%d N=%d" % (K, N))
        # blocks and planes walk a long row in different orders (lane groups / the whole workgroup): same products,
        # fp32 sums that differ in the last bits, so nearly every fp16 output is the same and none is far
        a, b = host(got).astype(np.float32), host(got2).astype(np.float32)
        assert (a == b).mean() > 0.97 and np.abs(a - b).max() <= 2e-3 * np.abs(a).max()


@pytest.mark.parametrize("K,N", [(1312, 96), (4128, 64), (14368, 32)])
def test_decode_ffn_forms_half_unit_tail(mx, K, N):
    """Q8_0 rows whose length is an odd number of 32-element blocks (a half unit at the end of the row), fp16 row
    quantized while staged: the same bits as the launch chain, AoS and SoA."""
    ops = mx.ops
    Wg, Wu = weights(O.Q8_0, 1900 + K, N, K), weights(O.Q8_0, 1910 + K, N, K)
    x16 = dev(acts(1920 + K, 1, K)).half().reshape(-1)
    xq = ops.quantize_q8_1(x16)
    for nm, g_w, u_w in (("q8_0", dev(Wg), dev(Wu)),
                         ("q8_0_soa",) + tuple(tuple(dev(p) for p in O.repack_q8_0_to_soa(W)) for W in (Wg, Wu))):
        g, u = ops.gemv_q8_x2(nm, xq, g_w, u_w, K, N)
        h_chain, _ = ops.swiglu_q8(g, u)
        assert torch.equal(ops.gemv_x2_silu(nm, x16, g_w, u_w, K, N), h_chain)
        assert torch.equal(ops.gemv_x2_silu(nm, xq, g_w, u_w, K, N), h_chain)
        assert torch.equal(ops.gemv_f16q8(nm, x16, g_w, K, N), g)
    check(host(g).astype(np.float32), O.gemv_q8chain(O.Q8_0, Wg, host(xq), K, N)[0], "gate K=%d" % K)


def test_decode_ffn_forms_reject_bad_arguments(mx):
    ops = mx.ops
    K, N = 512, 64
    W = dev(weights(O.Q4_K, 1700, N, K))
    x16 = dev(acts(1701, 1, K)).half().reshape(-1)
    with pytest.raises(ops.MxError):
        ops.gemv_f16q8("q4_K", x16, W, K + 32, N)                      # K not a multiple of 256
    with pytest.raises(ops.MxError):
        ops.gemv_f16q8("q4_K", x16[4:], W, K, N)                       # fp16 row not 16-byte aligned
    big = 65536
    with pytest.raises(ops.MxError):
        ops.gemv_f16q8("q6_K", torch.zeros(big, dtype=torch.float16, device="cuda"), torch.zeros(big // 256 * 210, dtype=torch.uint8, device="cuda"), big, 1)   # row longer than one LDS tile


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K, O.Q8_0))
@pytest.mark.parametrize("T", (2, 5, 8, 13))
def test_gemv_q8_batched_long_rows_split_k(mx, fmt, T):
    """Batched launches at K >= 8192 with few rows run as (row groups x K slices) plus a small reduction launch:
    results against the q8-chain oracle, and identical from launch to launch (the slices are added in slice order)."""
    K, N = 14336, 200
    W = weights(fmt, 1500 + fmt, N, K)
    xq = O.quantize_q8_1(acts(1510 + T, T, K))
    ref = O.gemv_q8chain(fmt, W, xq, K, N)
    first = run_q8(mx, fmt, W, xq, K, N, T)
    for t in range(T):
        check(first[t], ref[t], "%s K=%d T=%d row %d" % (O.FMT_NAMES[fmt], K, T, t))
    for _ in range(3):
        assert np.array_equal(run_q8(mx, fmt, W, xq, K, N, T), first)


@pytest.mark.parametrize("K,N,seed", [(12288, 4096, 0x6C01), (4096, 2048, 0x6C02), (12288 + 256, 1024, 0x6C03), (2304, 257, 0x6C04), (2048, 512, 0x6C05)])
def test_gemv_q6_K_q8_reference_ktiled_shapes(mx, K, N, seed):
    """The five shapes of the reference's K-tiled Q6_K test (tests/gemv_q6k_ktiled_test.cpp:195-208: the qwen3-8b
    ffn_down decode shape, a fitting K, a partial last K tile, odd N, exactly one tile), against the q8-chain oracle
    as there (:89-103)."""
    W = weights(O.Q6_K, seed, N, K)
    xq = O.quantize_q8_1(acts(seed + 16, 1, K))
    check(run_q8(mx, O.Q6_K, W, xq, K, N, 1), O.gemv_q8chain(O.Q6_K, W, xq, K, N)[0], "gemv_q6_K_q8 K=%d N=%d" % (K, N))


def test_probe_stream_read(mx):
    """The bandwidth yardstick: launches on any 16-byte multiple, rejects what it cannot read whole."""
    buf = torch.empty(1 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
    for n in (16, 4096 + 16, 1 << 20):
        mx.ops.probe_stream_read(buf, n)
    torch.cuda.synchronize()
    with pytest.raises(mx.ops.MxError):
        mx.ops.probe_stream_read(buf, 24)          # not a multiple of 16
    with pytest.raises(mx.ops.MxError):
        mx.ops.probe_stream_read(buf[8:], 16)      # misaligned
