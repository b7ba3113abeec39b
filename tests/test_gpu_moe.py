"""GPU parity: expert-indexed GEMV kernels (MoE decode with device-side expert ids
and the expert-grouped form) for MXFP4 experts (gpt-oss shape family, BASELINE
config 4) and Q8_0 SoA experts, stage by stage against the oracle, and the whole
layer against a per-token per-expert brute-force loop."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import check, dev, host

pytestmark = pytest.mark.gpu


_EXPERTS = {}


def make_experts(fmt, seed, E, N, K):
    """E experts of [N, K] weights -> (AoS blocks [E, N, row_bytes], SoA planes).  Kept per (fmt, seed, shape): the
    full-size cases share their banks."""
    key = (fmt, seed, E, N, K)
    if key not in _EXPERTS:
        W = np.stack([O.quantize(fmt, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
        if fmt == O.MXFP4:
            qs, sc = O.repack_mxfp4_to_soa(W)
            _EXPERTS[key] = (W, qs, sc, N * K // 2, N * K // 32)
        else:
            qs, sc = O.repack_q8_0_to_soa(W)
            _EXPERTS[key] = (W, qs, sc, N * K, N * K // 32)
        if N * K * E < (1 << 24):
            return _EXPERTS.pop(key)
    return _EXPERTS[key]


def route(seed, T, E, k):
    ids, w = O.route_from_logits(O.normal(seed, (T, E)), k)
    return ids, w


def f16(a):
    return O.round_fp16(np.asarray(a, np.float32))


def check_rows(a, b, what):
    """Two fp16 results of the same arithmetic in different fp32 summation orders (vector-ALU decode kernels, matrix-core
    grouped kernels): equal up to a few fp16 ulps where fp32 noise crosses a rounding boundary (and is then re-quantised
    downstream: after gate/up, quantize, down and the weighted sum about 3 % of a layer's outputs move by one ulp)."""
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    rms = float(np.sqrt(np.mean(b32 * b32)))
    frac_equal = float(np.mean(a == b))
    err = float(np.abs(a32 - b32).max() / rms)
    print("%s: %.4f bit-equal, max_abs/rms=%.2e" % (what, frac_equal, err), flush=True)
    assert frac_equal > 0.95 and err < 1e-2, what


# Stages that mirror the reference's chain of fp16 roundings (half(acc + bias), then the fp16
# activation or bias add) can land one fp16 ulp (2^-10 relative) away from the fp64 evaluation
# when an intermediate value sits next to a rounding boundary; their gate is 2 fp16 ulps.
CHAIN_GATE = 2e-3


def sum_noise(acc, other=0.0):
    """What the order of an fp32 accumulation can move a sum by: a few fp32 ulps of the partial sums, whose scale is
    the row's rms and the two addends.  Implementations (the reference's sub-group reductions included) differ by
    this much before the fp16 rounding, and for an element whose acc + bias nearly cancels that exceeds one fp16 ulp
    of the small result."""
    a = np.asarray(acc, np.float64)
    return 2.0 ** -18 * (np.abs(a) + np.abs(other) + float(np.sqrt(np.mean(a * a))))


def f16_candidates(s64, eta):
    """fp16 values a chain may hold for the fp64 sum s64 known to +-eta: one ulp beyond the rounded ends."""
    inf = np.float16(np.inf)
    return (np.nextafter(f16(s64 - eta).astype(np.float16), -inf), f16(s64).astype(np.float16), np.nextafter(f16(s64 + eta).astype(np.float16), inf))


def ref_gate_up_oai(Wg, Wu, bg, bu, e, xq_row, K, N):
    """-> (lo, hi, g16, u16, eta_g, eta_u): envelope of half(swiglu_oai(g16, u16)) over the admissible roundings of the
    two intermediates: the fp32 device sums may sit on the other side of an fp16 rounding boundary than
    the fp64 oracle sums (by the accumulation-order noise `sum_noise`, then one fp16 ulp), and swiglu_oai's (up + 1)
    factor can amplify that ulp without bound in relative terms, so the stage is checked against the set of results the
    reference chain can produce when g16 / u16 move that far."""
    ag = O.gemv_q8chain(O.MXFP4, Wg[e], xq_row, K, N)[0].astype(np.float64)
    au = O.gemv_q8chain(O.MXFP4, Wu[e], xq_row, K, N)[0].astype(np.float64)
    eta_g, eta_u = sum_noise(ag, bg[e]), sum_noise(au, bu[e])
    gc, uc = f16_candidates(ag + bg[e], eta_g), f16_candidates(au + bu[e], eta_u)
    outs = [f16(O.swiglu_oai_np(gg.astype(np.float32), uu.astype(np.float32))) for gg in gc for uu in uc]
    return np.min(outs, axis=0), np.max(outs, axis=0), gc[1].astype(np.float32), uc[1].astype(np.float32), eta_g, eta_u


def ulp16(v):
    """Spacing of fp16 at |v| (normal range)."""
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(v).astype(np.float64), 2.0 ** -14))) - 10)


def explained_outliers(got, centre, budget, what, min_frac):
    """The envelope says WHETHER every element is a value the reference chain can produce; this says HOW FAR the
    results sit from the chain evaluated in fp64: the share of elements within the 1e-3 gate is printed and bounded
    below, and each element beyond the gate must be explained by its own cancellation, i.e. lie within the first-order
    effect `budget` of one-ulp moves of the fp16 intermediates (large only where z + 1 or acc + bias nearly cancels)."""
    r = centre.astype(np.float64)
    rms = float(np.sqrt(np.mean(r * r)))
    den = np.maximum(np.abs(r), max(1e-2 * rms, 2.0 ** -14))
    rel = np.abs(got.astype(np.float64) - r) / den
    out = rel > 1e-3
    frac = 1.0 - out.mean()
    worst = float((rel[out] / (budget / den)[out]).max()) if out.any() else 0.0
    print("%s: %.4f %% of %d elements within 1e-3 of the fp64 chain; %d beyond, largest error / explained budget = %.2f"
          % (what, 100 * frac, rel.size, int(out.sum()), worst), flush=True)
    assert frac >= min_frac, (what, frac)
    assert np.all(rel[out] <= 1.5 * (budget / den)[out]), (what, "an element beyond the gate is not explained by cancellation")


def check_envelope(got, lo, hi, what):
    got16 = got.astype(np.float16)
    inf = np.float16(np.inf)
    ok = (got16 >= np.nextafter(lo.astype(np.float16), -inf)) & (got16 <= np.nextafter(hi.astype(np.float16), inf))
    print("%s: %d / %d inside the 1-ulp envelope" % (what, ok.sum(), ok.size), flush=True)
    assert ok.all(), (what, np.argwhere(~ok)[:5], got[~ok][:5], lo[~ok][:5], hi[~ok][:5])



def check_gate_up_oai_rows(got, env, what, min_frac=0.999):
    """Rows of half(swiglu_oai(half(g + bias), half(u + bias))) against the oracle: envelope of the reference chain,
    cosine, and every element beyond 1e-3 of the fp64 chain explained by its own cancellation.  `env` holds one
    ref_gate_up_oai() result per row."""
    check_envelope(got, np.stack([e[0] for e in env]), np.stack([e[1] for e in env]), what)
    g16, u16 = np.stack([e[2] for e in env]).astype(np.float64), np.stack([e[3] for e in env]).astype(np.float64)
    centre = f16(O.swiglu_oai_np(g16.astype(np.float32), u16.astype(np.float32)))
    check(got, centre, "  ... cosine against the fp64 chain", max_rel=1.0, cos=0.99999)
    # first-order effect of one-ulp moves of g16 and u16 plus the output's own rounding
    xg, z = np.minimum(g16, 7.0), np.clip(u16, -7.0, 7.0)
    sg = 1.0 / (1.0 + np.exp(-1.702 * xg))
    glu, dglu = xg * sg, np.where(g16 < 7.0, sg * (1.0 + 1.702 * xg * (1.0 - sg)), 0.0)
    eta_g, eta_u = np.stack([e[4] for e in env]), np.stack([e[5] for e in env])
    budget = ((ulp16(g16) + eta_g) * np.abs(dglu) * np.abs(z + 1.0) + np.where(np.abs(u16) < 7.0, ulp16(u16) + eta_u, 0.0) * np.abs(glu)
              + ulp16(centre))
    explained_outliers(got, centre, budget, what, min_frac)


def check_down_bias_rows(got, Wd, bd, experts, hq_rows, EF, H, what, min_frac=0.999):
    """Rows of half(half(acc) + bias) against the oracle: `experts[r]` is the expert of row r, `hq_rows` the block_q8_1x
    bytes the kernel read (one row of EF / 32 * 40 bytes per output row)."""
    hrb = EF // 32 * 40
    lo, hi, ctr, a16s = [], [], [], []
    for r, e in enumerate(experts):   # envelope over half(acc) moving by one ulp (the sum with the bias can cancel)
        acc = O.gemv_q8chain(O.MXFP4, Wd[e], hq_rows[r * hrb:(r + 1) * hrb], EF, H)[0].astype(np.float64)
        cands = f16_candidates(acc, sum_noise(acc))
        c = [f16(v.astype(np.float32) + bd[e]) for v in cands]
        lo.append(np.min(c, axis=0))
        hi.append(np.max(c, axis=0))
        ctr.append(c[1])
        a16s.append(cands[1].astype(np.float32))
    check_envelope(got, np.stack(lo), np.stack(hi), what)
    ctr = np.stack(ctr)
    explained_outliers(got, ctr, ulp16(np.stack(a16s)) + ulp16(ctr), what, min_frac)


@pytest.mark.parametrize("T,H,EF,E,Kt", [(1, 2880, 2880, 32, 4), (3, 512, 320, 6, 2), (32, 704, 384, 8, 4), (48, 704, 384, 4, 2), (32, 2880, 2880, 32, 4)])
def test_moe_mxfp4_decode_and_grouped(mx, T, H, EF, E, Kt):
    """gpt-oss style layer: gate/up (+bias, swiglu_oai) -> quantize -> down (+bias) -> weighted reduce.
    H=EF=2880, E=32, top-4 at T=1 and T=32 are BASELINE config 4's two cases at full size (every packed row of
    both is recomputed by the oracle)."""
    ops = mx.ops
    Wg, gq, ge, qs_st, e_st = make_experts(O.MXFP4, 100, E, EF, H)
    Wu, uq, ue, _, _ = make_experts(O.MXFP4, 200, E, EF, H)
    Wd, dq, de, dqs_st, de_st = make_experts(O.MXFP4, 300, E, H, EF)
    bg, bu, bd = O.normal(1, (E, EF)), O.normal(2, (E, EF)), O.normal(3, (E, H))
    x = f16(O.normal(4, (T, H)))
    ids, w = route(5, T, E, Kt)
    xq = O.quantize_q8_1(x)
    rb = H // 32 * 40
    D = dict(gq=dev(gq), ge=dev(ge), uq=dev(uq), ue=dev(ue), dq=dev(dq), de=dev(de), bg=dev(bg), bu=dev(bu), bd=dev(bd))
    # ---- decode form: expert ids stay on the device
    h = ops.moe_gate_up_oai_mxfp4(dev(xq), D["gq"], D["ge"], D["uq"], D["ue"], qs_st, e_st, D["bg"], D["bu"], dev(ids.ravel()), T, Kt, H, EF, E)
    h_h = host(h).astype(np.float32)
    env = [ref_gate_up_oai(Wg, Wu, bg, bu, ids[t, k], xq[t * rb:(t + 1) * rb], H, EF) for t in range(T) for k in range(Kt)]
    check_gate_up_oai_rows(h_h, env, "moe gate_up swiglu_oai (decode) T=%d" % T)
    hq = ops.quantize_q8_1(h)
    hq_h = host(hq)
    assert np.array_equal(hq_h, O.quantize_q8_1(h_h))
    out = ops.moe_down_mxfp4(hq, D["dq"], D["de"], dqs_st, de_st, D["bd"], dev(ids.ravel()), T, Kt, EF, H, E)
    out_h = host(out).astype(np.float32)
    # h taken as fp16 and quantized while staged: the same q8 tile, so the same bits out
    out_f = ops.moe_down_mxfp4_f16(h, D["dq"], D["de"], dqs_st, de_st, D["bd"], dev(ids.ravel()), T, Kt, EF, H, E)
    assert np.array_equal(host(out_f), host(out)), "down on fp16 h != quantize + down"
    check_down_bias_rows(out_h, Wd, bd, ids.ravel(), hq_h, EF, H, "moe down + bias (decode) T=%d" % T)
    y = torch.zeros((T, H), dtype=torch.float16, device="cuda")
    ident = dev(np.arange(T * Kt, dtype=np.uint32))
    ops.moe_prefill_reduce(out, ident, dev(w.ravel()).half(), y, T, Kt, H)
    w16 = f16(w)
    y_ref = f16((w16[:, :, None] * out_h.reshape(T, Kt, H)).sum(axis=1))
    check(host(y).astype(np.float32), y_ref, "moe weighted reduce")
    # ---- grouped form: host packing, expert-sorted rows, every expert's weights streamed once
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    assert all(np.array_equal(a, b) for a, b in zip((off, si, wp, t2p), O.build_moe_packing(ids, w, E)))
    TK = T * Kt
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, H)
    assert np.array_equal(host(xp), x[si].astype(np.float16))
    xpq = ops.quantize_q8_1(xp)
    hp = ops.moe_grouped_gate_up_oai_mxfp4(xpq, D["gq"], D["ge"], D["uq"], D["ue"], qs_st, e_st, D["bg"], D["bu"], dev(off), TK, E, H, EF)
    # The grouped kernels (for H, EF >= 256 the scaled FP8 x FP4 matrix instruction) against the oracle itself: packed row
    # t2p[slot] holds the same token and expert as decode slot `slot`, and its q8 row is the same bytes, so the
    # per-slot envelopes apply to it unchanged.
    assert np.array_equal(host(xpq).reshape(TK, -1)[t2p].ravel(), xq.reshape(T, -1).repeat(Kt, axis=0).ravel())
    check_gate_up_oai_rows(host(hp).astype(np.float32)[t2p], env, "moe gate_up swiglu_oai (grouped) T=%d" % T)
    check_rows(host(hp)[t2p], host(h), "grouped gate_up vs decode rows")
    hpq = ops.quantize_q8_1(hp)
    hpq_h = host(hpq)
    assert np.array_equal(hpq_h, O.quantize_q8_1(host(hp).astype(np.float32)))
    op = ops.moe_grouped_down_mxfp4(hpq, D["dq"], D["de"], dqs_st, de_st, D["bd"], dev(off), TK, E, H, EF)
    row_expert = np.repeat(np.arange(E), np.diff(off.astype(np.int64)))
    check_down_bias_rows(host(op).astype(np.float32), Wd, bd, row_expert, hpq_h, EF, H, "moe down + bias (grouped) T=%d" % T)
    check_rows(host(op)[t2p], host(out), "grouped down vs decode rows")
    op_f = ops.moe_grouped_down_mxfp4_f16(hp, D["dq"], D["de"], dqs_st, de_st, D["bd"], dev(off), TK, E, H, EF)
    assert np.array_equal(host(op_f), host(op)), "grouped down on fp16 h != quantize + grouped down"
    y2 = torch.zeros((T, H), dtype=torch.float16, device="cuda")
    ops.moe_prefill_reduce(op, dev(t2p.astype(np.uint32)), dev(wp).half(), y2, T, Kt, H)
    check_rows(host(y2), host(y), "grouped layer output == decode layer output")


@pytest.mark.parametrize("T,H,EF,E,Kt", [(1, 2048, 768, 16, 8), (5, 512, 256, 8, 2), (40, 256, 128, 4, 2)])
def test_moe_q8_0_decode_and_grouped(mx, T, H, EF, E, Kt):
    """Q8_0 SoA experts (include/ie/moe_q8.hpp): silu(gate)*up, route weight folded into down, plain-sum reduce."""
    ops = mx.ops
    Wg, gq, gd, qs_st, d_st = make_experts(O.Q8_0, 400, E, EF, H)
    Wu, uq, ud, _, _ = make_experts(O.Q8_0, 500, E, EF, H)
    Wd, dq, dd, dqs_st, dd_st = make_experts(O.Q8_0, 600, E, H, EF)
    x = f16(O.normal(7, (T, H)))
    ids, w = route(8, T, E, Kt)
    xq = O.quantize_q8_1(x)
    rb, hrb = H // 32 * 40, EF // 32 * 40
    idsd = dev(ids.ravel())
    h = ops.moe_gate_up_silu_q8(dev(xq), dev(gq), dev(gd), dev(uq), dev(ud), qs_st, d_st, idsd, T, Kt, H, EF)
    h_h = host(h).astype(np.float32)
    h_ref = np.stack([O.swiglu_np(O.gemv_q8chain(O.Q8_0, Wg[ids[t, k]], xq[t * rb:(t + 1) * rb], H, EF)[0].astype(np.float32),
                                  O.gemv_q8chain(O.Q8_0, Wu[ids[t, k]], xq[t * rb:(t + 1) * rb], H, EF)[0].astype(np.float32))
                      for t in range(T) for k in range(Kt)])
    check(h_h, h_ref, "moe_gate_up_silu_q8 T=%d" % T)
    hq = ops.quantize_q8_1(h)
    hq_h = host(hq)
    w16 = dev(w.ravel()).half()
    yp = ops.moe_down_q8(hq, dev(dq), dev(dd), dqs_st, dd_st, idsd, w16, T, Kt, EF, H)
    yp_ref = np.stack([f16(w.ravel()[s]) * O.gemv_q8chain(O.Q8_0, Wd[ids.ravel()[s]], hq_h[s * hrb:(s + 1) * hrb], EF, H)[0]
                       for s in range(T * Kt)])
    check(host(yp).astype(np.float32), yp_ref, "moe_down_q8")
    yp_f = ops.moe_down_q8_f16(h, dev(dq), dev(dd), dqs_st, dd_st, idsd, w16, T, Kt, EF, H)
    assert np.array_equal(host(yp_f), host(yp)), "down on fp16 h != quantize + down"
    y = ops.moe_reduce_q8(yp, T, Kt, H)
    check(host(y).astype(np.float32), host(yp).astype(np.float32).reshape(T, Kt, H).sum(axis=1), "moe_reduce_q8")
    # grouped form == decode form, row for row
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    TK = T * Kt
    xpq = ops.quantize_q8_1(ops.moe_gather_rows(dev(x).half(), dev(si), TK, H))
    hp = ops.moe_prefill_gate_up_silu_q8(xpq, dev(gq), dev(gd), dev(uq), dev(ud), qs_st, d_st, dev(off), TK, E, H, EF)
    check(host(hp).astype(np.float32)[t2p], h_ref, "moe_prefill_gate_up_silu_q8 (grouped) T=%d" % T)
    check_rows(host(hp)[t2p], host(h), "grouped gate_up vs decode rows")
    hpq = ops.quantize_q8_1(hp)
    hpq_h = host(hpq)
    op = ops.moe_prefill_down_q8(hpq, dev(dq), dev(dd), dqs_st, dd_st, dev(off), dev(wp).half(), TK, E, H, EF)
    row_expert = np.repeat(np.arange(E), np.diff(off.astype(np.int64)))
    op_ref = np.stack([f16(wp[r]) * O.gemv_q8chain(O.Q8_0, Wd[row_expert[r]], hpq_h[r * hrb:(r + 1) * hrb], EF, H)[0] for r in range(TK)])
    check(host(op).astype(np.float32), op_ref, "moe_prefill_down_q8 (grouped) T=%d" % T)
    check_rows(host(op)[t2p], host(yp), "grouped down vs decode rows")
    y2 = ops.moe_prefill_reduce_sum(op, dev(t2p.astype(np.uint32)), T, Kt, H)
    check_rows(host(y2), host(y), "grouped layer output == decode layer output")


def _mxfp4_bank(seed, E, N, K, e_choices):
    """Random E2M1 codes and per-block exponents drawn from `e_choices` -> (AoS blocks [E, N, K/32*17], qs plane, e plane)."""
    rng = np.random.default_rng(seed)
    W = rng.integers(0, 256, size=(E, N, K // 32, 17), dtype=np.uint8)
    W[..., 0] = rng.choice(np.asarray(e_choices, np.uint8), size=(E, N, K // 32))
    W = W.reshape(E, N, K // 32 * 17)
    qs, e = O.repack_mxfp4_to_soa(W)
    return W, qs, e


def _q8_rows(seed, rows, K, d, qmax):
    """Hand-built block_q8_1x rows: every block {d, d * sum(q), q[32]} with q uniform in [-qmax, qmax]."""
    rng = np.random.default_rng(seed)
    q = rng.integers(-qmax, qmax + 1, size=(rows, K // 32, 32)).astype(np.int8)
    buf = np.zeros((rows, K // 32, 40), np.uint8)
    buf[..., 0:4] = np.frombuffer(np.float32(d).tobytes(), np.uint8)
    buf[..., 4:8] = (np.float32(d) * q.sum(axis=2).astype(np.float32)).astype(np.float32).view(np.uint8).reshape(rows, K // 32, 4)
    buf[..., 8:] = q.view(np.uint8)
    return buf.reshape(-1), q.reshape(rows, K).astype(np.int64)


E2M1_X2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)   # doubled E2M1 values, include/ie/quant_blocks.hpp:46-60


def _mxfp4_codes_x2(W, N, K):
    """[E, N, K] doubled E2M1 values of a bank of 17-byte blocks (element j in the low, j + 16 in the high nibble of byte j)."""
    b = W.reshape(W.shape[0], N, K // 32, 17)[..., 1:]
    return np.concatenate([E2M1_X2[b & 15], E2M1_X2[b >> 4]], axis=-1).reshape(W.shape[0], N, K)


@pytest.mark.parametrize("counts", [(5, 20, 33), (1, 0, 16, 17)])
def test_moe_grouped_mxfp4_integer_part_exact(mx, counts):
    """Grouped MXFP4 down projection with every scale a power of two (e = 127: weights are the E2M1 values themselves;
    activation rows with d = 1 and small codes): the sum is an exact multiple of 1/2 well inside fp32's integer range,
    so whatever the summation order the fp32 result is the brute-force integer sum and the output is its one rounding
    to fp16, bit for bit.  Expert sizes cover one partial token pass, a full one, and one row beyond a full pass."""
    ops = mx.ops
    E, K, N = len(counts), 512, 96
    W, qs, e = _mxfp4_bank(31, E, N, K, [127])
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    TK = int(off[-1])
    xq, q = _q8_rows(32, TK, K, 1.0, 3)
    bias = np.zeros((E, N), np.float32)
    out = ops.moe_grouped_down_mxfp4(dev(xq), dev(qs), dev(e), N * K // 2, N * K // 32, dev(bias), dev(off), TK, E, N, K)
    codes = _mxfp4_codes_x2(W, N, K)
    row_expert = np.repeat(np.arange(E), counts)
    exact = np.stack([codes[row_expert[r]] @ q[r] for r in range(TK)]).astype(np.float64) / 2.0   # e8m0_half(127) = 1/2 of the doubled value
    assert np.abs(exact).max() < 2048
    assert np.array_equal(host(out), exact.astype(np.float16)), "grouped MXFP4 down: integer part not exact"
    # gate/up: with all-zero up codes u = 0 and z + 1 = 1, so h = half(glu(half(g))) is a function of the exact gate sum
    # alone (2 fp16 ulps for the device exponential); then the same with the roles swapped through a constant gate.
    EF = 64
    Wg, gq, ge = _mxfp4_bank(33, E, EF, K, [120])       # scale 2^-8 of the doubled value: |g| stays below the clamp at 7
    zero_q, zero_e = np.zeros_like(gq), np.full_like(ge, 120)
    bz = np.zeros((E, EF), np.float32)
    g_exact = np.stack([_mxfp4_codes_x2(Wg, EF, K)[row_expert[r]] @ q[r] for r in range(TK)]).astype(np.float64) / 256.0
    assert np.abs(g_exact).max() < 7.0
    g16 = g_exact.astype(np.float16).astype(np.float64)
    hp = ops.moe_grouped_gate_up_oai_mxfp4(dev(xq), dev(gq), dev(ge), dev(zero_q), dev(zero_e), EF * K // 2, EF * K // 32, dev(bz), dev(bz), dev(off), TK, E, K, EF)
    ref = g16 / (1.0 + np.exp(-1.702 * g16))
    assert np.all(np.abs(host(hp).astype(np.float64) - ref) <= 2.0 * ulp16(ref) + 2.0 ** -24), "gate sums through swiglu_oai"
    bg1 = np.ones((E, EF), np.float32)
    hp = ops.moe_grouped_gate_up_oai_mxfp4(dev(xq), dev(zero_q), dev(zero_e), dev(gq), dev(ge), EF * K // 2, EF * K // 32, dev(bg1), dev(bz), dev(off), TK, E, K, EF)
    ref = (1.0 / (1.0 + np.exp(-1.702))) * (g16 + 1.0)
    assert np.all(np.abs(host(hp).astype(np.float64) - ref) <= 2.0 * ulp16(ref) + 2.0 ** -24), "up sums through swiglu_oai"


def test_moe_grouped_mxfp4_exponent_range(mx):
    """Exponent bytes across the range real MXFP4 tensors use and well beyond (2^-100 .. 2^+60 of the doubled value), with
    activation scales that bring the products back into fp16 range: the grouped kernel hands the stored byte to the
    matrix instruction as its block scale, the oracle goes through e8m0_half (include/ie/quant_blocks.hpp:46-54)."""
    ops = mx.ops
    E, K, N, counts = 2, 512, 64, (9, 20)
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    TK = int(off[-1])
    bias = np.zeros((E, N), np.float32)
    row_expert = np.repeat(np.arange(E), counts)
    for e_lo, d in ((28, 2.0 ** 88), (100, 2.0 ** 16), (126, 2.0 ** -10), (186, 2.0 ** -70)):
        W, qs, e = _mxfp4_bank(40 + e_lo, E, N, K, [e_lo, e_lo + 1, e_lo + 2])
        xq, _ = _q8_rows(41, TK, K, d, 127)
        out = ops.moe_grouped_down_mxfp4(dev(xq), dev(qs), dev(e), N * K // 2, N * K // 32, dev(bias), dev(off), TK, E, N, K)
        ref = np.stack([O.gemv_q8chain(O.MXFP4, W[row_expert[r]], xq[r * (K // 32 * 40):(r + 1) * (K // 32 * 40)], K, N)[0] for r in range(TK)])
        check(host(out).astype(np.float32), ref, "grouped MXFP4 down, exponents %d..%d" % (e_lo, e_lo + 2))


def test_moe_q8_decode_skips_ids_outside_the_bank(mx):
    """The *_n decode entry points: slots whose expert id is negative or not below n_experts are skipped (their output
    rows keep their contents), every other slot equals the plain entry point's row."""
    ops = mx.ops
    T, Kt, E, H, EF = 3, 4, 4, 512, 256
    Wg, gq, gd, qs_st, d_st = make_experts(O.Q8_0, 900, E, EF, H)
    Wu, uq, ud, _, _ = make_experts(O.Q8_0, 910, E, EF, H)
    Wd, dq, dd, dqs_st, dd_st = make_experts(O.Q8_0, 920, E, H, EF)
    x = f16(O.normal(11, (T, H)))
    ids = np.array([[0, 1, 2, 3], [3, E, 1, -1], [2, 7, 1 << 20, 0]], np.int32)
    good = ((ids >= 0) & (ids < E)).ravel()
    safe = np.where(good.reshape(ids.shape), ids, 0).astype(np.int32)
    w16 = dev(f16(np.full(ids.size, 0.25, np.float32))).half()
    xq = dev(O.quantize_q8_1(x))
    args = (xq, dev(gq), dev(gd), dev(uq), dev(ud), qs_st, d_st)
    h_ref = ops.moe_gate_up_silu_q8(*args, dev(safe.ravel()), T, Kt, H, EF)
    h = torch.full((T * Kt, EF), 7.0, dtype=torch.float16, device="cuda")
    ops.moe_gate_up_silu_q8(*args, dev(ids.ravel()), T, Kt, H, EF, h_out=h, n_experts=E)
    assert np.array_equal(host(h)[good], host(h_ref)[good]) and np.all(host(h)[~good] == 7.0)
    hq = ops.quantize_q8_1(h_ref)
    dargs = (dev(dq), dev(dd), dqs_st, dd_st)
    y_ref = ops.moe_down_q8(hq, *dargs, dev(safe.ravel()), w16, T, Kt, EF, H)
    for fn, act in ((ops.moe_down_q8, hq), (ops.moe_down_q8_f16, h_ref)):
        y = torch.full((T * Kt, H), 7.0, dtype=torch.float16, device="cuda")
        fn(act, *dargs, dev(ids.ravel()), w16, T, Kt, EF, H, y_packed=y, n_experts=E)
        assert np.array_equal(host(y)[good], host(y_ref)[good]) and np.all(host(y)[~good] == 7.0)


def test_moe_grouped_skips_empty_and_single_row_experts(mx):
    """Experts with 0 rows write nothing; 1-row experts are exact (the reference notes
    wrong rows for tiny per-expert batches on its dense-GEMM route, gptoss_tp.cpp:702-765)."""
    ops = mx.ops
    E, H, EF = 6, 256, 128
    Wg, gq, gd, qs_st, d_st = make_experts(O.Q8_0, 700, E, EF, H)
    Wu, uq, ud, _, _ = make_experts(O.Q8_0, 800, E, EF, H)
    ids = np.array([[1], [1], [4], [1], [5], [1], [1], [1], [1], [1], [1]], np.int32)   # expert 1: 9 rows (two tiles), 4 and 5: one row
    w = np.ones(ids.shape, np.float32)
    x = f16(O.normal(9, (ids.shape[0], H)))
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    assert off.tolist() == [0, 0, 9, 9, 9, 10, 11]
    xpq = ops.quantize_q8_1(ops.moe_gather_rows(dev(x).half(), dev(si), 11, H))
    hp = torch.full((11, EF), 7.0, dtype=torch.float16, device="cuda")
    ops.moe_prefill_gate_up_silu_q8(xpq, dev(gq), dev(gd), dev(uq), dev(ud), qs_st, d_st, dev(off), 11, E, H, EF, h_packed=hp)
    xq_h = host(xpq)
    rb = H // 32 * 40
    ref = np.stack([O.swiglu_np(O.gemv_q8chain(O.Q8_0, Wg[ids[si[r], 0]], xq_h[r * rb:(r + 1) * rb], H, EF)[0].astype(np.float32),
                                O.gemv_q8chain(O.Q8_0, Wu[ids[si[r], 0]], xq_h[r * rb:(r + 1) * rb], H, EF)[0].astype(np.float32))
                    for r in range(11)])
    check(host(hp).astype(np.float32), ref, "grouped with empty experts")


@pytest.mark.parametrize("T,E,Kt,H,EF", [(1, 16, 8, 2048, 512), (3, 8, 4, 512, 768), (1, 4, 2, 256, 256)])
def test_moe_decode_kquant_fp16_activations(mx, T, E, Kt, H, EF):
    """moe_decode_gate_up_silu_q4k / moe_decode_down_q4k / _q6k (include/ie/ops.hpp:1034-1095): fp16
    activations, AoS expert banks, device-resident expert ids; against the float-activation oracle,
    expert by expert (the per-token per-expert loop of tests/unit/moe_test.cpp:62-169)."""
    ops = mx.ops
    mk = lambda F, seed, N, K: np.stack([O.quantize(F, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
    Wg, Wu = mk(O.Q4_K, 8100, EF, H), mk(O.Q4_K, 8200, EF, H)
    x = f16(O.normal(8300, (T, H)))
    ids, w = route(8400, T, E, Kt)
    w16 = f16(w)
    idd = dev(ids.astype(np.int32).reshape(-1))
    h = ops.moe_decode_gate_up_silu_q4k(dev(x).half(), dev(Wg), dev(Wu), idd, H, EF, Kt, Wg[0].size, T)
    # per-expert SoA regions (include/ie/quant_soa.hpp:33-51): same bits, same arithmetic, same result
    soa = lambda fmt, W: dev(ops.repack_moe_kquant_soa(fmt, W, E, W[0].size // O.BLOCK_BYTES[O.Q4_K if fmt == "q4k" else O.Q6_K]))
    h_soa = ops.moe_decode_gate_up_silu_q4k(dev(x).half(), soa("q4k", Wg), soa("q4k", Wu), idd, H, EF, Kt, Wg[0].size, T, soa=True)
    assert torch.equal(h, h_soa)
    h_h = host(h).astype(np.float32)
    h_ref = np.zeros((T * Kt, EF), np.float32)
    for t in range(T):
        for k in range(Kt):
            e = int(ids[t, k])
            g = O.gemv_f64(O.Q4_K, Wg[e], x[t:t + 1], H, EF)[0]
            u = O.gemv_f64(O.Q4_K, Wu[e], x[t:t + 1], H, EF)[0]
            h_ref[t * Kt + k] = O.swiglu_np(g.astype(np.float32), u.astype(np.float32))
    check(h_h, h_ref, "moe decode gate_up silu q4k")
    for fmt, F in (("q4k", O.Q4_K), ("q6k", O.Q6_K)):
        Wd = mk(F, 8500, H, EF)
        y = ops.moe_decode_down_kquant(fmt, h, dev(Wd), idd, dev(w16.reshape(-1)).half(), H, EF, Kt, Wd[0].size, T)
        assert torch.equal(y, ops.moe_decode_down_kquant(fmt, h, soa(fmt, Wd), idd, dev(w16.reshape(-1)).half(), H, EF, Kt, Wd[0].size, T, soa=True))
        y_ref = np.zeros((T, H), np.float64)
        for t in range(T):
            for k in range(Kt):
                e = int(ids[t, k])
                y_ref[t] += float(w16[t, k]) * O.gemv_f64(F, Wd[e], h_h[t * Kt + k:t * Kt + k + 1], EF, H)[0]
        check(host(y).astype(np.float32), y_ref, "moe decode down %s" % fmt)


@pytest.mark.parametrize("T,E,Kt,H,EF", [(40, 8, 2, 512, 256), (200, 32, 4, 256, 768)])
def test_moe_grouped_kquant_int_dot(mx, T, E, Kt, H, EF):
    """moe_prefill_gate_up_silu_q4k_q8 / _q6k_q8 and moe_prefill_down_packed_q4k_q8 / _q6k_q8, all on block_q8_1s rows
    (the layout the reference kernels read, src/ops/moe_fused.cpp:559-566,672-687), against the q8_1s-chain oracle
    (min terms on the stored half sums), expert by expert."""
    ops = mx.ops
    mk = lambda F, seed, N, K: np.stack([O.quantize(F, O.normal(seed + e, (N, K), 0.0, 0.02)) for e in range(E)])
    x = f16(O.normal(8600, (T, H)))
    ids, w = route(8601, T, E, Kt)
    off, si, wp, t2p = ops.build_moe_packing(ids, w, E)
    TK = T * Kt
    counts = np.diff(off.astype(np.int64))
    xp = ops.moe_gather_rows(dev(x).half(), dev(si), TK, H)
    xq = ops.quantize_q8_1s(xp)
    xq_h = host(xq).reshape(TK, -1)
    assert np.array_equal(xq_h.ravel(), O.quantize_q8_1s(host(xp).astype(np.float32)))
    h_keep = None
    for fmt, F in (("q4k", O.Q4_K), ("q6k", O.Q6_K)):
        Wg, Wu = mk(F, 8700, EF, H), mk(F, 8800, EF, H)
        hp = ops.moe_prefill_gate_up_silu_kquant_q8(fmt, xq, dev(Wg), dev(Wu), dev(off), TK, E, H, EF, Wg[0].size)
        soa = lambda W: dev(ops.repack_moe_kquant_soa(fmt, W, E, W[0].size // O.BLOCK_BYTES[F]))
        assert torch.equal(hp, ops.moe_prefill_gate_up_silu_kquant_q8(fmt, xq, soa(Wg), soa(Wu), dev(off), TK, E, H, EF, Wg[0].size, soa=True))
        h_ref = np.zeros((TK, EF), np.float32)
        for e in range(E):
            if counts[e]:
                rows = slice(off[e], off[e + 1])
                g = O.gemv_q8schain(F, Wg[e], xq_h[rows], H, EF)
                u = O.gemv_q8schain(F, Wu[e], xq_h[rows], H, EF)
                h_ref[rows] = O.swiglu_np(g.astype(np.float32), u.astype(np.float32))
        check(host(hp).astype(np.float32), h_ref, "grouped gate_up silu %s int-dot (q8_1s rows)" % fmt)
        h_keep = hp
    hq = ops.quantize_q8_1s(h_keep)
    hq_h = host(hq).reshape(TK, -1)
    for fmt, F in (("q4k", O.Q4_K), ("q6k", O.Q6_K)):
        Wd = mk(F, 8900, H, EF)
        op = ops.moe_prefill_down_packed_kquant_q8(fmt, hq, dev(Wd), dev(off), TK, E, H, EF, Wd[0].size)
        Wd_soa = dev(ops.repack_moe_kquant_soa(fmt, Wd, E, Wd[0].size // O.BLOCK_BYTES[F]))
        assert torch.equal(op, ops.moe_prefill_down_packed_kquant_q8(fmt, hq, Wd_soa, dev(off), TK, E, H, EF, Wd[0].size, soa=True))
        o_ref = np.zeros((TK, H), np.float64)
        for e in range(E):
            if counts[e]:
                rows = slice(off[e], off[e + 1])
                o_ref[rows] = O.gemv_q8schain(F, Wd[e], hq_h[rows], EF, H)
        check(host(op).astype(np.float32), o_ref, "grouped down packed %s int-dot (q8_1s rows)" % fmt)


@pytest.mark.parametrize("n_tok,hidden", [(7, 2048), (5, 100), (1, 8)])
def test_moe_scatter_add_bit_exact(mx, n_tok, hidden):
    """moe_scatter_add (src/ops/moe.cpp:284-313): y[idx[i]] = half(float(y[idx[i]]) + float(x[i]) * w[i]).
    fp16 x fp16 products are exact in fp32, so the result is fixed bit for bit."""
    T = n_tok + 3
    xp = O.round_fp16(O.normal(1300 + hidden, (n_tok, hidden), 0.0, 1.0))
    y0 = O.round_fp16(O.normal(1301 + hidden, (T, hidden), 0.0, 1.0))
    w = O.round_fp16(np.abs(O.normal(1302, (n_tok,), 0.0, 0.5)))
    idx = np.random.default_rng(1303).permutation(T)[:n_tok].astype(np.int32)
    y = mx.ops.moe_scatter_add(dev(xp).half(), dev(idx), dev(w).half(), dev(y0).half(), n_tok, hidden)
    ref = y0.copy()
    ref[idx] = (y0[idx].astype(np.float32) + xp.astype(np.float32) * w[:, None].astype(np.float32)).astype(np.float16).astype(np.float32)
    assert np.array_equal(host(y).astype(np.float32), ref)
