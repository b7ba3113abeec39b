"""Synthetic, valid GGUF-block weights generated directly in HBM (torch RNG).

Used by bench.py and smoke runs where only the shape and validity of the blocks
matter: every field is filled with seeded random codes and scale fields in the
range real tensors use, so the kernels do the same work as on N(0, 0.02) weights
and produce finite outputs.  (Parity tests use the oracle's ggml-faithful
encoders instead; this module never touches the oracle.)
"""
import torch

BLOCK = {"q8_0": (32, 34), "q4_K": (256, 144), "q6_K": (256, 210), "mxfp4": (32, 17)}


def row_bytes(fmt, K):
    e, b = BLOCK[fmt]
    return K // e * b


def _f16_bytes(vals):
    """fp32 tensor [...] -> uint8 [..., 2] holding the fp16 bit pattern (little endian)."""
    return vals.to(torch.float16).contiguous().view(torch.uint8).reshape(*vals.shape, 2)


def random_weights(fmt, N, K, seed, device="cuda:0"):
    """uint8 [N, row_bytes(fmt, K)] of valid blocks; block scales mimic N(0, 0.02) weights."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    e, b = BLOCK[fmt]
    nb = K // e
    blk = torch.randint(0, 256, (N, nb, b), dtype=torch.uint8, device=device, generator=g)
    u = torch.rand((N, nb), device=device, generator=g)
    if fmt == "q8_0":
        blk[:, :, 0:2] = _f16_bytes((0.045 + 0.02 * u) / 127.0)
    elif fmt == "q4_K":
        blk[:, :, 0:2] = _f16_bytes((0.07 + 0.03 * u) / 63.0 / 15.0 * 2.0)
        blk[:, :, 2:4] = _f16_bytes((0.045 + 0.02 * u) / 63.0)
    elif fmt == "q6_K":
        blk[:, :, 208:210] = _f16_bytes((0.05 + 0.02 * u) / 31.0 / 100.0)
    else:  # mxfp4: exponent near 2^-7 so that 6 * 2^(e-127) ~ 0.05
        blk[:, :, 0] = (119 + (u * 3).to(torch.uint8)).to(torch.uint8)
    return blk.reshape(N, nb * b)


def split_mxfp4(blocks):
    """[N, nb*17] AoS -> (qs_plane [N*nb*16], e_plane [N*nb]) as the SoA kernels take them."""
    b = blocks.reshape(-1, 17)
    return b[:, 1:].contiguous().reshape(-1), b[:, 0].contiguous()


def split_q8_0(blocks):
    """[N, nb*34] AoS -> (qs_plane int8 [N*K], d_plane uint16-as-int16 [N*K/32])."""
    b = blocks.reshape(-1, 34)
    return b[:, 2:].contiguous().reshape(-1).view(torch.int8), b[:, 0:2].contiguous().reshape(-1).view(torch.int16)


# ---------------------------------------------------------------- encoders: seeded N(0, std) -> GGUF blocks, in torch
# Plain min/max encoders (not ggml's iterative search): they write valid blocks whose codes, sub-block scales and
# super-block scales have the statistics of quantized N(0, 0.02) tensors, which is what a throughput measurement needs
# (the matrix-core rate on this part depends on the operand bits).  Layouts: include/ie/quant_blocks.hpp:26-98,
# element order include/ie/dequant_ref.hpp:20-96.  They run on any torch device, rows in slabs to bound memory.
def _le16(h):
    """fp16 tensor [...] -> uint8 [..., 2]"""
    return h.contiguous().view(torch.uint8).reshape(*h.shape, 2)


def _enc_q8_0(x):
    b = x.reshape(x.shape[0], -1, 32)
    amax = b.abs().amax(dim=2)
    d = (amax / 127.0).to(torch.float16)
    inv = torch.where(amax > 0, 127.0 / amax, torch.zeros_like(amax))
    q = torch.round(b * inv[..., None]).clamp_(-127, 127).to(torch.int8)
    return torch.cat([_le16(d), q.view(torch.uint8)], dim=2)


def _enc_q4_K(x):
    R = x.shape[0]
    b = x.reshape(R, -1, 8, 32)                                   # [R, nb, sub-block, 32]
    lo = b.amin(dim=3).clamp_(max=0.0)
    hi = b.amax(dim=3)
    scale, mn = (hi - lo) / 15.0, -lo                             # value = scale * q - mn, q in 0..15
    d = (scale.amax(dim=2) / 63.0).to(torch.float16)
    dmin = (mn.amax(dim=2) / 63.0).to(torch.float16)
    df, dmf = d.float()[..., None], dmin.float()[..., None]
    sc = torch.where(df > 0, torch.round(scale / df), torch.zeros_like(scale)).clamp_(0, 63)
    m = torch.where(dmf > 0, torch.round(mn / dmf), torch.zeros_like(mn)).clamp_(0, 63)
    d1 = (df * sc)[..., None]
    q = torch.where(d1 > 0, torch.round((b + (dmf * m)[..., None]) / d1), torch.zeros_like(b)).clamp_(0, 15).to(torch.uint8)
    sc, m = sc.to(torch.uint8), m.to(torch.uint8)
    s12 = torch.cat([sc[..., :4] | ((sc[..., 4:] >> 4) << 6), m[..., :4] | ((m[..., 4:] >> 4) << 6), (sc[..., 4:] & 15) | ((m[..., 4:] & 15) << 4)], dim=2)
    q = q.reshape(R, -1, 4, 2, 32)                                # [.., group of 64, low / high nibble, l]
    qs = (q[:, :, :, 0] | (q[:, :, :, 1] << 4)).reshape(R, -1, 128)
    return torch.cat([_le16(d), _le16(dmin), s12, qs], dim=2)


def _enc_q6_K(x):
    R = x.shape[0]
    b = x.reshape(R, -1, 16, 16)                                  # [R, nb, 16-element group, 16]
    amax = b.abs().amax(dim=3)
    scale = amax / 31.0
    d = (scale.amax(dim=2) / 127.0).to(torch.float16)
    df = d.float()[..., None]
    sc = torch.where(df > 0, torch.round(scale / df), torch.zeros_like(scale)).clamp_(0, 127)
    c = (df * sc)[..., None]
    q = (torch.where(c > 0, torch.round(b / c), torch.zeros_like(b)).clamp_(-32, 31) + 32).to(torch.uint8)
    q = q.reshape(R, -1, 2, 4, 32)                                # element 128 h + 32 s + l
    lo4, hi2 = q & 15, q >> 4
    ql = torch.stack([lo4[:, :, :, 0] | (lo4[:, :, :, 2] << 4), lo4[:, :, :, 1] | (lo4[:, :, :, 3] << 4)], dim=3).reshape(R, -1, 128)
    qh = (hi2[:, :, :, 0] | (hi2[:, :, :, 1] << 2) | (hi2[:, :, :, 2] << 4) | (hi2[:, :, :, 3] << 6)).reshape(R, -1, 64)
    return torch.cat([ql, qh, sc.to(torch.int8).view(torch.uint8), _le16(d)], dim=2)


def _enc_mxfp4(x):
    b = x.reshape(x.shape[0], -1, 32)
    amax = b.abs().amax(dim=2)
    # value = 2^(e-128) * {0,1,2,3,4,6,8,12}: the smallest e whose largest magnitude 12 * 2^(e-128) covers amax
    e = torch.ceil(torch.log2(amax.clamp_min(1e-30) / 12.0)).clamp_(-126, 120) + 128.0
    unit = torch.exp2(e - 128.0)[..., None]
    lut = torch.tensor([0., 1., 2., 3., 4., 6., 8., 12.], device=x.device)
    code = (b.abs() / unit)[..., None].sub(lut).abs_().argmin(dim=3).to(torch.uint8) | ((b < 0).to(torch.uint8) << 3)
    qs = code[:, :, :16] | (code[:, :, 16:] << 4)
    return torch.cat([e.to(torch.uint8)[..., None], qs], dim=2)


_ENCODERS = {"q8_0": _enc_q8_0, "q4_K": _enc_q4_K, "q6_K": _enc_q6_K, "mxfp4": _enc_mxfp4}


def encode(fmt, x):
    """fp32 [N, K] -> uint8 [N, row_bytes(fmt, K)] of GGUF blocks."""
    return _ENCODERS[fmt](x.float()).reshape(x.shape[0], -1)


def normal_weights(fmt, N, K, seed, std=0.02, device="cuda:0", slab_elems=1 << 25):
    """Seeded N(0, std) fp32 weights [N, K] quantized to `fmt`, generated and encoded slab by slab on `device`."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = torch.empty((N, row_bytes(fmt, K)), dtype=torch.uint8, device=device)
    step = max(1, slab_elems // K)
    for r0 in range(0, N, step):
        n = min(step, N - r0)
        out[r0:r0 + n] = encode(fmt, torch.randn((n, K), device=device, generator=g) * std)
    return out
