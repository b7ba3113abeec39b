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
