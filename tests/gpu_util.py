"""Helpers shared by the GPU parity tests: seeded inputs from the oracle's RNG,
torch<->numpy transfers, and the parity gate."""
import numpy as np
import torch

import oracle as O

DEV = "cuda:0"
GATE_MAX_REL = 1e-3     # BASELINE gate: max relative error (see oracle.parity for the floor)
GATE_COS = 0.99999


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def f16_bits_to_f32(t):
    return host(t).view(np.float16).astype(np.float32) if t.dtype != torch.float16 else host(t).astype(np.float32)


def weights(fmt, seed, N, K, std=0.02):
    """Seeded N(0, std) fp32 -> packed GGUF blocks, uint8 [N, row_bytes]."""
    return O.quantize(fmt, O.normal(seed, (N, K), 0.0, std))


def check(got, ref, what, max_rel=GATE_MAX_REL, cos=GATE_COS, abs_floor=2.0 ** -14):
    """abs_floor: 2^-14 for fp16 outputs (default; subnormal halfs carry absolute precision), 0 for fp32 outputs."""
    p = O.parity(got, ref, abs_floor)
    msg = "%s: max_rel=%.3e cos=%.7f max_abs/rms=%.3e (%d of %d under the 1%%-rms floor, %d under the 2^-14 floor)" % (
        what, p["max_rel"], p["cos"], p["max_abs_over_rms"], p["n_under_rms_floor"], p["n"], p["n_under_abs_floor"])
    print(msg, flush=True)
    assert np.isfinite(np.asarray(got, np.float64)).all(), what + ": non-finite output"
    assert p["max_rel"] <= max_rel and p["cos"] >= cos, msg
    return p
