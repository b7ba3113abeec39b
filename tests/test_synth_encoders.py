"""The torch encoders that write the benchmark's and the full-size tests' weights (seeded N(0, 0.02) -> GGUF blocks,
machx_inference_engine_amd/synth.py): every block they write must decode, through the oracle's dequant, to within the
format's quantization step of the fp32 value it encodes."""
import numpy as np
import pytest
import torch

import oracle as O
from machx_inference_engine_amd import synth

CASES = [("q8_0", O.Q8_0, 32, 0.5 / 127 + 2.0 ** -11), ("q4_K", O.Q4_K, 32, 0.09), ("q6_K", O.Q6_K, 16, 0.02), ("mxfp4", O.MXFP4, 32, 0.26)]


@pytest.mark.parametrize("name,fmt,grp,bound", CASES)
def test_encoder_round_trip(name, fmt, grp, bound):
    N, K = 48, 1024
    W = synth.normal_weights(name, N, K, seed=3, device="cpu")
    assert W.dtype == torch.uint8 and tuple(W.shape) == (N, synth.row_bytes(name, K)) == (N, O.row_bytes(fmt, K))
    g = torch.Generator(device="cpu")
    g.manual_seed(3)
    x = (torch.randn((N, K), generator=g) * 0.02).numpy()
    y = O.dequant(fmt, W.numpy().ravel()).reshape(N, K)
    amax = np.abs(x).reshape(N, -1, grp).max(axis=2, keepdims=True)
    assert (np.abs(x - y).reshape(N, -1, grp) / amax).max() <= bound
    # about the error of the oracle's (ggml-faithful) encoder on the same values
    yo = O.dequant(fmt, O.quantize(fmt, x).ravel()).reshape(N, K)
    assert np.sqrt(((x - y) ** 2).mean()) <= 1.15 * np.sqrt(((x - yo) ** 2).mean())


def test_q8_0_encoder_is_the_reference_recipe():
    """d = fp16(amax / 127), q = round(x * 127 / amax) (tools/q8_0_repack_bench.cpp:62-74): same bytes as the oracle's encoder."""
    x = O.normal(77, (8, 512), 0, 0.02)
    assert np.array_equal(synth.encode("q8_0", torch.from_numpy(x)).numpy(), O.quantize(O.Q8_0, x))


def test_zero_rows_encode_to_zero():
    for name, fmt, _, _ in CASES:
        W = synth.encode(name, torch.zeros((2, 256)))
        assert np.array_equal(O.dequant(fmt, W.numpy().ravel()), np.zeros(512, np.float32)), name
