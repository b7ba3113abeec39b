"""GPU parity: block dequant (bit-exact vs the oracle, fp32 and fp16 outputs,
flat and transposed) and the q8_1 / q8_1s activation quantizers (bit-exact)."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import dev, host

pytestmark = pytest.mark.gpu
FMTS = (O.Q8_0, O.Q4_K, O.Q6_K, O.MXFP4, O.Q4_0)


def random_blocks(fmt, seed, nb):
    """1024 seeded random blocks per format as the reference's dequant test does
    (tests/unit/dequant_test.cpp:112-150); scale fields kept finite."""
    raw = O.rand_bytes(seed, nb * O.BLOCK_BYTES[fmt]).reshape(nb, -1).copy()
    for off in {O.Q8_0: [1], O.Q4_K: [1, 3], O.Q6_K: [209], O.MXFP4: [], O.Q4_0: [1]}[fmt]:
        raw[:, off] &= 0xBB
    if fmt == O.MXFP4:  # the reference test's exponent list, then random ones below overflow
        lst = [0, 1, 2, 3, 64, 126, 127, 128, 200, 254, 255]
        raw[:len(lst), 0] = lst
    return raw


@pytest.mark.parametrize("fmt", FMTS)
def test_dequant_bit_exact(mx, fmt):
    name = O.FMT_NAMES[fmt]
    raw = random_blocks(fmt, 0xC0FFEE + fmt, 1024)
    enc = O.quantize(fmt, O.normal(3 + fmt, (8, 2048), 0.0, 0.02)).reshape(-1, O.BLOCK_BYTES[fmt])
    blocks = np.concatenate([raw, enc, np.zeros((1, O.BLOCK_BYTES[fmt]), np.uint8)])
    n = blocks.shape[0] * O.BLOCK_ELEMS[fmt]
    ref = O.dequant(fmt, blocks)
    got32 = host(mx.ops.dequant(name, dev(blocks), n, dtype=torch.float32))
    assert np.array_equal(got32.view(np.uint32), ref.view(np.uint32)), "%s fp32 dequant not bit-exact" % name
    got16 = host(mx.ops.dequant(name, dev(blocks), n)).view(np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(got16, O.fp32_to_fp16(ref)), "%s fp16 dequant not bit-exact" % name


@pytest.mark.parametrize("fmt", FMTS)
def test_dequant_to_Bt_is_transpose(mx, fmt):
    """Bt[k*N+n] == flat[n*K+k] (tests/unit/dequant_bt_test.cpp:44-72)."""
    name, K, N = O.FMT_NAMES[fmt], 512, 200
    W = O.quantize(fmt, O.normal(20260611 + fmt, (N, K), 0.0, 0.02))
    flat = host(mx.ops.dequant(name, dev(W), N * K)).view(np.uint16).reshape(N, K)
    bt = host(mx.ops.dequant_to_Bt(name, dev(W), K, N)).view(np.uint16)
    assert np.array_equal(bt, flat.T)
    assert np.array_equal(bt, O.dequant_to_Bt(fmt, W, K, N))


def test_dequant_q5_K_bit_exact_and_Bt(mx):
    """Q5_K (dequant only: src/ops/dequant_kernels.cpp:149-210,567-609).  Blocks: random bytes with
    finite scales, and Q4_K-encoded rows given a random fifth-bit plane (realistic scale fields)."""
    K, N = 512, 40
    raw = O.rand_bytes(0xC0FFEE + 5, 600 * 176).reshape(600, 176).copy()
    raw[:, 1] &= 0xBB
    raw[:, 3] &= 0xBB
    q4 = O.quantize(O.Q4_K, O.normal(55, (N, K), 0.0, 0.02)).reshape(-1, 144)
    q5 = np.zeros((q4.shape[0], 176), np.uint8)
    q5[:, :16] = q4[:, :16]
    q5[:, 16:48] = O.rand_bytes(56, q4.shape[0] * 32).reshape(-1, 32)
    q5[:, 48:] = q4[:, 16:]
    blocks = np.concatenate([raw, q5, np.zeros((1, 176), np.uint8)])
    n = blocks.shape[0] * 256
    ref = O.dequant(O.Q5_K, blocks)
    got32 = host(mx.ops.dequant("q5_K", dev(blocks), n, dtype=torch.float32))
    assert np.array_equal(got32.view(np.uint32), ref.view(np.uint32))
    with np.errstate(over="ignore"):
        assert np.array_equal(host(mx.ops.dequant("q5_K", dev(blocks), n)).view(np.uint16), O.fp32_to_fp16(ref))
    W = q5.reshape(N, -1)
    bt = host(mx.ops.dequant_to_Bt("q5_K", dev(W), K, N)).view(np.uint16)
    assert np.array_equal(bt, O.fp32_to_fp16(O.dequant(O.Q5_K, W)).reshape(N, K).T)
    assert np.array_equal(bt, O.dequant_to_Bt(O.Q5_K, W, K, N))


@pytest.mark.parametrize("dtype", (torch.float16, torch.float32))
def test_quantize_q8_1_bit_exact(mx, dtype):
    x = O.normal(0x0801, 32 * 1000, 0.0, 1.0)
    x[64:96] = 0.0
    x[96:128] = 1e-30      # tiny amax
    x[128] = 127.0
    x[129], x[130] = 2.5, -2.5   # ties, inv = 1
    if dtype == torch.float16:
        x = O.round_fp16(x)
    xt = dev(x).to(dtype)
    got = host(mx.ops.quantize_q8_1(xt))
    assert np.array_equal(got, O.quantize_q8_1(x))
    got_s = host(mx.ops.quantize_q8_1s(xt))
    assert np.array_equal(got_s, O.quantize_q8_1s(x))


def test_quantize_rejects_ragged(mx):
    with pytest.raises(mx.MxError):
        mx.ops.quantize_q8_1(torch.zeros(48, dtype=torch.float16, device="cuda"))
