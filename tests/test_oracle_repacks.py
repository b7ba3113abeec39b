"""K-quant repacks (CPU): the oracle's numpy restatements against the reference's own host repackers
where oracle/_ref is built, against the layouts the reference documents (one-hot probes with the
expected byte and bit written out), and against the identity that a repack never changes a weight's
value; then the library's host repackers against the oracle, byte for byte."""
import numpy as np
import pytest

import oracle as O
from machx_inference_engine_amd import ops


def blocks(fmt, seed, N, K):
    return O.quantize(fmt, O.normal(seed, (N, K), 0.0, 0.05))


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K))
def test_stream_repack_matches_reference_host_code(fmt):
    ref = O.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built")
    E, nb = 3, 24
    bank = O.rand_bytes(900 + fmt, E * nb * O.BLOCK_BYTES[fmt])
    want = np.empty_like(bank)
    (ref.ref_repack_moe_q4k_soa if fmt == O.Q4_K else ref.ref_repack_moe_q6k_soa)(bank.ctypes.data, want.ctypes.data, E, nb)
    assert np.array_equal(O.repack_kquant_streams(fmt, bank, E, nb), want)


@pytest.mark.parametrize("fmt", (O.Q4_K, O.Q6_K))
def test_stream_repack_matches_reference_golden(fmt):
    """The same check against vectors written from the reference's host code (tests/golden/make_golden.py),
    for where oracle/_ref is not built."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"))
    name = O.FMT_NAMES[fmt]
    assert np.array_equal(O.repack_kquant_streams(fmt, g["soa_in_" + name], 3, 20), g["soa_out_" + name])
    assert np.array_equal(ops.repack_moe_kquant_soa("q4k" if fmt == O.Q4_K else "q6k", g["soa_in_" + name], 3, 20), g["soa_out_" + name])


def test_stream_layout_probe():
    """One region of two Q4_K blocks: qs x 2 | scales x 2 | {d,dmin} x 2 (include/ie/quant_soa.hpp:33-41)."""
    bank = np.arange(288, dtype=np.uint16).astype(np.uint8)   # byte i = i mod 256
    out = O.repack_kquant_streams(O.Q4_K, bank, 1, 2)
    assert out[0] == 16 and out[127] == 143                    # block 0 qs
    assert out[128] == (144 + 16) % 256                        # block 1 qs
    assert out[256] == 4 and out[256 + 12] == (144 + 4) % 256  # scales of block 0, block 1
    assert out[280] == 0 and out[284] == 144                   # {d,dmin} of block 0, block 1


def test_q4_K_codes_scale_unpack_matches_get_scale_min_k4():
    W = blocks(O.Q4_K, 910, 4, 512)
    _, sc, mn, _, _ = O.q4_K_codes(W)
    b = W.reshape(-1, 144)
    for i in range(b.shape[0]):
        for j in range(8):
            assert (sc[i, j], mn[i, j]) == O.get_scale_min_k4(j, b[i, 4:16])


def test_natural_order_probes():
    """Element k of a row: Q4 nibble (k&1) of byte k/2; Q6 low nibble likewise, high bits = bits 2(k&3) of
    byte k/4 (src/ops/gemv_q4_soa.cpp:21-23, src/ops/gemv_q6_soa.cpp:97-110)."""
    # Q4_K block, only element 37 = 64*0 + 32*1 + 5 non-zero (high nibble of qs[5])
    b = np.zeros(144, np.uint8)
    b[16 + 5] = 0xB0
    q = O.repack_q4_K_to_soa(b)[0]
    assert q[18] == 0xB0 and q.sum() == 0xB0                  # byte 37//2, high nibble (37 odd)
    # Q6_K block, only element 198 = 128*1 + 32*2 + 6: low nibble = high half of ql[64 + 6], high bits qh[32 + 6] >> 4
    b = np.zeros(210, np.uint8)
    b[64 + 6] = 0x90
    b[128 + 32 + 6] = 0x20
    lo, hi, _, _ = O.repack_q6_K_to_soa(b)
    assert lo[99] == 0x09 and lo.sum() == 0x09                # byte 198//2, low nibble (198 even)
    assert hi[49] == 0x20 and hi.sum() == 0x20                # byte 198//4, bits 2*(198&3) = 4..5, value 2


# the shapes of the reference's own host-side check of this repack (tools/q4_soa_test.cpp:75-77) plus two more
@pytest.mark.parametrize("K,N", [(256, 1), (256, 5), (512, 3), (2048, 7), (768, 4), (256, 64), (1024, 7)])
def test_natural_order_repack_keeps_every_value(K, N):
    W4, W6 = blocks(O.Q4_K, 920, N, K), blocks(O.Q6_K, 921, N, K)
    assert np.array_equal(O.dequant_q4_soa(O.repack_q4_K_to_soa(W4)).view(np.uint32), O.dequant(O.Q4_K, W4).view(np.uint32))
    assert np.array_equal(O.dequant_q6_soa(O.repack_q6_K_to_soa(W6)).view(np.uint32), O.dequant(O.Q6_K, W6).view(np.uint32))


def test_library_host_repackers_match_oracle():
    K, N = 512, 5
    W4, W6 = blocks(O.Q4_K, 930, N, K), blocks(O.Q6_K, 931, N, K)
    nb = N * K // 256
    assert np.array_equal(ops.repack_q4_K_to_reorder(W4, K, N), O.repack_kquant_streams(O.Q4_K, W4, 1, nb))
    assert np.array_equal(ops.repack_moe_kquant_soa("q4k", W4, 5, nb // 5), O.repack_kquant_streams(O.Q4_K, W4, 5, nb // 5))
    assert np.array_equal(ops.repack_moe_kquant_soa("q6k", W6, 2, nb // 2), O.repack_kquant_streams(O.Q6_K, W6, 2, nb // 2))
    for got, want in zip(ops.repack_q4_K_to_soa(W4, K, N), O.repack_q4_K_to_soa(W4)):
        assert np.array_equal(got, want)
    for got, want in zip(ops.repack_q6_K_to_soa(W6, K, N), O.repack_q6_K_to_soa(W6)):
        assert np.array_equal(got, want)
