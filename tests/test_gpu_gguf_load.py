"""GPU: weights read from a GGUF file through the library's reader go straight into the kernels —
the AoS blocks as they lie in the file, and the repacked forms via the load-time repackers."""
import numpy as np
import pytest
import torch

import gguf_util as G
import oracle as O
from gpu_util import check, dev, host

pytestmark = pytest.mark.gpu


def test_gemv_from_gguf_file(mx, tmp_path):
    from machx_inference_engine_amd import gguf
    K, N = 1024, 96
    W4 = O.quantize(O.Q4_K, O.normal(5000, (N, K), 0.0, 0.02))
    W6 = O.quantize(O.Q6_K, O.normal(5001, (N, K), 0.0, 0.02))
    W8 = O.quantize(O.Q8_0, O.normal(5002, (N, K), 0.0, 0.02))
    Wm = O.quantize(O.MXFP4, O.normal(5003, (N, K), 0.0, 0.02))
    path = tmp_path / "w.gguf"
    G.write_gguf(path, [("general.architecture", G.STR, "test")],
                 [("a", 12, (K, N), W4), ("b", 14, (K, N), W6), ("c", 8, (K, N), W8), ("d", 39, (K, N), Wm)])
    xq = O.quantize_q8_1(O.round_fp16(O.normal(5004, (1, K))))
    xd = dev(xq)
    ops = mx.ops
    with gguf.GgufFile(path) as f:
        y4 = ops.gemv_q4_K_q8(xd, f.load("a"), K, N)
        check(host(y4).astype(np.float32), O.gemv_q8chain(O.Q4_K, W4, xq, K, N)[0], "q4_K from file (AoS)")
        assert torch.equal(ops.gemv_q4_K_reorder_q8(xd, f.load("a", "reorder"), K, N), y4)
        assert torch.equal(ops.gemv_q4_soa_q8(xd, f.load("a", "soa"), K, N), y4)
        y6 = ops.gemv_q6_K_q8(xd, f.load("b"), K, N)
        check(host(y6).astype(np.float32), O.gemv_q8chain(O.Q6_K, W6, xq, K, N)[0], "q6_K from file (AoS)")
        check(host(ops.gemv_q6_soa_q8(xd, f.load("b", "soa"), K, N)).astype(np.float32), O.gemv_q8chain(O.Q6_K, W6, xq, K, N)[0], "q6_K from file (planes)")
        y8 = ops.gemv_q8_0_q8(xd, f.load("c"), K, N)
        qs, d = f.load("c", "soa")
        assert torch.equal(ops.gemv_q8_0_soa_q8(xd, qs, d, K, N), y8)
        qs, e = f.load("d", "soa")
        check(host(ops.gemv_mxfp4_soa_q8(xd, qs, e, K, N)).astype(np.float32), O.gemv_q8chain(O.MXFP4, Wm, xq, K, N)[0], "mxfp4 from file (planes)")
