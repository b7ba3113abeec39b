"""The C-ABI library: loads without a GPU, exports every symbol include/mxq.h
declares, and rejects bad arguments before any HIP call."""
import ctypes as C
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from machx_inference_engine_amd import _lib
    return _lib.load(), _lib.parse_header()


def test_every_declared_symbol_is_exported(lib):
    l, protos = lib
    assert len(protos) >= 40
    raw = C.CDLL(os.path.join(ROOT, "machx_inference_engine_amd", "libmxq.so"))
    for name in protos:
        assert hasattr(raw, name), name


def test_status_strings_and_version(lib):
    l, _ = lib
    assert l.mx_version() >= 100
    assert l.mx_status_string(0) == b"ok"
    assert len({l.mx_status_string(i) for i in range(6)}) == 6


def test_argument_validation_without_gpu(lib):
    l, protos = lib
    OK, NULL, SHAPE, ALIGN = 0, 1, 2, 3
    p16, p8, p2 = 0x1000, 0x1008, 0x1002
    # NULL pointers
    assert l.mx_gemv_q4_K_q8(None, None, p16, p16, 4096, 4096) == NULL
    assert l.mx_gemv_q4_K_q8(None, p16, None, p16, 4096, 4096) == NULL
    assert l.mx_quantize_q8_1(None, None, p16, 64) == NULL
    assert l.mx_dequant_q6_K(None, p16, None, 256) == NULL
    # shape preconditions: K % 256 for K-quants, K % 32 for Q8_0 / MXFP4, T in 1..16, n % 32
    assert l.mx_gemv_q4_K_q8(None, p16, p16, p16, 4096 + 32, 16) == SHAPE
    assert l.mx_gemv_q6_K_q8(None, p16, p16, p16, 100, 16) == SHAPE
    assert l.mx_gemv_q8_0_q8(None, p16, p16, p16, 48, 16) == SHAPE
    assert l.mx_gemv_mxfp4_soa_q8(None, p16, p16, p16, p16, 2880 + 16, 16) == SHAPE
    assert l.mx_gemv_q4_K_q8(None, p16, p16, p16, 4096, 0) == SHAPE
    assert l.mx_gemv_q4_K_q8_batched(None, p16, p16, p16, 4096, 16, 0) == SHAPE
    assert l.mx_gemv_q4_K_q8_batched(None, p16, p16, p16, 4096, 16, 17) == SHAPE
    assert l.mx_quantize_q8_1(None, p16, p16, 33) == SHAPE
    assert l.mx_dequant_q4_K(None, p16, p16, 255) == SHAPE
    assert l.mx_dequant_q8_0_to_Bt(None, p16, p16, 48, 4) == SHAPE
    # alignment: Q4_K weights 16 B, q8 stream 8 B, SoA quant plane 16 B
    assert l.mx_gemv_q4_K_q8(None, p16, p8, p16, 4096, 16) == ALIGN
    assert l.mx_gemv_q4_K_q8(None, 0x1004, p16, p16, 4096, 16) == ALIGN
    assert l.mx_gemv_q8_0_soa_q8(None, p16, p8, p16, p16, 4096, 16) == ALIGN
    assert l.mx_gemv_q6_K_q8(None, p16, 0x1001, p16, 4096, 16) == ALIGN
    # host repackers work without a GPU
    import numpy as np
    blk = np.arange(17 * 3, dtype=np.uint8)
    qs, e = np.zeros(48, np.uint8), np.zeros(3, np.uint8)
    assert l.mx_repack_mxfp4_to_soa(blk.ctypes.data, 3, qs.ctypes.data, e.ctypes.data) == OK
    assert e.tolist() == [0, 17, 34] and qs[:16].tolist() == list(range(1, 17))
    assert l.mx_repack_mxfp4_to_soa(None, 3, qs.ctypes.data, e.ctypes.data) == NULL


def test_workspace_forms_validate_before_any_hip_call(lib):
    """The *_ws entry points: size query, NULL / misaligned / too-small workspace."""
    l, _ = lib
    OK, NULL, SHAPE, ALIGN, WORKSPACE = 0, 1, 2, 3, 9
    p16 = 0x1000
    n = C.c_uint64(7)
    # without a GPU the library assumes 256 CUs: 128 blocks of 32 rows want 4 K ranges of T x N partial sums
    assert l.mx_gemv_batched_ws_bytes(14336, 4096, 8, C.addressof(n)) == OK and n.value == 4 * 8 * 4096 * 4
    assert l.mx_gemv_batched_ws_bytes(4096, 151936, 8, C.addressof(n)) == OK and n.value == 0                   # enough row blocks: K is never split
    assert l.mx_gemv_batched_ws_bytes(14336, 4096, 1, C.addressof(n)) == OK and n.value == 0
    assert l.mx_gemv_batched_ws_bytes(14336, 4096, 8, None) == NULL
    assert l.mx_gemv_batched_ws_bytes(14336, 4096, 17, C.addressof(n)) == SHAPE
    need = 4 * 8 * 4096 * 4
    assert l.mx_gemv_q8_0_soa_q8_batched_ws(None, p16, p16, p16, p16, 14336, 4096, 8, None, need) == NULL
    assert l.mx_gemv_q8_0_soa_q8_batched_ws(None, p16, p16, p16, p16, 14336, 4096, 8, 0x1004, need) == ALIGN
    assert l.mx_gemv_q8_0_soa_q8_batched_ws(None, p16, p16, p16, p16, 14336, 4096, 8, p16, need - 4) == WORKSPACE
    assert l.mx_gemv_q6_K_q8_batched_ws(None, p16, p16, p16, 14336, 4096, 8, p16, 16) == WORKSPACE
    assert l.mx_status_string(WORKSPACE).startswith(b"workspace")
    assert l.mx_gemm_ws_bytes(128, 14336, 4096, None) == NULL
    assert l.mx_gemm_q4_K_ws(None, p16, p16, p16, 128, 14336, 4096, None, 64) == NULL
    assert l.mx_gemm_q4_K_ws(None, p16, p16, p16, 128, 14336, 4096, 0x1004, 64) == ALIGN


def test_query_sized_workspace_is_never_refused(lib):
    """mx_gemv_batched_ws_bytes carries no weight format, while the launch picks its kernel (and with it the number of K
    slices) by format: whatever the format, batch and shape, a workspace of the size the query names must not come back
    as MX_ERR_WORKSPACE.  Without a GPU the call gets past the workspace check and fails at the launch instead."""
    l, _ = lib
    WORKSPACE = 9
    p16 = 0x1000
    n = C.c_uint64(0)
    shapes = [(14336, 4096), (14336, 1000), (8192, 14336), (8192, 512), (4096, 14336), (4096, 4096), (12288, 256), (16384, 151936)]
    for K, N in shapes:
        for T in range(2, 17):
            assert l.mx_gemv_batched_ws_bytes(K, N, T, C.addressof(n)) == 0
            ws = p16 if n.value else None
            for rc in (l.mx_gemv_q8_0_soa_q8_batched_ws(None, p16, p16, p16, p16, K, N, T, ws, n.value),
                       l.mx_gemv_q4_K_q8_batched_ws(None, p16, p16, p16, K, N, T, ws, n.value),
                       l.mx_gemv_q6_K_q8_batched_ws(None, p16, p16, p16, K, N, T, ws, n.value),
                       l.mx_gemv_q8_0_q8_batched_ws(None, p16, p16, p16, K, N, T, ws, n.value)):
                assert rc != WORKSPACE, (K, N, T, n.value)
