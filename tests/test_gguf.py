"""GGUF reader (host, no GPU): files written here from the container layout, read back through
mx_gguf_* (GgufReader, include/ie/gguf.hpp:72-117): metadata of every value type, tensor directory,
alignment, zero-copy tensor bytes, split shards, and the error paths."""
import os
import struct

import numpy as np
import pytest

import gguf_util as G
import oracle as O
from machx_inference_engine_amd import gguf, lib


def sample_tensors():
    K, N = 512, 3
    return [
        ("tok.weight", 12, (K, N), O.quantize(O.Q4_K, O.normal(10, (N, K), 0.0, 0.02))),
        ("out.weight", 14, (K, N), O.quantize(O.Q6_K, O.normal(11, (N, K), 0.0, 0.02))),
        ("attn.weight", 8, (K, N), O.quantize(O.Q8_0, O.normal(12, (N, K), 0.0, 0.02))),
        ("exp.weight", 39, (64, 2, 4), O.quantize(O.MXFP4, O.normal(13, (8, 64), 0.0, 0.02))),
        ("norm.weight", 0, (7,), np.arange(7, dtype=np.float32)),
    ]


def test_roundtrip_metadata_and_tensors(tmp_path):
    kvs = [("general.architecture", G.STR, "qwen3"), ("general.alignment", G.U32, 64), ("a.u8", G.U8, 200), ("a.i8", G.I8, -5),
           ("a.u16", G.U16, 65000), ("a.i16", G.I16, -300), ("a.i32", G.I32, -70000), ("a.f32", G.F32, 1.5), ("a.bool", G.BOOL, True),
           ("a.u64", G.U64, 2 ** 40), ("a.i64", G.I64, -2 ** 40), ("a.f64", G.F64, 0.1),
           ("tokens", G.ARR, (G.STR, ["<s>", "hello", ""])), ("ids", G.ARR, (G.I32, [3, -1, 7])), ("empty", G.ARR, (G.F32, []))]
    tensors = sample_tensors()
    path = tmp_path / "m.gguf"
    offs = G.write_gguf(path, kvs, tensors, alignment=64)
    with gguf.GgufFile(path) as f:
        assert (f.version, f.alignment) == (3, 64) and f.tensor_data_offset % 64 == 0
        assert f.kv["general.architecture"] == "qwen3" and f.kv["a.u8"] == 200 and f.kv["a.i8"] == -5 and f.kv["a.u16"] == 65000
        assert f.kv["a.i16"] == -300 and f.kv["a.i32"] == -70000 and f.kv["a.f32"] == 1.5 and f.kv["a.bool"] is True
        assert f.kv["a.u64"] == 2 ** 40 and f.kv["a.i64"] == -2 ** 40 and f.kv["a.f64"] == 0.1
        assert f.kv["tokens"] == ["<s>", "hello", ""] and f.kv["ids"] == [3, -1, 7] and f.kv["empty"] == []
        assert list(f.tensors) == [t[0] for t in tensors]                      # file order kept
        for i, (name, gtype, shape, data) in enumerate(tensors):
            info = f.tensors[name]
            raw = np.ascontiguousarray(data).view(np.uint8).ravel()
            assert (info.ggml_type, info.shape, info.nbytes, info.offset_in_data) == (gtype, shape, raw.size, offs[name])
            assert np.array_equal(f.tensor_bytes(name), raw)
            assert f.find_tensor(name) == i
        assert f.tensors["exp.weight"].type_name == "mxfp4" and f.tensors["exp.weight"].nbytes == 8 * 2 * 17
        with pytest.raises(gguf.GgufError) as e:
            f.find_tensor("missing")
        assert e.value.status == 8
        # the file's bytes at data offset + tensor offset are the tensor (the view is into the mapping, not a copy)
        blob = open(path, "rb").read()
        o = f.tensor_data_offset + offs["out.weight"]
        assert blob[o:o + 16] == bytes(f.tensor_bytes("out.weight")[:16])


def test_default_alignment_and_v2(tmp_path):
    path = tmp_path / "v2.gguf"
    G.write_gguf(path, [("k", G.U32, 1)], sample_tensors()[:1], alignment=32, version=2)
    with gguf.GgufFile(path) as f:
        assert (f.version, f.alignment) == (2, 32) and f.tensor_data_offset % 32 == 0
        assert f.tensors["tok.weight"].type_name == "q4_K"


def test_split_shards(tmp_path):
    t = sample_tensors()
    p1, p2 = tmp_path / "m-00001-of-00002.gguf", tmp_path / "m-00002-of-00002.gguf"
    G.write_gguf(p1, [("general.architecture", G.STR, "x"), ("split.count", G.U16, 2), ("split.tensors.count", G.I32, 5)], t[:2])
    G.write_gguf(p2, [("split.no", G.U16, 1), ("split.count", G.U16, 2)], t[2:])      # as gguf-split writes them
    with gguf.GgufFile(p1) as f:
        assert list(f.tensors) == [x[0] for x in t] and "split.no" not in f.kv     # metadata from the first shard only
        for name, _, _, data in t:
            assert np.array_equal(f.tensor_bytes(name), np.ascontiguousarray(data).view(np.uint8).ravel())
    with pytest.raises(gguf.GgufError) as e:
        gguf.GgufFile(p2)                                                          # a later shard is not an entry point
    os.remove(p2)
    with pytest.raises(gguf.GgufError) as e:
        gguf.GgufFile(p1)
    assert e.value.status == 6 and "00002-of-00002" in str(e.value)


def test_errors(tmp_path):
    with pytest.raises(gguf.GgufError) as e:
        gguf.GgufFile(tmp_path / "absent.gguf")
    assert e.value.status == 6
    good = tmp_path / "g.gguf"
    G.write_gguf(good, [("k", G.STR, "v" * 50)], sample_tensors())
    blob = open(good, "rb").read()
    cases = {"magic": b"GGUX" + blob[4:], "version": blob[:4] + struct.pack("<I", 9) + blob[8:], "short": blob[:20],
             "truncated metadata": blob[:60], "tensor outside file": blob[:-400]}
    for what, data in cases.items():
        p = tmp_path / "bad.gguf"
        p.write_bytes(data)
        with pytest.raises(gguf.GgufError) as e:
            gguf.GgufFile(p)
        assert e.value.status == 7, what
    # a directory entry whose element count would overflow the size computation
    p = tmp_path / "huge.gguf"
    G.write_gguf(p, [], [("t", 0, (2 ** 62, 8), np.zeros(4, np.float32))])
    with pytest.raises(gguf.GgufError) as e:
        gguf.GgufFile(p)
    assert e.value.status == 7
    assert lib.mx_gguf_open(None, None) == 1
