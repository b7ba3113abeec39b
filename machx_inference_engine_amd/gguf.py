"""Host-side view of a GGUF file through the library's memory-mapped reader (mx_gguf_*), plus the
load-time step from a tensor in the file to the device tensors a kernel takes.

Mirrors the reference's GgufReader (include/ie/gguf.hpp:72-117): `tensors` / `kv` directories,
`find`-style lookups, zero-copy views of the tensor bytes.  The weight layouts on disk are the GGUF
block layouts, which the AoS kernels read as they are; `load()` optionally runs one of the library's
host repackers on the way to the device.
"""
import ctypes as C
import struct

import numpy as np

from . import lib

GGML_TYPE_NAMES = {0: "f32", 1: "f16", 2: "q4_0", 8: "q8_0", 12: "q4_K", 13: "q5_K", 14: "q6_K", 30: "bf16", 39: "mxfp4"}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}


class _Tensor(C.Structure):
    _fields_ = [("name", C.c_void_p), ("name_len", C.c_uint64), ("ggml_type", C.c_uint32), ("n_dims", C.c_uint32),
                ("shape", C.c_uint64 * 4), ("offset_in_data", C.c_uint64), ("nbytes", C.c_uint64), ("data", C.c_void_p)]


class _Kv(C.Structure):
    _fields_ = [("key", C.c_void_p), ("key_len", C.c_uint64), ("type", C.c_uint32), ("inner_type", C.c_uint32),
                ("n_array", C.c_uint64), ("payload", C.c_void_p)]


class GgufError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        detail = lib.mx_gguf_last_error().decode() if status in (6, 7) else ""
        super().__init__("%s: %s%s" % (fn, lib.mx_status_string(status).decode(), (": " + detail) if detail else ""))


class TensorInfo:
    def __init__(self, t):
        self.name = C.string_at(t.name, t.name_len).decode()
        self.ggml_type = t.ggml_type
        self.type_name = GGML_TYPE_NAMES.get(t.ggml_type, "ggml_%d" % t.ggml_type)
        self.shape = tuple(t.shape[i] for i in range(t.n_dims))     # shape[0] = contiguous (K) dimension
        self.offset_in_data = t.offset_in_data
        self.nbytes = t.nbytes
        self._data = t.data

    def __repr__(self):
        return "TensorInfo(%r, %s, shape=%s, nbytes=%d)" % (self.name, self.type_name, self.shape, self.nbytes)


def _read_value(vtype, addr):
    """-> (python value, bytes consumed) for a scalar or string at addr."""
    if vtype == 8:
        n = struct.unpack("<Q", C.string_at(addr, 8))[0]
        return C.string_at(addr + 8, n).decode("utf-8", "replace"), 8 + n
    fmt = _SCALAR[vtype]
    sz = struct.calcsize(fmt)
    return struct.unpack(fmt, C.string_at(addr, sz))[0], sz


class GgufFile:
    def __init__(self, path):
        h = C.c_void_p()
        rc = lib.mx_gguf_open(str(path).encode(), C.byref(h))
        if rc:
            raise GgufError("mx_gguf_open", rc)
        self._h = h
        ver, nt, nkv, al, off = C.c_uint32(), C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        lib.mx_gguf_info(h, C.byref(ver), C.byref(nt), C.byref(nkv), C.byref(al), C.byref(off))
        self.version, self.alignment, self.tensor_data_offset = ver.value, al.value, off.value
        self.tensors, self.kv = {}, {}
        for i in range(nt.value):
            t = _Tensor()
            lib.mx_gguf_tensor(h, i, C.byref(t))
            info = TensorInfo(t)
            self.tensors[info.name] = info
        for i in range(nkv.value):
            k = _Kv()
            lib.mx_gguf_kv(h, i, C.byref(k))
            key = C.string_at(k.key, k.key_len).decode()
            if k.type == 9:
                vals, addr = [], k.payload
                for _ in range(k.n_array):
                    v, used = _read_value(k.inner_type, addr)
                    vals.append(v)
                    addr += used
                self.kv[key] = vals
            else:
                self.kv[key] = _read_value(k.type, k.payload)[0]

    def close(self):
        if self._h:
            lib.mx_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def find_tensor(self, name):
        """Index of the tensor in file order; raises GgufError (MX_ERR_NOT_FOUND) if absent."""
        idx = C.c_uint64()
        rc = lib.mx_gguf_find_tensor(self._h, name.encode(), C.byref(idx))
        if rc:
            raise GgufError("mx_gguf_find_tensor(%s)" % name, rc)
        return idx.value

    def tensor_bytes(self, name):
        """Zero-copy uint8 view of the tensor's bytes in the mapping (valid until close())."""
        info = self.tensors[name]
        if info.nbytes == 0:
            raise ValueError("%s: type %s is not sized by the reader" % (name, info.type_name))
        return np.ctypeslib.as_array(C.cast(info._data, C.POINTER(C.c_uint8)), shape=(info.nbytes,))

    def load(self, name, layout="aos", device="cuda"):
        """Tensor `name` (rows of K = shape[0] elements, N = product of the other dims) -> device tensors.
        layout 'aos': the GGUF blocks as one uint8 tensor [N, row_bytes]; 'soa': the planes of the format's
        SoA kernels (q8_0: qs, d; mxfp4: qs, e; q4_K: q, sc, mn, d, dmin; q6_K: lo, hi, sc, d);
        'reorder' (q4_K): the three-stream form of gemv_q4_K_reorder_q8."""
        import torch

        from . import ops
        info = self.tensors[name]
        K = info.shape[0]
        N = int(np.prod(info.shape[1:], dtype=np.int64)) if len(info.shape) > 1 else 1
        raw = self.tensor_bytes(name)
        to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
        if layout == "aos":
            return to_dev(raw.reshape(N, -1))
        t = info.type_name
        if layout == "reorder" and t == "q4_K":
            return to_dev(ops.repack_q4_K_to_reorder(raw, K, N))
        if layout == "soa":
            if t == "q4_K":
                return tuple(to_dev(p) for p in ops.repack_q4_K_to_soa(raw, K, N))
            if t == "q6_K":
                return tuple(to_dev(p) for p in ops.repack_q6_K_to_soa(raw, K, N))
            if t in ("q8_0", "mxfp4"):
                return tuple(to_dev(p) for p in ops.repack_block32_to_soa(t, raw))
        raise ValueError("layout %r is not defined for type %s" % (layout, t))
