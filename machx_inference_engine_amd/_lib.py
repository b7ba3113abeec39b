"""ctypes binding of libmxq.so.  Prototypes are read from include/mxq.h so the
binding cannot drift from the C ABI.  There is no fallback: if the library is
missing, importing this module raises."""
import ctypes as C
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(_HERE, "..", "include", "mxq.h")
LIB_PATH = os.path.join(_HERE, "libmxq.so")

_CTYPES = {"uint32_t": C.c_uint32, "uint64_t": C.c_uint64, "int": C.c_int, "float": C.c_float,
           "mx_stream_t": C.c_void_p, "size_t": C.c_size_t, "int32_t": C.c_int32}


def parse_header(path=HEADER):
    """-> {name: (restype, [(argname, ctype)])} for every function declared in the header."""
    src = open(path).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    src = re.sub(r"//[^\n]*", "", src)
    protos = {}
    for m in re.finditer(r"\b(int|const char\*)\s+(mx_\w+)\s*\(([^)]*)\)\s*;", src):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        argl = []
        if args and args != "void":
            for a in args.split(","):
                a = " ".join(a.split())
                if "*" in a:
                    argl.append((a.split("*")[-1].strip(), C.c_void_p))
                else:
                    ty, an = a.rsplit(" ", 1)
                    argl.append((an, _CTYPES[ty.replace("const ", "")]))
        protos[name] = (C.c_char_p if "char" in ret else C.c_int, argl)
    return protos


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError("libmxq.so is not built (%s): run `python machx_inference_engine_amd/build.py`; "
                          "there is no CPU fallback for this path" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in parse_header().items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = [t for _, t in args]
    return lib
