"""MI355X-native quantized-weight matmul path (GGUF Q4_K / Q6_K / Q8_0 / MXFP4).

`ops` mirrors the reference's `src/ops` free functions on torch device tensors;
every call goes through the C ABI of libmxq.so (include/mxq.h).  PyTorch is
used only for device memory and the current HIP stream.
"""
import torch  # noqa: F401  -- before libmxq.so: the library must bind to the HIP runtime torch has loaded,
#                      or the process ends up with two runtimes and the second one sees no device

from . import _lib

lib = _lib.load()

from . import ops  # noqa: E402
from . import gguf  # noqa: E402,F401
from .ops import MxError  # noqa: E402,F401
