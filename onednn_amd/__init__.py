"""MI355X-native quantized matmul behind oneDNN's matmul interface.

Layers:
  onednn_amd/csrc   hand-written gfx950 HIP kernels + the thin C ABI
                    (include/mi355_matmul.h) -> onednn_amd/lib/libmi355_matmul.so
  onednn_amd/host   host C++: the dnnl_* C API subset over that ABI
                    (include/dnnl_amd.h) -> onednn_amd/lib/libdnnl_amd.so
  onednn_amd/cabi.py, onednn_amd/dnnl.py   ctypes mirrors used by tests and bench
"""
from . import cabi  # noqa: F401
