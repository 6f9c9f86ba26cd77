"""MI355X-native implementation of SharpNet's Tensor.Dot / BatchMatrixMultiplication path.

The product is ``libsharpnet_hip.so`` (C ABI in ``include/sharpnet_hip.h``); this
package holds its sources (``csrc/``), the build step, and a ctypes host that
mirrors the reference's ``GPUWrapper`` / ``GPUTensor<float>`` for that path.
"""
from .hiplib import CublasStatus, SharpNetHipError, load_library, library_path  # noqa: F401
from .gpu_tensor import GPUWrapper, GPUTensor  # noqa: F401
from . import linear, attention, recurrent  # noqa: F401

