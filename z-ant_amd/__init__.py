"""MI355X (gfx950) backend for Z-Ant's tensor-math hot path.

The product is the C-ABI shared library ``libzant_hip.so`` (sources in ``csrc/``, header in
``include/zant_hip.h``).  This Python package is a thin host-side mirror of the reference's operator
interface (``conv_lean``, ``gemm_lean``, ``mat_mul_lean``, ``onnx_maxpool_lean``, ``ReLU_lean`` ... as
re-exported by the reference's tensor_math_standard.zig:43-149) over that library, with torch used only
for device memory and streams.  There is no CPU fallback: importing fails if the library is not built.
"""
from .capi import Context, ZantError, lib, lib_path, status_name  # noqa: F401
from . import tensor_math  # noqa: F401
from . import model  # noqa: F401
from . import onnx_front  # noqa: F401
