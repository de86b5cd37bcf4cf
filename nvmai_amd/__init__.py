"""MI355X-native quantized mixture-of-experts hot path (gfx950 HIP kernels behind a C ABI).

The package holds the C ABI library (csrc/, include/nvmai_hip.h) and a thin host
layer over it.  PyTorch is used for device memory and streams only.
"""
from ._lib import LIB_PATH, NvmaiError, lib  # noqa: F401
from .ops import *  # noqa: F401,F403
