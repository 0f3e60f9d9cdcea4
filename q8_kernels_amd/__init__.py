"""q8_kernels_amd: the 8-bit inference hot path of q8_kernels on MI355X (gfx950).

`functional` and `modules` keep the reference's Python surface (names, argument order, defaults,
return shapes); everything below them is libq8_hip.so, reached through its C ABI with ctypes.
"""
from . import functional  # noqa: F401
from . import modules  # noqa: F401
from ._lib import Q8Error, device_info  # noqa: F401

__all__ = ["functional", "modules", "Q8Error", "device_info"]
