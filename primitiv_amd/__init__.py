"""MI355X (gfx950) backend for primitiv's matmul path.

`libphip.so` (C ABI, include/phip.h) holds all GPU code; `device` is the thin
Python mirror of primitiv's Device front used by the tests and the benchmark.
"""
from ._lib import Error, lib  # noqa: F401
from .device import HIP, HIP16, DeviceType, Shape, Tensor, shape_ops  # noqa: F401
