"""deep8_amd -- MI355X (gfx950) kernels for Deep8's MatrixMultiply / Conv2d / DeConv2d GPU path.

csrc/   hand-written HIP kernels and the C ABI (include/deep8_hip.h) -> libdeep8_hip.so
host/   C++ mirror of Deep8's Tensor / Shape / Device / Function API on top of that C ABI
capi    ctypes binding of the C ABI;  ops: numpy-level drivers used by tests and the benchmark
"""
from . import capi  # noqa: F401
