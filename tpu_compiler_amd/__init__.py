"""tpu_compiler_amd: MI355X (gfx950) implementation of the tpuc-interpreter INT8
inference path.  The compute lives in libtpuhip.so (hand-written HIP kernels
behind a C ABI, with the reference's op-level C++ classes on top); this package
is the ctypes binding, the pymlir-shaped `module`, and the seeded synthetic
graphs of the benchmark configurations."""
from . import _lib, capi  # noqa: F401
from .pymodule import module  # noqa: F401
