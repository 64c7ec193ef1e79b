"""Loads libtpuhip.so.  There is no fallback: without the built HIP library the
package cannot compute anything and says so."""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libtpuhip.so")
_lib = None


class TpuHipUnavailable(RuntimeError):
    pass


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TpuHipUnavailable(
                "%s is missing: build it with `python -m tpu_compiler_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib
