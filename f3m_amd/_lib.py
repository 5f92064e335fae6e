"""Loads the gfx950 engine library.  There is no fallback: without the built library (and a GPU to
run it on) every operator of this package raises."""
import ctypes
import os

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libf3m.so")
_lib = None


def get():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("f3m_amd: %s is missing; build it with `python -m f3m_amd.build` "
                               "(hipcc, --offload-arch=gfx950)" % LIB_PATH)
        _lib = capi.bind(ctypes.CDLL(LIB_PATH))
    return _lib
