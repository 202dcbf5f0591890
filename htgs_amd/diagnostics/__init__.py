"""Measurement aids of the benchmark, outside the rasterizer library: ``counters.py`` turns rocprofv3 counter runs into
the HBM-traffic record ``bench.py`` reports, and ``libhtgs_copy.so`` (``copy_kernel.hip``) is the plain copy of known
size that calibrates those counters (``bench.py --calibrate``)."""
from __future__ import annotations

import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libhtgs_copy.so")

SYMBOLS = {
    "htgs_diag_copy_bytes": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing; build it with `python -m htgs_amd.build`")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = handle
    return _lib
