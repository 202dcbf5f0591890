"""ctypes binding of the measurement probes (``include/htgs_probes.h``, ``libhtgs_probes.so``): a plain copy kernel
that calibrates the HBM traffic counters and micro-kernels that time single vector instructions.  Only the benchmark
uses them; the rasterizer library does not contain them."""
from __future__ import annotations

import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libhtgs_probes.so")

SYMBOLS = {
    "htgs_probe_issue_cost_name": (ctypes.c_char_p, [ctypes.c_int]),
    "htgs_probe_issue_cost_launch": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "htgs_probe_copy_bytes": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
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
