"""ctypes loader for ``benchlib/libtccl_probe.so``, the benchmark's measuring kernels
(``python -m tccl_amd.build`` compiles it from ``benchlib/probe.hip``)."""
from __future__ import annotations

import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtccl_probe.so")

_P, _SZ, _I = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
_PP = ctypes.POINTER(ctypes.c_void_p)

SIGNATURES = {
    "tccl_probe_read": (_I, [_PP, _I, _SZ, _P, _P]),
    "tccl_probe_write": (_I, [_P, _SZ, _P]),
    "tccl_probe_write_small": (_I, [_P, _SZ, _P]),
    "tccl_probe_write_dense": (_I, [_P, _SZ, _P]),
    "tccl_probe_read_dense": (_I, [_P, _SZ, _P, _P]),
    "tccl_probe_copy": (_I, [_P, _P, _SZ, _P]),
    "tccl_probe_sum_timed": (_I, [_PP, _P, _SZ, _P, _P]),
    "tccl_probe_empty": (_I, [_P]),
    "tccl_probe_stamp": (_I, [_P, _P]),
    "tccl_probe_empty_grid": (_I, [_I, _P]),
    "tccl_probe_touch": (_I, [_P, _P, _I, _P]),
    "tccl_probe_placement": (_I, [_P, _I, _I, _P]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -m tccl_amd.build`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib
