"""ctypes loader for ``libtccl_amd.so``.

There is no fallback: if the library has not been built, or a call returns an error code,
an exception is raised.  Nothing here computes anything on the host.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtccl_amd.so")

ABI_VERSION = 2
TCCL_OK, TCCL_EINVAL, TCCL_EALIGN, TCCL_EPOW2, TCCL_ESCRATCH, TCCL_ETIMEOUT = 0, -1, -2, -3, -4, -5
MAX_WORLD = 8
MAX_JOBS = 8
IPC_HANDLE_BYTES = 64

TCCL_BF16 = 0
TCCL_F32 = 1

CFG_NONTEMPORAL_LOAD = 1
CFG_NONTEMPORAL_STORE = 2
CFG_XCD_CONTIGUOUS = 4
CFG_TEMPORAL = 8
CFG_STREAMING = 16
CFG_PHASED = 32

PIPE_DRAW_PLACES = 1
PIPE_OWN_BARRIERS = 2


class TcclError(RuntimeError):
    """A C entry point returned a negative code."""

    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed with code {code}: {text}")
        self.code = code


class LaunchCfg(ctypes.Structure):
    """Mirror of ``tccl_launch_cfg``; any field left 0 is chosen by the library."""
    _fields_ = [("block", ctypes.c_int), ("unroll", ctypes.c_int), ("grid", ctypes.c_int),
                ("tile_iters", ctypes.c_int), ("flags", ctypes.c_int)]


class PipelineCfg(ctypes.Structure):
    """Mirror of ``tccl_pipeline_cfg``; any field left 0 is chosen by the library."""
    _fields_ = [("workgroups", ctypes.c_int), ("lag", ctypes.c_int), ("spin_limit", ctypes.c_uint),
                ("tile_kib", ctypes.c_int), ("timeout_flag", ctypes.POINTER(ctypes.c_uint32)),
                ("flags", ctypes.c_int), ("pad_", ctypes.c_int)]


class NodeJob(ctypes.Structure):
    """Mirror of ``tccl_node_job``."""
    _fields_ = [("src", ctypes.c_void_p * 3), ("dst", ctypes.c_void_p * 2), ("numel", ctypes.c_size_t),
                ("is_copy", ctypes.c_int), ("pad_", ctypes.c_int)]


_P = ctypes.c_void_p
_PP = ctypes.POINTER(ctypes.c_void_p)
_SZ = ctypes.c_size_t
_I = ctypes.c_int
_CFG = ctypes.POINTER(LaunchCfg)

# name -> (restype, argtypes); exactly the symbols include/tccl_amd.h declares.
SIGNATURES = {
    "tccl_abi_version": (_I, []),
    "tccl_error_string": (ctypes.c_char_p, [_I]),
    "tccl_all_reduce_sum": (_I, [_PP, _I, _P, _SZ, _I, _P]),
    "tccl_all_reduce_sum_ex": (_I, [_PP, _I, _P, _SZ, _I, _P, _CFG]),
    "tccl_reduce_scatter_sum": (_I, [_PP, _I, _I, _P, _SZ, _I, _P]),
    "tccl_reduce_scatter_sum_ex": (_I, [_PP, _I, _I, _P, _SZ, _I, _P, _CFG]),
    "tccl_all_gather": (_I, [_PP, _I, _P, _SZ, _P]),
    "tccl_all_gather_ex": (_I, [_PP, _I, _P, _SZ, _P, _CFG]),
    "tccl_tree_reduce_step": (_I, [_P, _P, _P, _P, _SZ, _I, _P]),
    "tccl_tree_copy_step": (_I, [_P, _P, _P, _SZ, _P]),
    "tccl_tree_level": (_I, [ctypes.POINTER(NodeJob), _I, _I, _SZ, _P]),
    "tccl_double_tree_arrays": (_I, [_I, ctypes.POINTER(_I), ctypes.POINTER(_I)]),
    "tccl_double_tree_indices": (_I, [_I, _I, ctypes.POINTER(_I)]),
    "tccl_double_tree_split": (_SZ, [_SZ, _SZ]),
    "tccl_double_tree_all_reduce": (_I, [_PP, _PP, _I, _SZ, _I, _SZ, _P]),
    "tccl_double_tree_all_reduce_fused": (_I, [_PP, _PP, _I, _SZ, _I, _P]),
    "tccl_double_tree_signal_pad_bytes": (_SZ, [_I, _SZ, _I, _SZ]),
    "tccl_double_tree_all_reduce_pipelined": (_I, [_PP, _PP, _PP, _SZ, _I, _SZ, _I, _SZ,
                                                   ctypes.POINTER(PipelineCfg), _P]),
    "tccl_double_tree_all_reduce_pipelined_rank": (_I, [_PP, _P, _PP, _SZ, _I, _I, _SZ, _I, _SZ,
                                                        ctypes.POINTER(PipelineCfg), _P]),
    "tccl_signal_pad_timeouts": (_I, [_P, _SZ, ctypes.POINTER(ctypes.c_uint), _P]),
    "tccl_two_shot_all_reduce": (_I, [_PP, _PP, _PP, _SZ, _I, _SZ, _I, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_two_shot_all_reduce_rank": (_I, [_PP, _P, _PP, _SZ, _I, _I, _SZ, _I, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_all_reduce_sum_rank": (_I, [_PP, _P, _PP, _SZ, _I, _I, _SZ, _I, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_reduce_scatter_sum_rank": (_I, [_PP, _P, _PP, _SZ, _I, _I, _SZ, _I, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_all_gather_rank": (_I, [_PP, _P, _PP, _SZ, _I, _I, _SZ, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_two_shot_all_reduce_static": (_I, [_PP, _PP, _I, _SZ, _I, ctypes.POINTER(PipelineCfg), _P]),
    "tccl_timeout_flag_create": (_I, [ctypes.POINTER(ctypes.POINTER(ctypes.c_uint32))]),
    "tccl_timeout_flag_destroy": (_I, [ctypes.POINTER(ctypes.c_uint32)]),
    "tccl_symm_alloc": (_I, [_SZ, _PP]),
    "tccl_symm_free": (_I, [_P]),
    "tccl_ipc_export": (_I, [_P, ctypes.POINTER(ctypes.c_ubyte)]),
    "tccl_ipc_open": (_I, [ctypes.POINTER(ctypes.c_ubyte), _PP]),
    "tccl_ipc_close": (_I, [_P]),
    "tccl_blockwise_barrier": (_I, [_PP, _SZ, _I, _I, _I, ctypes.c_uint, ctypes.POINTER(ctypes.c_uint32), _P]),
    "tccl_double_tree_plan_create": (_I, [_PP, _PP, _I, _SZ, _I, _SZ, _PP]),
    "tccl_plan_launch": (_I, [_P, _P]),
    "tccl_plan_destroy": (_I, [_P]),
    "tccl_event_create": (_I, [_PP]),
    "tccl_event_destroy": (_I, [_P]),
    "tccl_event_record": (_I, [_P, _P]),
    "tccl_event_synchronize": (_I, [_P]),
    "tccl_event_elapsed_ms": (_I, [_P, _P, ctypes.POINTER(ctypes.c_float)]),
    "tccl_stream_synchronize": (_I, [_P]),
    "tccl_device_info": (_I, [ctypes.POINTER(_I), ctypes.POINTER(_I), ctypes.POINTER(_I), ctypes.POINTER(_SZ)]),
}

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Load the library once and set every prototype.  Raises if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP library has not been built "
            "(run `python -m tccl_amd.build`); there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.tccl_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libtccl_amd.so has ABI version {got}, this package expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(fn: str, code: int) -> None:
    if code != 0:
        raise TcclError(fn, code, load().tccl_error_string(code).decode())


def ptr_array(ptrs) -> ctypes.Array:
    """Host array of device pointers, as the entry points take their buffer tables."""
    return (ctypes.c_void_p * len(ptrs))(*ptrs)
