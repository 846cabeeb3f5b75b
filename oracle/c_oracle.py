"""ctypes binding of the C oracle (``tccl_oracle.c``).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libtccl_oracle.so")
_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> str:
    """Compile the C oracle with the Makefile beside it."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "tccl_oracle.c")
        if not os.path.exists(_SO) or (os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)):
            build()
        L = ctypes.CDLL(_SO)
        L.orc_bf16_from_f32.restype = ctypes.c_uint16
        L.orc_bf16_from_f32.argtypes = [ctypes.c_float]
        L.orc_f32_from_bf16.restype = ctypes.c_float
        L.orc_f32_from_bf16.argtypes = [ctypes.c_uint16]
        L.orc_double_tree_split.restype = ctypes.c_size_t
        L.orc_double_tree_split.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
        for name in ("orc_build_tree", "orc_build_double_tree", "orc_get_parents_and_children",
                     "orc_double_tree_all_reduce_bf16"):
            getattr(L, name).restype = ctypes.c_int
        _lib = L
    return _lib


def _ptr_array(arrs: Sequence[Optional[np.ndarray]]):
    t = ctypes.c_void_p * len(arrs)
    return t(*[(a.ctypes.data if a is not None else None) for a in arrs])


def _check(arrs: Sequence[np.ndarray], dtype) -> None:
    n = arrs[0].size
    for a in arrs:
        assert a.dtype == dtype and a.flags["C_CONTIGUOUS"] and a.size == n


def all_reduce_bf16(bufs: Sequence[np.ndarray], stepwise: bool = False) -> np.ndarray:
    _check(bufs, np.uint16)
    out = np.empty(bufs[0].size, dtype=np.uint16)
    fn = lib().orc_all_reduce_bf16_stepwise if stepwise else lib().orc_all_reduce_bf16
    fn(_ptr_array(bufs), ctypes.c_int(len(bufs)), ctypes.c_void_p(out.ctypes.data), ctypes.c_size_t(out.size))
    return out


def all_reduce_f32(bufs: Sequence[np.ndarray]) -> np.ndarray:
    _check(bufs, np.float32)
    out = np.empty(bufs[0].size, dtype=np.float32)
    lib().orc_all_reduce_f32(_ptr_array(bufs), ctypes.c_int(len(bufs)), ctypes.c_void_p(out.ctypes.data),
                             ctypes.c_size_t(out.size))
    return out


def reduce_scatter(bufs: Sequence[np.ndarray], rank: int) -> np.ndarray:
    dtype = bufs[0].dtype
    _check(bufs, dtype)
    world = len(bufs)
    out = np.empty(bufs[0].size // world, dtype=dtype)
    fn = {np.dtype(np.uint16): lib().orc_reduce_scatter_bf16,
          np.dtype(np.float32): lib().orc_reduce_scatter_f32}[np.dtype(dtype)]
    fn(_ptr_array(bufs), ctypes.c_int(world), ctypes.c_int(rank), ctypes.c_void_p(out.ctypes.data),
       ctypes.c_size_t(bufs[0].size))
    return out


def all_gather(bufs: Sequence[np.ndarray]) -> np.ndarray:
    _check(bufs, bufs[0].dtype)
    out = np.empty((len(bufs), bufs[0].size), dtype=bufs[0].dtype)
    lib().orc_all_gather(_ptr_array(bufs), ctypes.c_int(len(bufs)), ctypes.c_void_p(out.ctypes.data),
                         ctypes.c_size_t(bufs[0].nbytes))
    return out


def tree_reduce_step(own: np.ndarray, child0: Optional[np.ndarray], child1: Optional[np.ndarray]) -> np.ndarray:
    fn = {np.dtype(np.uint16): lib().orc_tree_reduce_step_bf16,
          np.dtype(np.float32): lib().orc_tree_reduce_step_f32}[np.dtype(own.dtype)]
    out = np.empty_like(own)
    p = lambda a: ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(None)
    fn(p(own), p(child0), p(child1), p(out), ctypes.c_size_t(own.size))
    return out


def tree_copy_step(src: np.ndarray, n_dst: int = 2) -> List[np.ndarray]:
    outs = [np.empty_like(src) for _ in range(n_dst)]
    p = lambda a: ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(None)
    lib().orc_tree_copy_step(p(src), p(outs[0]), p(outs[1] if n_dst > 1 else None), ctypes.c_size_t(src.nbytes))
    return outs


def build_tree(n: int) -> List[int]:
    arr = (ctypes.c_int * max(n, 1))()
    rc = lib().orc_build_tree(ctypes.c_int(n), arr)
    if rc:
        raise AssertionError("len(ranks) is not a power of 2!")
    return list(arr)[:n]


def build_double_tree(n: int) -> Tuple[List[int], List[int]]:
    a = (ctypes.c_int * max(n, 1))()
    b = (ctypes.c_int * max(n, 1))()
    rc = lib().orc_build_double_tree(ctypes.c_int(n), a, b)
    if rc:
        raise AssertionError("len(ranks) is not a power of 2!")
    return list(a)[:n], list(b)[:n]


def get_parents_and_children(n: int, rank: int) -> Tuple[int, ...]:
    out = (ctypes.c_int * 6)()
    rc = lib().orc_get_parents_and_children(ctypes.c_int(n), ctypes.c_int(rank), out)
    if rc:
        raise AssertionError(f"orc_get_parents_and_children({n}, {rank}) -> {rc}")
    return tuple(out)


def double_tree_split(numel: int, esize: int) -> int:
    return int(lib().orc_double_tree_split(numel, esize))


def double_tree_all_reduce_bf16(bufs: Sequence[np.ndarray]) -> Tuple[List[np.ndarray], List[np.ndarray]]:
    """Returns (final buffers, outputs); the inputs are copied first."""
    _check(bufs, np.uint16)
    work = [b.copy() for b in bufs]
    outs = [np.empty_like(b) for b in bufs]
    rc = lib().orc_double_tree_all_reduce_bf16(_ptr_array(work), _ptr_array(outs), ctypes.c_int(len(bufs)),
                                               ctypes.c_size_t(bufs[0].size))
    if rc:
        raise AssertionError(f"orc_double_tree_all_reduce_bf16 -> {rc}")
    return work, outs
