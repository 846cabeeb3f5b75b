"""Double binary tree index math with the reference's function names and results.

Mirrors ``tree.py`` of the reference (``build_tree`` tree.py:5-31, ``build_double_tree``
tree.py:34-91, ``get_parents_and_children`` tree.py:93-148); the numbers come from the
closed forms in the C library (``tccl_double_tree_arrays`` / ``tccl_double_tree_indices``),
not from building and searching lists.
"""
from __future__ import annotations

import ctypes
from functools import lru_cache
from typing import List, Tuple

from . import _lib


def _arrays(n: int) -> Tuple[List[int], List[int]]:
    a = (ctypes.c_int * n)()
    b = (ctypes.c_int * n)()
    _lib.check("tccl_double_tree_arrays", _lib.load().tccl_double_tree_arrays(n, a, b))
    return list(a), list(b)


def build_tree(N: int) -> List[int]:
    """Heap-ordered array of the first tree: position 0 is the extra node 0 whose only
    child is position 1; otherwise the children of position i are 2i and 2i+1."""
    assert N >= 1 and (N & (N - 1)) == 0, "len(ranks) is not a power of 2!"
    if N == 1:
        return [0]                      # what tree.py:13-31 yields for a single rank
    return _arrays(N)[0]


@lru_cache
def build_double_tree(N: int) -> Tuple[List[int], List[int]]:
    """Both arrays; the second is the first with every label lowered by one (mod N)."""
    assert N >= 2 and (N & (N - 1)) == 0, "len(ranks) is not a power of 2!"
    return _arrays(N)


def get_parents_and_children(N: int, rank: int) -> Tuple[int, int, int, int, int, int]:
    """``(a_parent, a_child0, a_child1, b_parent, b_child0, b_child1)``, -1 = none.

    A subroot has only its left child set.  Error behaviour follows the reference: a
    world that is not a power of two fails the assertion of tree.py:11, a single-rank
    world raises IndexError (tree.py:135) and a rank outside the world raises ValueError
    (``list.index`` at tree.py:131)."""
    assert N >= 1 and (N & (N - 1)) == 0, "len(ranks) is not a power of 2!"
    if not 0 <= rank < N:
        raise ValueError(f"{rank} is not in list")
    if N == 1:
        raise IndexError("list index out of range")
    out = (ctypes.c_int * 6)()
    _lib.check("tccl_double_tree_indices", _lib.load().tccl_double_tree_indices(N, rank, out))
    return tuple(out)
