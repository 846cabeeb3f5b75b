"""tccl_amd -- MI355X (gfx950) data path of tccl-style collectives for W virtual ranks on
one GPU: hand-written HIP kernels behind a C ABI (``libtccl_amd.so``), with host wrappers
that keep the reference's function names.
"""
from ._lib import LaunchCfg, TcclError, load as load_library
from .collectives import (DoubleTreePlan, all_gather, all_reduce, double_tree_all_reduce, double_tree_all_reduce_world, one_shot_all_gather,
                          one_shot_all_reduce, one_shot_reduce_scatter, reduce_scatter, signal_pad_timeouts, two_shot_all_reduce,
                          two_shot_all_reduce_world)
from .symm import SymmGroup, SymmHandle, empty_world, register, rendezvous, unregister
from . import ipc, spmd, tree
from .tree import build_double_tree, build_tree, get_parents_and_children

__all__ = [
    "LaunchCfg", "TcclError", "load_library",
    "one_shot_all_reduce", "one_shot_reduce_scatter", "one_shot_all_gather", "double_tree_all_reduce",
    "double_tree_all_reduce_world", "signal_pad_timeouts", "two_shot_all_reduce_world", "DoubleTreePlan", "reduce_scatter", "all_gather", "two_shot_all_reduce", "all_reduce",
    "SymmGroup", "SymmHandle", "empty_world", "register", "rendezvous", "unregister",
    "ipc", "spmd", "tree", "build_tree", "build_double_tree", "get_parents_and_children",
]
