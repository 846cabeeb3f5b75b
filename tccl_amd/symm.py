"""Virtual ranks on one GPU: W separate device allocations that stand in for the
symmetric-memory peer buffers of the reference.

The reference allocates one peer-mappable buffer per process with
``_SymmetricMemory.empty_strided_p2p`` (triton_one_shot_all_reduce_no_128.py:116-122) and
obtains the table of all W buffer addresses with ``_SymmetricMemory.rendezvous(tensor)``
(:82), whose handle carries ``buffer_ptrs_dev``, ``rank`` and ``world_size`` (:86-91).
Here one process owns all W buffers; ``rendezvous`` finds the group a tensor belongs to in
a process-local registry keyed by the address of the tensor's storage.  Ordering between
virtual ranks is the order of work on the HIP stream; signal pads (``signal_pad_ptrs_dev``,
:87) exist only for the two kernels that signal on the device, the pipelined double tree and
the one-launch two-shot all-reduce, and are allocated when one of them is first used.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib


class SymmHandle:
    """What ``rendezvous`` returns: the view of one virtual rank onto its group."""

    def __init__(self, group: "SymmGroup", rank: int):
        self.group = group
        self.rank = rank
        self.world_size = group.world_size
        self.buffer_ptrs: Tuple[int, ...] = group.buffer_ptrs

    @property
    def buffer_ptrs_host(self) -> ctypes.Array:
        """Host array of the W device addresses, in rank order (passed by value into the
        kernel arguments by the library)."""
        return self.group.ptr_array


class SymmGroup:
    """W same-shaped buffers, one per virtual rank, each its own allocation."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        if len(tensors) < 1:
            raise ValueError("a group needs at least one buffer")
        first = tensors[0]
        for t in tensors:
            if t.shape != first.shape or t.dtype != first.dtype or t.device != first.device:
                raise ValueError("all buffers of a group must share shape, dtype and device")
            if not t.is_contiguous() or t.storage_offset() != 0:
                raise ValueError("group buffers must be whole, contiguous allocations")
        if len({t.data_ptr() for t in tensors}) != len(tensors):
            raise ValueError("every virtual rank needs its own allocation")
        self.tensors: List[torch.Tensor] = list(tensors)
        self.world_size = len(tensors)
        self.buffer_ptrs = tuple(int(t.data_ptr()) for t in tensors)
        self.ptr_array = _lib.ptr_array(self.buffer_ptrs)
        self.handles = [SymmHandle(self, r) for r in range(self.world_size)]
        # double-tree bookkeeping: outputs produced by the collective that is in progress,
        # waiting to be picked up by the ranks that have not called yet
        self.pending_outputs: Dict[int, torch.Tensor] = {}
        self._signal_pads: List[torch.Tensor] = []
        self._signal_pad_array: Optional[ctypes.Array] = None
        # a word of pinned host memory that a signalling kernel sets when one of its waits expires
        self._timeout_flag = None
        # number of the double-tree collective whose outputs `pending_outputs` holds, and torch's
        # write counters of the W buffers when it ran
        self.collective_number = 0
        self.pending_versions: Tuple[int, ...] = ()

    def signal_pads(self, nbytes: int) -> ctypes.Array:
        """Host array of W device addresses of zero-filled signal pads of at least ``nbytes``
        each, one allocation per virtual rank (the reference's per-rank signal pad).  The
        pads are created on first use and replaced by larger ones when needed; the kernels
        that use them leave them zero-filled."""
        if not self._signal_pads or self._signal_pads[0].numel() < nbytes:
            self.check_signals()            # the old pads' time-out count goes away with them
            device = self.tensors[0].device
            self._signal_pads = [torch.zeros(nbytes, dtype=torch.uint8, device=device)
                                 for _ in range(self.world_size)]
            self._signal_pad_array = _lib.ptr_array([int(p.data_ptr()) for p in self._signal_pads])
        return self._signal_pad_array

    def clear_signal_pads(self) -> None:
        """Zero the pads again (needed only after a call that reported time-outs)."""
        for p in self._signal_pads:
            p.zero_()

    @property
    def timeout_flag(self):
        """``POINTER(c_uint32)`` to this group's word of pinned host memory; the signalling
        kernels launched for the group set it to 1 when a wait expires.  Created on first use."""
        if self._timeout_flag is None:
            flag = ctypes.POINTER(ctypes.c_uint32)()
            _lib.check("tccl_timeout_flag_create", _lib.load().tccl_timeout_flag_create(ctypes.byref(flag)))
            self._timeout_flag = flag
            weakref.finalize(self, _lib.load().tccl_timeout_flag_destroy, flag)
        return self._timeout_flag

    def check_signals(self) -> None:
        """Raise ``TcclError`` (code ``TCCL_ETIMEOUT``) if a wait of a signalling kernel launched
        for this group has expired since the last check: that collective left partial results
        in the buffers and its outputs.  Costs one read of host memory, no synchronisation, so
        every collective on the group calls it first; after a time-out it waits for the device,
        zeroes the pads and the flag (the group is usable again) and raises.  Because the flag is read
        without waiting for the device, a time-out can surface one collective late: then the collective
        launched just before the raise ran on pads that still held the expired one's flags, and its
        results are suspect as well."""
        if self._timeout_flag is None or self._timeout_flag[0] == 0:
            return
        torch.cuda.synchronize(self.tensors[0].device)
        self.clear_signal_pads()
        torch.cuda.synchronize(self.tensors[0].device)
        self._timeout_flag[0] = 0
        self.pending_outputs.clear()
        raise _lib.TcclError("a signalling collective on this group", _lib.TCCL_ETIMEOUT,
                             "a wait expired (workgroups it depended on did not run in time): the buffers and "
                             "outputs of that collective hold partial results; pads cleared, the group can be "
                             "used again")

    @property
    def signal_pad_bytes(self) -> int:
        return self._signal_pads[0].numel() if self._signal_pads else 0

    def tensor(self, rank: int) -> torch.Tensor:
        return self.tensors[rank]


# storage base address -> (weak group, rank)
_registry: Dict[int, Tuple["weakref.ReferenceType[SymmGroup]", int]] = {}


def register(tensors: Sequence[torch.Tensor]) -> SymmGroup:
    """Declare that ``tensors[r]`` is virtual rank r's buffer of one symmetric allocation."""
    group = SymmGroup(tensors)
    ref = weakref.ref(group)
    for r, t in enumerate(group.tensors):
        _registry[int(t.data_ptr())] = (ref, r)
    # the buffers keep their group alive for as long as any of them is alive
    for t in group.tensors:
        t._tccl_group = group           # noqa: SLF001 -- plain attribute on the tensor object
    return group


class RemoteSymmGroup(SymmGroup):
    """A group of which this process owns one buffer; the other ranks' buffers belong to other
    processes and are known by the addresses they are mapped at here (``tccl_amd.ipc``).  Serves
    the per-rank collectives only; anything that would run other ranks' work from this process
    (the ``*_world`` functions, the in-process double tree) refuses such a group."""

    def __init__(self, own: torch.Tensor, rank: int, buffer_ptrs: Sequence[int], world=None):   # noqa: super().__init__ not called
        if not own.is_contiguous() or int(own.data_ptr()) != int(buffer_ptrs[rank]):
            raise ValueError("the own buffer must be the whole allocation at buffer_ptrs[rank]")
        self.tensors = [own]
        self.world_size = len(buffer_ptrs)
        self.buffer_ptrs = tuple(int(p) for p in buffer_ptrs)
        self.ptr_array = _lib.ptr_array(self.buffer_ptrs)
        self.handles = [SymmHandle(self, r) for r in range(self.world_size)]
        self.pending_outputs = {}
        self.pending_versions = ()
        self.collective_number = 0
        self._signal_pads = []
        self._signal_pad_array = None
        self._timeout_flag = None
        self.own_rank = rank
        # the IpcWorld the buffer came from: it owns the signal pads the per-rank kernels meet through
        self._world = weakref.ref(world) if world is not None else None

    @property
    def world(self):
        return self._world() if self._world is not None else None

    def tensor(self, rank: int) -> torch.Tensor:
        if rank != self.own_rank:
            raise RuntimeError("only the own rank's buffer is a tensor in this process")
        return self.tensors[0]


def register_remote(own: torch.Tensor, rank: int, buffer_ptrs: Sequence[int], world=None) -> RemoteSymmGroup:
    """Declare that ``own`` is rank ``rank``'s buffer of a symmetric allocation whose other buffers
    live in other processes and are mapped here at ``buffer_ptrs`` (rank order).  ``world``: the
    ``IpcWorld`` the buffers were exchanged through; with it the reference-named wrappers run the
    per-rank kernels that carry their barriers themselves."""
    group = RemoteSymmGroup(own, rank, buffer_ptrs, world)
    _registry[int(own.data_ptr())] = (weakref.ref(group), rank)
    own._tccl_group = group           # noqa: SLF001
    return group


def empty_world(world_size: int, size, dtype: torch.dtype, device="cuda") -> SymmGroup:
    """Allocate one buffer per virtual rank (each a separate ``torch.empty``) and register
    the group: the single-GPU counterpart of every rank calling ``empty_strided_p2p``."""
    if isinstance(size, int):
        size = (size,)
    tensors = [torch.empty(size, dtype=dtype, device=device) for _ in range(world_size)]
    return register(tensors)


def rendezvous(tensor: torch.Tensor) -> SymmHandle:
    """Handle of the group ``tensor`` belongs to, as seen by the rank that owns it.

    ``tensor`` may be a rank's whole buffer or a view that starts at its first element
    (the reference's benchmarks pass ``tensor[:size]``, triton_reduce_scatter.py:222); the
    element count of a collective is taken from the tensor, the addresses from the group."""
    # Fast path: a view that starts at the buffer's first element has the buffer's address.
    hit = _registry.get(tensor.data_ptr())
    group = hit[0]() if hit is not None else None
    if group is None:
        base = int(tensor.untyped_storage().data_ptr())
        hit = _registry.get(base)
        group = hit[0]() if hit is not None else None
        if group is None:
            raise RuntimeError("tensor does not belong to a registered symmetric group "
                               "(allocate it with tccl_amd.empty_world or register the buffers)")
        raise RuntimeError("a collective must be given a view that starts at the buffer's first element")
    if not tensor.is_contiguous():
        raise RuntimeError("a collective must be given a contiguous view")
    return group.handles[hit[1]]


def unregister(group: SymmGroup) -> None:
    """Forget a group (its buffers become ordinary tensors again)."""
    for t in group.tensors:
        _registry.pop(int(t.data_ptr()), None)
        if getattr(t, "_tccl_group", None) is group:
            del t._tccl_group
    group.pending_outputs.clear()
