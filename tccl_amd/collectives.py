"""The four collectives with the reference's call signatures, for virtual ranks on one GPU.

Each function takes *this rank's* buffer, finds its peers with ``rendezvous`` exactly as
the reference's wrappers do, allocates the output with torch and launches one HIP kernel
(one per tree level for the double tree) through the C ABI on torch's current stream.
Preconditions are the reference's own assertions, raised before anything is launched.

The ``*_world`` functions run a collective for every virtual rank of a group at once; two of
them (``double_tree_all_reduce_world(pipelined=True)``, ``two_shot_all_reduce_world``) use
kernels in which the ranks' workgroups signal each other through the group's signal pads.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from . import _lib, spmd
from .symm import RemoteSymmGroup, SymmGroup, rendezvous

_SUM_DTYPES = {torch.bfloat16: _lib.TCCL_BF16, torch.float32: _lib.TCCL_F32}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: Optional[torch.device] = None) -> ctypes.c_void_p:
    """torch's current stream on the tensor's device as a raw ``hipStream_t``."""
    if _raw_stream is not None and device is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))       # no Stream object is built
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _sum_dtype(tensor: torch.Tensor) -> int:
    # the reference takes bfloat16 only (triton_one_shot_all_reduce_no_128.py:73); float32
    # is summed with the same kernel and no final rounding
    assert tensor.dtype in _SUM_DTYPES, "Only bfloat16 (and float32) is supported for now."
    return _SUM_DTYPES[tensor.dtype]


def _vec_elems(tensor: torch.Tensor) -> int:
    return 16 // tensor.element_size()


def _cfg_ptr(cfg: Optional[_lib.LaunchCfg]):
    return ctypes.byref(cfg) if cfg is not None else None


def _signalling_cfg(group: SymmGroup, cfg: Optional[_lib.PipelineCfg], draw_places: bool = False) -> _lib.PipelineCfg:
    """The caller's tuning values plus the group's time-out flag, so that an expired wait is
    seen by the next ``check_signals`` without anybody synchronising."""
    full = _lib.PipelineCfg()
    if cfg is not None:
        full.workgroups, full.lag, full.spin_limit, full.tile_kib = cfg.workgroups, cfg.lag, cfg.spin_limit, cfg.tile_kib
        full.flags = cfg.flags
    if draw_places:
        full.flags |= _lib.PIPE_DRAW_PLACES
    full.timeout_flag = group.timeout_flag
    return full


def _owner_world(group: SymmGroup, what: str, needed: bool = False):
    """The ``IpcWorld`` of a group whose other buffers belong to other processes, else None.  Such a
    rank must only ever launch its own work: the per-rank kernels of its world.  ``needed``: ``what``
    would run every rank's work from this process, so a remote group without a world is refused."""
    if not isinstance(group, RemoteSymmGroup):
        return None
    world = group.world
    if world is None and needed:
        raise RuntimeError(f"{what} would run every rank's steps from this process, but the other ranks' buffers "
                           "belong to other processes: use the IpcWorld the buffer came from")
    return world


def _refuse_remote(group: SymmGroup, what: str) -> None:
    if isinstance(group, RemoteSymmGroup):
        raise RuntimeError(f"{what} runs every rank's work from one process; this group's other buffers belong to "
                           "other processes: every rank calls the per-rank collectives of its IpcWorld instead")


def _no_launch_cfg(cfg, what: str) -> None:
    if cfg is not None:
        raise ValueError(f"{what}: launch-shape overrides do not apply to the per-rank kernels of an IpcWorld")


def _check_out(out: torch.Tensor, shape, like: torch.Tensor) -> torch.Tensor:
    if tuple(out.shape) != tuple(shape) or out.dtype != like.dtype or out.device != like.device \
            or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous {like.dtype} tensor of shape {tuple(shape)} on {like.device}")
    return out


def one_shot_all_reduce(tensor: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                        cfg: Optional[_lib.LaunchCfg] = None) -> torch.Tensor:
    """Sum of all ranks' buffers over ``tensor.numel()`` elements.

    Mirrors ``one_shot_all_reduce`` (triton_one_shot_all_reduce_no_128.py:67-96): same
    dtype and alignment assertions (:73-76), a fresh ``empty_like`` output (:83) unless the
    caller passes ``out``.  The sum is accumulated in fp32 in rank order and rounded once."""
    dtype = _sum_dtype(tensor)
    # the reference's own bound for this operation is 4 elements (NUMEL_PER_THREAD, :70 and :74), whatever
    # its message says; the kernels take any element count
    assert tensor.numel() % 4 == 0, "The number of elements must be 128-bit aligned."
    lib = _lib.load()
    with spmd.collective():
        symm = rendezvous(tensor)
        symm.group.check_signals()
        output = torch.empty_like(tensor) if out is None else _check_out(out, tensor.shape, tensor)
        world = _owner_world(symm.group, "one_shot_all_reduce")
        if world is not None:          # ranks are processes: this rank's launch, barriers inside (the reference's form)
            _no_launch_cfg(cfg, "one_shot_all_reduce")
            return world.one_shot_all_reduce(tensor, out=output)
        rc = lib.tccl_all_reduce_sum_ex(symm.buffer_ptrs_host, symm.world_size, output.data_ptr(), tensor.numel(),
                                        dtype, _stream(tensor.device), _cfg_ptr(cfg))
        _lib.check("tccl_all_reduce_sum", rc)
    return output


def one_shot_reduce_scatter(tensor: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                            cfg: Optional[_lib.LaunchCfg] = None) -> torch.Tensor:
    """This rank's 1/W share of the sum: elements ``[rank*P, (rank+1)*P)``, ``P = numel // W``.

    Mirrors ``one_shot_reduce_scatter`` (triton_reduce_scatter.py:95-127); rank and world
    size come from the handle (the reference reads module globals, :103-113)."""
    dtype = _sum_dtype(tensor)
    lib = _lib.load()
    with spmd.collective():
        symm = rendezvous(tensor)
        symm.group.check_signals()
        world, rank = symm.world_size, symm.rank
        assert tensor.numel() % (_vec_elems(tensor) * world) == 0, "The number of elements must be 128-bit aligned."
        per_rank = tensor.numel() // world
        if out is None:
            output = torch.empty((per_rank,), dtype=tensor.dtype, device=tensor.device)
        else:
            output = _check_out(out, (per_rank,), tensor)
        owner = _owner_world(symm.group, "one_shot_reduce_scatter")
        if owner is not None:
            _no_launch_cfg(cfg, "one_shot_reduce_scatter")
            return owner.reduce_scatter(tensor, out=output)
        rc = lib.tccl_reduce_scatter_sum_ex(symm.buffer_ptrs_host, world, rank, output.data_ptr(), tensor.numel(),
                                            dtype, _stream(tensor.device), _cfg_ptr(cfg))
        _lib.check("tccl_reduce_scatter_sum", rc)
    return output


def one_shot_all_gather(tensor: torch.Tensor, world_size: Optional[int] = None, *,
                        out: Optional[torch.Tensor] = None, cfg: Optional[_lib.LaunchCfg] = None) -> torch.Tensor:
    """``[W, *tensor.shape]`` tensor whose row i is a copy of rank i's buffer.

    Mirrors ``one_shot_all_gather(tensor, world_size)`` (triton_all_gather.py:66-95).  Any
    dtype is copied bit for bit (the reference asserts bfloat16, :72, though its copy is
    typeless); the byte count per rank must be a multiple of 16 (:73-75)."""
    nbytes = tensor.numel() * tensor.element_size()
    assert nbytes % 16 == 0, "The number of elements must be 128-bit aligned."
    lib = _lib.load()
    with spmd.collective():
        symm = rendezvous(tensor)
        symm.group.check_signals()
        if world_size is None:
            world_size = symm.world_size
        assert world_size == symm.world_size, "world_size does not match the tensor's symmetric group"
        if out is None:
            output = torch.empty((world_size, *tensor.shape), dtype=tensor.dtype, device=tensor.device)
        else:
            output = _check_out(out, (world_size, *tensor.shape), tensor)
        owner = _owner_world(symm.group, "one_shot_all_gather")
        if owner is not None:
            _no_launch_cfg(cfg, "one_shot_all_gather")
            return owner.all_gather(tensor, out=output)
        rc = lib.tccl_all_gather_ex(symm.buffer_ptrs_host, world_size, output.data_ptr(), nbytes,
                                    _stream(tensor.device), _cfg_ptr(cfg))
        _lib.check("tccl_all_gather", rc)
    return output


def two_shot_all_reduce(tensor: torch.Tensor) -> torch.Tensor:
    """All-reduce as reduce-scatter followed by all-gather (the composition the reference's
    slides name for large messages: "can be combined with reduce-scatter for all-reduce").

    Every rank reduces its own 1/W share (one ``tccl_reduce_scatter_sum`` launch per rank),
    the shares form a symmetric group of their own, and the output is their all-gather.  The
    result is bit-identical to ``one_shot_all_reduce``: every element is still the fp32 sum
    over the ranks in rank order.  Same precondition as the reduce-scatter
    (triton_reduce_scatter.py:101-104).  On several GPUs this moves (W-1)/W of a buffer per
    direction over the links instead of (W-1) whole buffers."""
    dtype = _sum_dtype(tensor)
    lib = _lib.load()
    with spmd.collective():
        symm = rendezvous(tensor)
        symm.group.check_signals()
        world = symm.world_size
        assert tensor.numel() % (_vec_elems(tensor) * world) == 0, "The number of elements must be 128-bit aligned."
        owner = _owner_world(symm.group, "two_shot_all_reduce", needed=True)
        if owner is not None:          # in place there: every buffer ends up holding the result
            return owner.two_shot_all_reduce(tensor)
        stream = _stream(tensor.device)
        per_rank = tensor.numel() // world
        shares = torch.empty((world, per_rank), dtype=tensor.dtype, device=tensor.device)
        output = torch.empty_like(tensor)
        for r in range(world):
            rc = lib.tccl_reduce_scatter_sum(symm.buffer_ptrs_host, world, r, shares[r].data_ptr(), tensor.numel(),
                                             dtype, stream)
            _lib.check("tccl_reduce_scatter_sum", rc)
        share_ptrs = _lib.ptr_array([int(shares[r].data_ptr()) for r in range(world)])
        rc = lib.tccl_all_gather(share_ptrs, world, output.data_ptr(), per_rank * tensor.element_size(), stream)
        _lib.check("tccl_all_gather", rc)
    return output


def all_reduce(tensor: torch.Tensor, algorithm: str = "auto") -> torch.Tensor:
    """All-reduce by the named algorithm: ``"one_shot"``, ``"two_shot"``, ``"double_tree"`` or
    ``"auto"``.  With every buffer in the same HBM the one-shot kernel moves the fewest bytes
    ((W+1)N against (W+3)N for two-shot and more for the tree), so ``"auto"`` is one-shot at
    every size; the other two exist for what they model across GPUs."""
    if algorithm not in ("auto", "one_shot", "two_shot", "double_tree"):
        raise ValueError(f"unknown all-reduce algorithm {algorithm!r}")
    # (inside a per-rank thread program the group only forms at the collective's own rendezvous)
    owner = _owner_world(rendezvous(tensor).group, "all_reduce") if spmd.current_rank() is None else None
    if owner is not None:              # ranks are processes: there the three really differ, by size
        return owner.all_reduce(tensor, algorithm)
    if algorithm in ("auto", "one_shot"):
        return one_shot_all_reduce(tensor)
    if algorithm == "two_shot":
        return two_shot_all_reduce(tensor)
    if algorithm == "double_tree":
        return double_tree_all_reduce(tensor)
    raise ValueError(f"unknown all-reduce algorithm {algorithm!r}")


# Below this many bytes per buffer the level schedule is bound by its 2*log2(W) dependent
# launches (about 27 us for W=8 whatever the size) and the one-launch kernel is used instead.
FUSED_TREE_MAX_BYTES = 8 << 20


# From this many bytes per buffer the pipelined single launch beats the level schedule for
# worlds of 2, 4 and 8 (W=8 x 256 MiB: 1.58 ms against 1.74 ms; W=4: 0.67 against 0.77 ms);
# between the two thresholds the level schedule is as fast or faster.
PIPELINED_TREE_MIN_BYTES = 192 << 20


def _run_double_tree(group: SymmGroup, numel: int, dtype: int, like: torch.Tensor,
                     chunk_elems: int, fused: Optional[bool] = None, pipelined: Optional[bool] = False,
                     pipeline_cfg: Optional[_lib.PipelineCfg] = None, draw_places: bool = False) -> List[torch.Tensor]:
    group.check_signals()
    # one allocation for all W outputs (rows are 16-byte aligned: numel is whole vectors)
    stacked = torch.empty((group.world_size,) + tuple(like.shape), dtype=like.dtype, device=like.device)
    outputs = list(stacked.unbind(0))
    lib = _lib.load()
    row_bytes = like.numel() * like.element_size()
    first = int(stacked.data_ptr())
    out_ptrs = _lib.ptr_array([first + r * row_bytes for r in range(group.world_size)])
    if pipelined is None:
        pipelined = (fused is None and group.world_size in (2, 4, 8)
                     and numel * like.element_size() >= PIPELINED_TREE_MIN_BYTES)
    if pipelined:
        need = lib.tccl_double_tree_signal_pad_bytes(group.world_size, numel, dtype, chunk_elems)
        if need == 0:
            raise ValueError("the pipelined double tree needs a world of 2, 4 or 8 and whole 16-byte vectors")
        pads = group.signal_pads(need)
        rc = lib.tccl_double_tree_all_reduce_pipelined(
            group.ptr_array, out_ptrs, pads, group.signal_pad_bytes, group.world_size, numel, dtype, chunk_elems,
            ctypes.byref(_signalling_cfg(group, pipeline_cfg, draw_places)), _stream(like.device))
        _lib.check("tccl_double_tree_all_reduce_pipelined", rc)
        return outputs
    if fused is None:
        fused = group.world_size <= 8 and numel * like.element_size() <= FUSED_TREE_MAX_BYTES
    if fused:
        rc = lib.tccl_double_tree_all_reduce_fused(group.ptr_array, out_ptrs, group.world_size, numel, dtype,
                                                   _stream(like.device))
        _lib.check("tccl_double_tree_all_reduce_fused", rc)
    else:
        rc = lib.tccl_double_tree_all_reduce(group.ptr_array, out_ptrs, group.world_size, numel, dtype, chunk_elems,
                                             _stream(like.device))
        _lib.check("tccl_double_tree_all_reduce", rc)
    return outputs


def double_tree_all_reduce(tensor: torch.Tensor, *, chunk_elems: int = 0,
                           fused: Optional[bool] = None, pipelined: Optional[bool] = None) -> torch.Tensor:
    """All-reduce over two complementary binary trees, one per half of the elements.

    Mirrors ``double_tree_all_reduce`` (triton_double_tree_allreduce.py:338-370) as its
    kernel was designed (:254-335): every interior node sums its children's buffers into
    its own buffer in place, then every rank copies its parent's buffer into its own buffer
    and its output.  World size and rank come from the handle (the reference hard-codes 8
    and a global, :356).

    A collective is one call per rank.  On one GPU the first rank to call runs the node
    steps of *all* virtual ranks (the ranks' buffers are overwritten with the result, as
    in the reference's design) and gets its output; the other ranks' outputs wait in the
    group until those ranks call.  A rank calling again starts the next collective, and so
    does any rank calling after a buffer of the group has been written to with torch (refilled
    for the next collective): outputs of an older collective are never handed out then.

    ``fused``: False = one launch per tree level (the node-step kernels), True = the whole
    tree in one launch (worlds of 2, 4, 8; same values, same final memory), None = the
    one-launch kernel up to ``FUSED_TREE_MAX_BYTES`` per buffer, the level schedule above.
    ``pipelined``: True = one persistent launch in which the ranks' workgroups wait for,
    reduce and signal chunks through the group's signal pads -- the reference kernel's own
    design (worlds of 2, 4, 8); None = that launch from ``PIPELINED_TREE_MIN_BYTES`` per buffer
    when ``fused`` is None too, where it is the fastest of the three."""
    dtype = _sum_dtype(tensor)
    assert tensor.numel() % _vec_elems(tensor) == 0, "The number of elements must be 128-bit aligned."
    owner = None
    if spmd.current_rank() is None:    # (a per-rank thread program's group only forms at the collective's own rendezvous)
        owner = _owner_world(rendezvous(tensor).group, "double_tree_all_reduce", needed=True)
    if owner is not None:
        # ranks are processes: this rank's own launch of the pipelined kernel between barriers; running
        # the node steps of all ranks from here would reduce the mapped buffers W times over
        if fused or pipelined is False:
            raise ValueError("double_tree_all_reduce on an IpcWorld buffer runs the per-rank pipelined kernel only")
        return owner.double_tree_all_reduce(tensor, chunk_elems=chunk_elems)
    if spmd.current_rank() is not None:
        # W rank threads arrive together: one of them runs the collective for everybody,
        # the others pick their output up once it has been enqueued.
        with spmd.collective() as turn:
            symm = rendezvous(tensor)
            group = symm.group
            if turn.first:
                group.pending_outputs = dict(enumerate(
                    _run_double_tree(group, tensor.numel(), dtype, tensor, chunk_elems, fused, pipelined)))
        return group.pending_outputs[symm.rank]
    symm = rendezvous(tensor)
    group = symm.group
    # The outputs of the collective in progress wait in the group for the ranks that have not
    # called yet.  They are handed out only while every buffer is as that collective left it:
    # torch counts in-place writes per tensor, so a buffer that has been refilled since (the
    # next collective's input) makes the cache stale and this call starts a new collective, and
    # so does a rank that already has its output and calls again.
    versions = tuple(t._version for t in group.tensors)                 # noqa: SLF001
    pending = group.pending_outputs.pop(symm.rank, None)
    if pending is not None and pending.shape == tensor.shape and versions == group.pending_versions:
        return pending
    outputs = _run_double_tree(group, tensor.numel(), dtype, tensor, chunk_elems, fused, pipelined)
    group.collective_number += 1
    group.pending_outputs = {r: o for r, o in enumerate(outputs) if r != symm.rank}
    group.pending_versions = versions
    return outputs[symm.rank]


def double_tree_all_reduce_world(group: SymmGroup, numel: Optional[int] = None, *,
                                 chunk_elems: int = 0, fused: Optional[bool] = None, pipelined: Optional[bool] = None,
                                 pipeline_cfg: Optional[_lib.PipelineCfg] = None,
                                 draw_places: bool = False) -> List[torch.Tensor]:
    """One whole collective for every virtual rank of ``group``; returns the W outputs.

    ``pipelined``: one persistent launch in which the ranks' workgroups hand chunks to each
    other through the group's signal pads (the reference kernel's wait/reduce/send design,
    triton_double_tree_allreduce.py:254-335) instead of one launch per tree level.  Should a
    wait of that launch expire (it cannot hang: every wait is bounded), the next collective on
    the group -- or ``group.check_signals()`` -- raises ``TcclError``.
    ``draw_places``: the launch's workgroups draw their places (rank, index) when they start to
    run instead of taking them from their hardware index; the launch then makes progress
    however few of its workgroups are resident at once (for use beside other kernels on the
    same GPU), at up to 15 % of the speed on large inputs."""
    _refuse_remote(group, "double_tree_all_reduce_world")
    like = group.tensors[0].reshape(-1)
    if numel is not None:
        like = like[:numel]
    dtype = _sum_dtype(like)
    assert like.numel() % _vec_elems(like) == 0, "The number of elements must be 128-bit aligned."
    group.pending_outputs.clear()
    return _run_double_tree(group, like.numel(), dtype, like, chunk_elems, fused, pipelined, pipeline_cfg, draw_places)


def signal_pad_timeouts(group: SymmGroup) -> int:
    """Waits of signalling kernels (pipelined double tree, one-launch two-shot) on ``group``
    that expired since its pads were last cleared; 0 after correct runs.  Synchronises the
    current stream."""
    if group.signal_pad_bytes == 0:
        return 0
    count = ctypes.c_uint(0)
    pads = group.signal_pads(group.signal_pad_bytes)
    rc = _lib.load().tccl_signal_pad_timeouts(pads[0], group.signal_pad_bytes, ctypes.byref(count),
                                              _stream(group.tensors[0].device))
    _lib.check("tccl_signal_pad_timeouts", rc)
    return int(count.value)


# Signal pad size the one-launch two-shot asks for: room for 1024 workgroups per rank.
TWO_SHOT_PAD_BYTES = 4 * (8 * 1024 + 288)


def two_shot_all_reduce_world(group: SymmGroup, numel: Optional[int] = None, *, with_outputs: bool = True,
                              pipeline_cfg: Optional[_lib.PipelineCfg] = None,
                              draw_places: bool = False) -> Optional[List[torch.Tensor]]:
    """Two-shot all-reduce of every virtual rank of ``group`` in one launch, in place: every
    buffer ends up holding the sum (bit-identical to ``one_shot_all_reduce``); with
    ``with_outputs`` the W results are also written to fresh tensors, which are returned.
    Shot 1 reduces each rank's share, the reference's blockwise barrier
    (triton_barrier.py:39-142) separates it from shot 2, which gathers the other shares.
    ``draw_places``: as for ``double_tree_all_reduce_world``."""
    _refuse_remote(group, "two_shot_all_reduce_world")
    like = group.tensors[0].reshape(-1)
    if numel is not None:
        like = like[:numel]
    dtype = _sum_dtype(like)
    world = group.world_size
    assert like.numel() % (_vec_elems(like) * world) == 0, "The number of elements must be 128-bit aligned."
    lib = _lib.load()
    outputs = None
    out_ptrs = None
    if with_outputs:
        stacked = torch.empty((world, like.numel()), dtype=like.dtype, device=like.device)
        outputs = list(stacked.unbind(0))
        out_ptrs = _lib.ptr_array([int(o.data_ptr()) for o in outputs])
    group.check_signals()
    pads = group.signal_pads(TWO_SHOT_PAD_BYTES)
    rc = lib.tccl_two_shot_all_reduce(group.ptr_array, out_ptrs, pads, group.signal_pad_bytes, world, like.numel(),
                                      dtype, ctypes.byref(_signalling_cfg(group, pipeline_cfg, draw_places)),
                                      _stream(like.device))
    _lib.check("tccl_two_shot_all_reduce", rc)
    return outputs


class DoubleTreePlan:
    """The whole double-tree all-reduce of a group recorded into a HIP graph.

    ``run()`` replays it with a single launch on torch's current stream and returns the W
    outputs (the same tensors every time; the group's buffers are overwritten with the
    result, as by ``double_tree_all_reduce``).  Worth it when the collective is repeated on
    the same buffers and is small enough to be bound by its launches."""

    def __init__(self, group: SymmGroup, numel: Optional[int] = None, *, chunk_elems: int = 0):
        _refuse_remote(group, "DoubleTreePlan")
        like = group.tensors[0].reshape(-1)
        if numel is not None:
            like = like[:numel]
        dtype = _sum_dtype(like)
        assert like.numel() % _vec_elems(like) == 0, "The number of elements must be 128-bit aligned."
        self.group = group
        self.outputs = [torch.empty_like(like) for _ in range(group.world_size)]
        self._out_ptrs = _lib.ptr_array([int(o.data_ptr()) for o in self.outputs])
        self._plan = ctypes.c_void_p()
        lib = _lib.load()
        rc = lib.tccl_double_tree_plan_create(group.ptr_array, self._out_ptrs, group.world_size, like.numel(), dtype,
                                              chunk_elems, ctypes.byref(self._plan))
        _lib.check("tccl_double_tree_plan_create", rc)

    def run(self) -> List[torch.Tensor]:
        if not self._plan:
            raise RuntimeError("plan has been closed")
        _lib.check("tccl_plan_launch", _lib.load().tccl_plan_launch(self._plan, _stream(self.outputs[0].device)))
        return self.outputs

    def close(self) -> None:
        if self._plan:
            _lib.load().tccl_plan_destroy(self._plan)
            self._plan = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# short names for the same functions
reduce_scatter = one_shot_reduce_scatter
all_gather = one_shot_all_gather
