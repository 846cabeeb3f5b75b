"""Run a per-rank program for W virtual ranks in one process.

The reference's programs are SPMD: ``torchrun`` starts one process per GPU, every process
allocates its symmetric buffer, fills it and calls the collective; the kernels' leading
``blockwise_barrier`` (triton_barrier.py:39-142) makes sure every rank's earlier writes are
visible before any rank reads its peers.  Here the W ranks are W Python threads that share
one GPU and one HIP stream.  Work enqueued on a stream runs in enqueue order, so the
device-side barrier becomes a host-side one: a rank entering a collective waits until all
W ranks have entered it, i.e. until everything they did before has been enqueued.

    def main(rank, world_size):                      # the body of a reference __main__
        tensor = spmd.empty_strided_p2p((8192,), (1,), torch.bfloat16, device).fill_(rank)
        output = tccl_amd.one_shot_all_reduce(tensor)
        assert output.eq(world_size * (world_size - 1) // 2).all().item()

    spmd.run(8, main)
"""
from __future__ import annotations

import threading
from typing import Any, Callable, Dict, List, Optional

import torch

from . import symm

_tls = threading.local()


class _World:
    def __init__(self, world_size: int):
        self.world_size = world_size
        self.barrier = threading.Barrier(world_size)
        self.lock = threading.Lock()
        # allocation number -> the tensors handed out so far for it, by rank
        self.pending: Dict[int, Dict[int, torch.Tensor]] = {}
        self.groups: List[symm.SymmGroup] = []


def current_rank() -> Optional[int]:
    """Rank of the calling thread inside ``run``; None outside."""
    return getattr(_tls, "rank", None)


def current_world_size() -> Optional[int]:
    world = getattr(_tls, "world", None)
    return world.world_size if world is not None else None


def rendezvous_barrier() -> int:
    """Wait for all W ranks; returns a number in 0..W-1 that is 0 for exactly one rank.
    Outside ``run`` it returns 0 at once."""
    world = getattr(_tls, "world", None)
    if world is None:
        return 0
    return world.barrier.wait()


class collective:
    """Brackets one collective call, from the rendezvous to the last launch.  Entering waits
    until every rank has entered -- so every rank's buffer exists (``rendezvous`` is itself
    collective in the reference) and whatever any rank enqueued before is ahead of every
    rank's kernels in the stream (the guarantee of the reference's leading device barrier).
    Leaving waits
    until every rank has enqueued its kernels, so that nothing a rank does afterwards to
    its buffer can overtake a peer's read of it (the trailing barrier the reference
    lacks).  A no-op outside ``run``."""

    def __enter__(self):
        self.first = rendezvous_barrier() == 0
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is None:
            rendezvous_barrier()
        else:
            world = getattr(_tls, "world", None)
            if world is not None:
                world.barrier.abort()
        return False


def empty_strided_p2p(size, stride=None, dtype: torch.dtype = torch.bfloat16, device="cuda",
                      group_name: Optional[str] = None) -> torch.Tensor:
    """This rank's buffer of a symmetric allocation, as
    ``_SymmetricMemory.empty_strided_p2p(size, stride, dtype, device, group_name)``
    (triton_one_shot_all_reduce_no_128.py:116-122).  Every rank must make the same sequence
    of allocations; the k-th allocations of all ranks form one group, registered when the
    last rank has made it.  Only contiguous strides are supported; ``group_name`` is
    accepted and ignored (there is one world)."""
    world = getattr(_tls, "world", None)
    if world is None:
        raise RuntimeError("empty_strided_p2p must be called from a per-rank program started with spmd.run")
    if isinstance(size, int):
        size = (size,)
    size = tuple(size)
    tensor = torch.empty(size, dtype=dtype, device=device)
    if stride is not None and tuple(stride) != tuple(tensor.stride()):
        raise ValueError("only contiguous symmetric buffers are supported")
    rank = _tls.rank
    number = _tls.allocations
    _tls.allocations += 1
    with world.lock:
        slot = world.pending.setdefault(number, {})
        slot[rank] = tensor
        if len(slot) == world.world_size:
            world.groups.append(symm.register([slot[r] for r in range(world.world_size)]))
            del world.pending[number]
    return tensor


def run(world_size: int, fn: Callable[..., Any], *args, **kwargs) -> List[Any]:
    """Call ``fn(rank, world_size, *args, **kwargs)`` once per rank, each in its own thread,
    and return the W results in rank order.  The first exception of any rank is re-raised
    (the other ranks are released from their barriers)."""
    world = _World(world_size)
    results: List[Any] = [None] * world_size
    errors: List[Optional[BaseException]] = [None] * world_size
    device = torch.cuda.current_device() if torch.cuda.is_available() else None

    def body(rank: int) -> None:
        _tls.world, _tls.rank, _tls.allocations = world, rank, 0
        try:
            if device is not None:
                torch.cuda.set_device(device)
            results[rank] = fn(rank, world_size, *args, **kwargs)
        except threading.BrokenBarrierError as e:        # another rank failed first
            errors[rank] = e
        except BaseException as e:                       # noqa: BLE001 -- re-raised below
            errors[rank] = e
            world.barrier.abort()
        finally:
            _tls.world, _tls.rank = None, None

    threads = [threading.Thread(target=body, args=(r,), name=f"tccl-rank-{r}") for r in range(world_size)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for g in world.groups:
        g.pending_outputs.clear()
    real = [e for e in errors if e is not None and not isinstance(e, threading.BrokenBarrierError)]
    if real:
        raise real[0]
    broken = [e for e in errors if e is not None]
    if broken:
        raise broken[0]
    return results
